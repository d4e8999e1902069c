// Layout-agnostic kernels: the one-work-item-per-output convolution (serves every
// format/precision combination the path accepts, e.g. plain bfyx int8 topologies),
// the raw-accumulator probe and the reorder.
#include "epilogue.h"
#include "kernels.h"

namespace chip {

struct RefConvArgs {
    Pitch in, out, eltw;
    int B, IFM, IH, IW, OFM, OH, OW, FY, FX;
    int sy, sx, dy, dx, py, px, groups;
    int esy, esx;
    int in_dt, w_dt;
    Epilogue epi;
};

template <typename InT>
__device__ __forceinline__ int dot_int(const RefConvArgs& a, const InT* __restrict__ in, const int8_t* __restrict__ w,
                                       int b, int f, int y, int x)
{
    const int ifm_g = a.IFM / a.groups, ofm_g = a.OFM / a.groups;
    const int g = f / ofm_g;
    const int iy0 = y * a.sy - a.py, ix0 = x * a.sx - a.px;
    int acc = 0;
    for (int k = 0; k < ifm_g; ++k) {
        const int c = g * ifm_g + k;
        const int8_t* wk = w + ((int64_t)f * ifm_g + k) * a.FY * a.FX;
        for (int j = 0; j < a.FY; ++j) {
            const int iy = iy0 + j * a.dy;
            if (iy < 0 || iy >= a.IH) continue;
            for (int i = 0; i < a.FX; ++i) {
                const int ix = ix0 + i * a.dx;
                if (ix < 0 || ix >= a.IW) continue;
                acc += (int)in[a.in.at(b, c, iy, ix)] * (int)wk[j * a.FX + i];
            }
        }
    }
    return acc;
}

// float data: accumulate in float in the reference's k -> j -> i order; under quantisation the
// operands are truncated to int first (fused_conv_eltwise_gpu_ref.cl:21,140)
__device__ __forceinline__ void dot_f32(const RefConvArgs& a, const float* __restrict__ in, const float* __restrict__ w,
                                        int b, int f, int y, int x, float& facc, int& iacc)
{
    const int ifm_g = a.IFM / a.groups, ofm_g = a.OFM / a.groups;
    const int g = f / ofm_g;
    const int iy0 = y * a.sy - a.py, ix0 = x * a.sx - a.px;
    facc = 0.f;
    iacc = 0;
    for (int k = 0; k < ifm_g; ++k) {
        const int c = g * ifm_g + k;
        const float* wk = w + ((int64_t)f * ifm_g + k) * a.FY * a.FX;
        for (int j = 0; j < a.FY; ++j) {
            const int iy = iy0 + j * a.dy;
            if (iy < 0 || iy >= a.IH) continue;
            for (int i = 0; i < a.FX; ++i) {
                const int ix = ix0 + i * a.dx;
                if (ix < 0 || ix >= a.IW) continue;
                const float v = in[a.in.at(b, c, iy, ix)], wv = wk[j * a.FX + i];
                facc = facc + v * wv;
                iacc += (int)v * (int)wv;
            }
        }
    }
}

__global__ void __launch_bounds__(256) conv_ref_kernel(RefConvArgs a, const void* __restrict__ in,
                                                       const void* __restrict__ w, const void* __restrict__ eltw,
                                                       void* __restrict__ out, int* __restrict__ acc_out)
{
    const int64_t total = (int64_t)a.B * a.OFM * a.OH * a.OW;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int x = (int)(idx % a.OW);
    int64_t r = idx / a.OW;
    const int y = (int)(r % a.OH);
    r /= a.OH;
    const int f = (int)(r % a.OFM);
    const int b = (int)(r / a.OFM);

    int acc = 0;
    float facc = 0.f;
    if (a.in_dt == CLDNN_HIP_U8) acc = dot_int(a, (const uint8_t*)in, (const int8_t*)w, b, f, y, x);
    else if (a.in_dt == CLDNN_HIP_S8) acc = dot_int(a, (const int8_t*)in, (const int8_t*)w, b, f, y, x);
    else dot_f32(a, (const float*)in, (const float*)w, b, f, y, x, facc, acc);

    if (acc_out) {
        acc_out[idx] = acc;
        return;
    }
    const Epilogue& e = a.epi;
    const int64_t oi = a.out.at(b, f, y, x);
    float ev = 0.f;
    if (e.fused) ev = load_as_float(eltw, e.eltw_dt, a.eltw.at(b, f, y * a.esy, x * a.esx));

    if (e.mode == MODE_NAT) {
        EpiOut o;
        if (a.in_dt == CLDNN_HIP_F32) {
            float v = facc;
            if (e.bias) v = v + load_as_float(e.bias, e.bias_dt, f);
            v = act_f(e.act, e.act_m, e.act_n, v);
            if (e.fused) {
                if (e.ncs_on) ev = ev * e.ncs;
                v = act_f(e.eltw_act, e.eltw_m, e.eltw_n, v + ev);
                if (e.eltw_calib) v = v * e.eltw_calib[f];
                if (e.out_dt != CLDNN_HIP_F32) v = round_sel(v, e.round_even);
            }
            o = finish(e, v);
        } else {
            // unquantised int8: accumulator, bias and activation live in the input's char type
            signed char c = (signed char)acc;
            if (e.bias) c = (signed char)(c + (signed char)(int)load_as_float(e.bias, e.bias_dt, f));
            int ci = c;
            if (e.act == CLDNN_HIP_ACT_RELU) ci = ci > 0 ? ci : 0;
            else if (e.act == CLDNN_HIP_ACT_RELU_SLOPE) {
                signed char s = (signed char)(int)e.act_m;
                ci = (signed char)((ci > 0 ? ci : 0) + s * (ci < 0 ? ci : 0));
            }
            o.i = ci;
            o.f = (float)ci;
            if (e.out_dt == CLDNN_HIP_U8) o.i = ci < 0 ? 0 : ci;
        }
        store_out(out, e.out_dt, oi, o);
        return;
    }
    store_out(out, e.out_dt, oi, epilogue_generic(e, acc, f, ev));
}

// ------------------------------------------------------------------------------------------ reorder
struct ReorderArgs {
    Pitch src, dst;
    int B, F, Y, X;
    int src_dt, dst_dt;
    int dst_fs_fill;  // features physically present in dst beyond F (zero-filled), blocked formats only
};

__device__ __forceinline__ float f32_to_int_round(float v) { return round_half_away(v); }

__global__ void __launch_bounds__(256) reorder_kernel(ReorderArgs a, const void* __restrict__ src, void* __restrict__ dst)
{
    // iterate in DESTINATION memory order of the innermost two logical axes so stores coalesce
    const int Fd = a.F + a.dst_fs_fill;
    const int64_t total = (int64_t)a.B * Fd * a.Y * a.X;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int b, f, y, x;
    if (a.dst.fsv > 1) {  // [..][y][x][fsv]
        const int fsv = a.dst.fsv;
        const int fi = (int)(idx % fsv);
        int64_t r = idx / fsv;
        x = (int)(r % a.X);
        r /= a.X;
        y = (int)(r % a.Y);
        r /= a.Y;
        const int nfs = Fd / fsv;
        if (a.dst.pb < a.dst.pf) {  // fs outermost
            b = (int)(r % a.B);
            f = (int)(r / a.B) * fsv + fi;
        } else {
            f = (int)(r % nfs) * fsv + fi;
            b = (int)(r / nfs);
        }
    } else if (a.dst.px == 1) {  // bfyx
        x = (int)(idx % a.X);
        int64_t r = idx / a.X;
        y = (int)(r % a.Y);
        r /= a.Y;
        f = (int)(r % Fd);
        b = (int)(r / Fd);
    } else if (a.dst.pf == 1) {  // byxf
        f = (int)(idx % Fd);
        int64_t r = idx / Fd;
        x = (int)(r % a.X);
        r /= a.X;
        y = (int)(r % a.Y);
        b = (int)(r / a.Y);
    } else {  // yxfb
        b = (int)(idx % a.B);
        int64_t r = idx / a.B;
        f = (int)(r % Fd);
        r /= Fd;
        x = (int)(r % a.X);
        y = (int)(r / a.X);
    }
    const int64_t di = a.dst.at(b, f, y, x);
    if (f >= a.F) {  // feature padding of a blocked destination
        if (a.dst_dt == CLDNN_HIP_F32) ((float*)dst)[di] = 0.f;
        else if (a.dst_dt == CLDNN_HIP_I32) ((int*)dst)[di] = 0;
        else ((uint8_t*)dst)[di] = 0;
        return;
    }
    const int64_t si = a.src.at(b, f, y, x);
    if (a.src_dt == a.dst_dt) {
        if (a.src_dt == CLDNN_HIP_F32 || a.src_dt == CLDNN_HIP_I32) ((uint32_t*)dst)[di] = ((const uint32_t*)src)[si];
        else ((uint8_t*)dst)[di] = ((const uint8_t*)src)[si];
        return;
    }
    const bool src_fp = a.src_dt == CLDNN_HIP_F32;
    float fv = 0.f;
    int iv = 0;
    switch (a.src_dt) {
    case CLDNN_HIP_S8: iv = ((const int8_t*)src)[si]; break;
    case CLDNN_HIP_U8: iv = ((const uint8_t*)src)[si]; break;
    case CLDNN_HIP_I32: iv = ((const int*)src)[si]; break;
    default: fv = ((const float*)src)[si]; break;
    }
    switch (a.dst_dt) {
    case CLDNN_HIP_F32: ((float*)dst)[di] = src_fp ? fv : (float)iv; break;
    case CLDNN_HIP_I32: ((int*)dst)[di] = src_fp ? (int)f32_to_int_round(fv) : iv; break;
    case CLDNN_HIP_S8: {
        int v = src_fp ? sat_s8(f32_to_int_round(fv)) : (iv < -128 ? -128 : (iv > 127 ? 127 : iv));
        ((int8_t*)dst)[di] = (int8_t)v;
        break;
    }
    default: {
        int v = src_fp ? sat_u8(f32_to_int_round(fv)) : (iv < 0 ? 0 : (iv > 255 ? 255 : iv));
        ((uint8_t*)dst)[di] = (uint8_t)v;
        break;
    }
    }
}

// ------------------------------------------------------------------------------------------ host launchers
void launch_conv_ref(hipStream_t s, const ConvProblem& p, const Epilogue& epi, const void* in, const void* w,
                     const void* eltw, void* out, int* acc_out)
{
    RefConvArgs a{};
    a.in = p.in_p, a.out = p.out_p, a.eltw = p.eltw_p;
    a.B = p.B, a.IFM = p.IFM, a.IH = p.IH, a.IW = p.IW, a.OFM = p.OFM, a.OH = p.OH, a.OW = p.OW;
    a.FY = p.FY, a.FX = p.FX, a.sy = p.sy, a.sx = p.sx, a.dy = p.dy, a.dx = p.dx, a.py = p.py, a.px = p.px;
    a.groups = p.groups, a.esy = p.esy, a.esx = p.esx, a.in_dt = p.in_dt, a.w_dt = p.w_dt;
    a.epi = epi;
    const int64_t total = (int64_t)a.B * a.OFM * a.OH * a.OW;
    const int64_t blocks = (total + 255) / 256;
    CHIP_REQUIRE(blocks < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "output too large for the reference kernel grid");
    hipLaunchKernelGGL(conv_ref_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, in, w, eltw, out, acc_out);
    CHIP_CHECK(hipGetLastError());
}

void launch_reorder(hipStream_t s, const cldnn_hip_tensor& st, const void* src, const cldnn_hip_tensor& dt, void* dst)
{
    CHIP_REQUIRE(st.b == dt.b && st.f == dt.f && st.y == dt.y && st.x == dt.x, CLDNN_HIP_DIMENSION_MISMATCH,
                 "reorder: logical sizes differ");
    ReorderArgs a{};
    a.src = make_pitch(st), a.dst = make_pitch(dt);
    a.B = st.b, a.F = st.f, a.Y = st.y, a.X = st.x;
    a.src_dt = st.dtype, a.dst_dt = dt.dtype;
    a.dst_fs_fill = a.dst.fsv > 1 ? a.dst.fs_count * a.dst.fsv - dt.f : 0;
    const int64_t total = (int64_t)a.B * (a.F + a.dst_fs_fill) * a.Y * a.X;
    const int64_t blocks = (total + 255) / 256;
    CHIP_REQUIRE(blocks < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "tensor too large for the reorder grid");
    hipLaunchKernelGGL(reorder_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, src, dst);
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
