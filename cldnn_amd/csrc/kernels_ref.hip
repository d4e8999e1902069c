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

// float -> integer in a reorder is the reference's convert_char / convert_uchar / convert_int: towards zero
// (kernel_selector/core/common/jitter.cpp:483,497,511; cl_kernels/reorder_data.cl:142).  Values outside the target
// range, which OpenCL leaves undefined, saturate here.
__device__ __forceinline__ float f32_to_int_round(float v) { return truncf(v); }

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

// ------------------------------------------------------------------------------------------ concatenation
// One input of a concatenation copied to its place in the output: one work-item per element, any two layouts of one
// element type (reference kernel_selector/core/cl_kernels/concatenation_gpu_ref.cl:18-46, one kernel per input with
// the offset along the concatenation axis as its argument).
struct CopyRegionArgs {
    Pitch src, dst;
    int B, F, Y, X;      // logical size of the source
    int ob, of, oy, ox;  // where its element (0, 0, 0, 0) lies in the destination
    int wide;            // 4-byte elements
};

__global__ void __launch_bounds__(256) copy_region_kernel(CopyRegionArgs a, const void* __restrict__ src, void* __restrict__ dst)
{
    const int64_t total = (int64_t)a.B * a.F * a.Y * a.X;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int b, f, y, x;
    if (a.dst.fsv > 1 || a.dst.pf == 1) {  // features innermost in the destination
        f = (int)(idx % a.F);
        int64_t r = idx / a.F;
        x = (int)(r % a.X);
        r /= a.X;
        y = (int)(r % a.Y);
        b = (int)(r / a.Y);
    } else {
        x = (int)(idx % a.X);
        int64_t r = idx / a.X;
        y = (int)(r % a.Y);
        r /= a.Y;
        f = (int)(r % a.F);
        b = (int)(r / a.F);
    }
    const int64_t si = a.src.at(b, f, y, x), di = a.dst.at(b + a.ob, f + a.of, y + a.oy, x + a.ox);
    if (a.wide) ((uint32_t*)dst)[di] = ((const uint32_t*)src)[si];
    else ((uint8_t*)dst)[di] = ((const uint8_t*)src)[si];
}

void launch_copy_region(hipStream_t s, const cldnn_hip_tensor& st, const void* src, const cldnn_hip_tensor& dt, void* dst, int ob, int of,
                        int oy, int ox)
{
    CHIP_REQUIRE(dtype_size(st.dtype) == dtype_size(dt.dtype), CLDNN_HIP_INVALID_ARG, "concatenation: element sizes differ");
    CHIP_REQUIRE(ob >= 0 && of >= 0 && oy >= 0 && ox >= 0 && ob + st.b <= dt.b && of + st.f <= dt.f && oy + st.y <= dt.y && ox + st.x <= dt.x,
                 CLDNN_HIP_DIMENSION_MISMATCH, "concatenation: the input does not fit into the output at this offset");
    CopyRegionArgs a{};
    a.src = make_pitch(st), a.dst = make_pitch(dt);
    a.B = st.b, a.F = st.f, a.Y = st.y, a.X = st.x;
    a.ob = ob, a.of = of, a.oy = oy, a.ox = ox;
    a.wide = dtype_size(st.dtype) == 4;
    const int64_t total = (int64_t)a.B * a.F * a.Y * a.X;
    if (total == 0) return;
    const int64_t blocks = (total + 255) / 256;
    CHIP_REQUIRE(blocks < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "tensor too large for the copy grid");
    hipLaunchKernelGGL(copy_region_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, src, dst);
    CHIP_CHECK(hipGetLastError());
}

// ------------------------------------------------------------------------------------------ eltwise / activation
// Stand-alone forms of what the convolution epilogue fuses (reference
// kernel_selector/core/cl_kernels/generic_eltwise_ref.cl:311-328 for the sum, activation_ref.cl for the
// activation).  One work-item per logical element, any layout.
struct PointwiseArgs {
    Pitch a, b, dst;
    int B, F, Y, X;
    int a_dt, b_dt, dst_dt;
    int has_b;        // 0: activation only
    int quantized;    // int sum, then round(sum * factor), saturate to char, then activation
    const float* calib;
    float oqf;
    int act;
    float m, n;
};

__global__ void __launch_bounds__(256) pointwise_kernel(PointwiseArgs p, const void* __restrict__ a, const void* __restrict__ b,
                                                        void* __restrict__ dst)
{
    const int64_t total = (int64_t)p.B * p.F * p.Y * p.X;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    // destination memory order for the innermost axis keeps the stores coalesced
    int bi, f, y, x;
    if (p.dst.fsv > 1 || p.dst.pf == 1) {
        f = (int)(idx % p.F);
        int64_t r = idx / p.F;
        x = (int)(r % p.X);
        r /= p.X;
        y = (int)(r % p.Y);
        bi = (int)(r / p.Y);
    } else {
        x = (int)(idx % p.X);
        int64_t r = idx / p.X;
        y = (int)(r % p.Y);
        r /= p.Y;
        f = (int)(r % p.F);
        bi = (int)(r / p.F);
    }
    const int64_t ai = p.a.at(bi, f, y, x), di = p.dst.at(bi, f, y, x);
    const bool fp = p.a_dt == CLDNN_HIP_F32;
    EpiOut o;
    if (fp) {
        float v = ((const float*)a)[ai];
        if (p.has_b) v = v + load_as_float(b, p.b_dt, p.b.at(bi, f, y, x));
        v = act_f(p.act, p.m, p.n, v);
        o.f = v;
        o.i = p.dst_dt == CLDNN_HIP_U8 ? sat_u8(round_half_away(v)) : sat_s8(round_half_away(v));
    } else {
        int v = p.a_dt == CLDNN_HIP_U8 ? (int)((const uint8_t*)a)[ai] : (int)((const int8_t*)a)[ai];
        if (p.has_b) v += (int)load_as_float(b, p.b_dt, p.b.at(bi, f, y, x));
        if (p.quantized) {
            const float s = p.calib ? p.calib[f] : p.oqf;
            v = (int)round_half_away((float)v * s);
            v = v < -128 ? -128 : (v > 127 ? 127 : v);  // convert_char_sat
        } else if (p.a_dt == CLDNN_HIP_S8) {
            v = (int)(signed char)v;  // arithmetic in the unit type wraps
        } else {
            v = (int)(unsigned char)v;
        }
        v = act_i(p.act, p.m, p.n, v);
        o.i = v;
        o.f = (float)v;
        if (p.dst_dt == CLDNN_HIP_S8) o.i = v < -128 ? -128 : (v > 127 ? 127 : v);
        else if (p.dst_dt == CLDNN_HIP_U8) o.i = v < 0 ? 0 : (v > 255 ? 255 : v);
    }
    store_out(dst, p.dst_dt, di, o);
}

void launch_pointwise(hipStream_t s, const cldnn_hip_tensor& at, const void* a, const cldnn_hip_tensor* bt, const void* b,
                      const cldnn_hip_tensor& dt, void* dst, int quantized, const float* calib, float oqf, int act, float m,
                      float n)
{
    CHIP_REQUIRE(at.b == dt.b && at.f == dt.f && at.y == dt.y && at.x == dt.x, CLDNN_HIP_DIMENSION_MISMATCH,
                 "pointwise: logical sizes differ");
    PointwiseArgs p{};
    p.a = make_pitch(at), p.dst = make_pitch(dt);
    p.B = at.b, p.F = at.f, p.Y = at.y, p.X = at.x;
    p.a_dt = at.dtype, p.dst_dt = dt.dtype, p.has_b = bt != nullptr;
    if (bt) {
        CHIP_REQUIRE(bt->b == at.b && bt->f == at.f && bt->y == at.y && bt->x == at.x, CLDNN_HIP_DIMENSION_MISMATCH,
                     "eltwise: input sizes differ");
        p.b = make_pitch(*bt), p.b_dt = bt->dtype;
    }
    p.quantized = quantized, p.calib = calib, p.oqf = oqf, p.act = act, p.m = m, p.n = n;
    const int64_t total = (int64_t)p.B * p.F * p.Y * p.X;
    const int64_t blocks = (total + 255) / 256;
    CHIP_REQUIRE(blocks < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "tensor too large for the pointwise grid");
    hipLaunchKernelGGL(pointwise_kernel, dim3((unsigned)blocks), dim3(256), 0, s, p, a, b, dst);
    CHIP_CHECK(hipGetLastError());
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

// 8-bit data from a plain layout into a blocked one (the step in front of the first convolution of a network): one
// work-item gathers the FSV features of one pixel and writes them with one FSV-byte store; consecutive work-items
// take consecutive pixels of a row, so the stores of a wavefront are contiguous and the loads run along the rows of
// FSV feature planes.  Feature padding is written as zero, spatial padding is left untouched.
template <int FSV>
__global__ void __launch_bounds__(256) reorder_to_blocked_kernel(ReorderArgs a, const uint8_t* __restrict__ src, uint8_t* __restrict__ dst)
{
    const int slices = (a.F + FSV - 1) / FSV;
    const int64_t total = (int64_t)slices * a.B * a.Y * a.X;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int x = (int)(idx % a.X);
    int64_t r = idx / a.X;
    const int y = (int)(r % a.Y);
    r /= a.Y;
    const int fs = (int)(r % slices), b = (int)(r / slices);
    unsigned w[FSV / 4];
#pragma unroll
    for (int i = 0; i < FSV / 4; ++i) w[i] = 0;
    const int64_t s0 = a.src.at(b, fs * FSV, y, x);
#pragma unroll
    for (int c = 0; c < FSV; ++c)
        if (fs * FSV + c < a.F) w[c >> 2] |= (unsigned)src[s0 + (int64_t)c * a.src.pf] << (8 * (c & 3));
    uint8_t* o = dst + a.dst.at(b, fs * FSV, y, x);
    if constexpr (FSV == 4) *reinterpret_cast<unsigned*>(o) = w[0];
    else *reinterpret_cast<uint4*>(o) = make_uint4(w[0], w[1], w[2], w[3]);
}

// The same for FSV = 4 when rows are whole dwords (X % 4 == 0, 4-byte aligned planes): one lane = 4 consecutive pixels
// of a row: one dword load per feature plane, a 4x4 byte transpose in registers, one 16-byte store.
template <bool ALIGNED16>
__global__ void __launch_bounds__(256) reorder_to_fsv4_x4_kernel(ReorderArgs a, const uint8_t* __restrict__ src, uint8_t* __restrict__ dst)
{
    const int slices = (a.F + 3) / 4, xq = a.X / 4;
    const unsigned total = (unsigned)slices * a.B * a.Y * xq;
    const unsigned idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int x = (int)(idx % xq) * 4;
    unsigned r = idx / xq;
    const int y = (int)(r % a.Y);
    r /= a.Y;
    const int fs = (int)(r % slices), b = (int)(r / slices);
    const int64_t s0 = a.src.at(b, fs * 4, y, x);
    unsigned p[4] = {0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < 4; ++c)
        if (fs * 4 + c < a.F) p[c] = *reinterpret_cast<const unsigned*>(src + s0 + (int64_t)c * a.src.pf);
    unsigned w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)  // pixel i: byte i of every plane
        w[i] = ((p[0] >> (8 * i)) & 255u) | (((p[1] >> (8 * i)) & 255u) << 8) | (((p[2] >> (8 * i)) & 255u) << 16)
               | (((p[3] >> (8 * i)) & 255u) << 24);
    uint8_t* o = dst + a.dst.at(b, fs * 4, y, x);
    if constexpr (ALIGNED16) {
        *reinterpret_cast<uint4*>(o) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {  // a left border whose width is not a multiple of 4 pixels
#pragma unroll
        for (int i = 0; i < 4; ++i) reinterpret_cast<unsigned*>(o)[i] = w[i];
    }
}

void launch_reorder(hipStream_t s, const cldnn_hip_tensor& st, const void* src, const cldnn_hip_tensor& dt, void* dst)
{
    CHIP_REQUIRE(st.b == dt.b && st.f == dt.f && st.y == dt.y && st.x == dt.x, CLDNN_HIP_DIMENSION_MISMATCH,
                 "reorder: logical sizes differ");
    ReorderArgs a{};
    a.src = make_pitch(st), a.dst = make_pitch(dt);
    a.B = st.b, a.F = st.f, a.Y = st.y, a.X = st.x;
    a.src_dt = st.dtype, a.dst_dt = dt.dtype;
    const bool bytes = (st.dtype == CLDNN_HIP_S8 || st.dtype == CLDNN_HIP_U8) && st.dtype == dt.dtype;
    if (bytes && a.src.fsv == 1 && (a.dst.fsv == 4 || a.dst.fsv == 16)) {
        const int64_t work = (int64_t)((a.F + a.dst.fsv - 1) / a.dst.fsv) * a.B * a.Y * a.X;
        const int64_t nb = (work + 255) / 256;
        CHIP_REQUIRE(nb < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "tensor too large for the reorder grid");
        // dword path: every row of every plane starts on a 4-byte boundary on both sides
        const bool dwords = a.dst.fsv == 4 && a.X % 4 == 0 && a.src.px == 1 && a.src.off % 4 == 0 && a.src.py % 4 == 0 && a.src.pf % 4 == 0
                            && a.src.pb % 4 == 0 && (uintptr_t)src % 4 == 0 && (uintptr_t)dst % 4 == 0 && work / 4 < (1ll << 31);
        const bool aligned16 = a.dst.off % 16 == 0 && a.dst.py % 16 == 0 && a.dst.pf % 16 == 0 && a.dst.pb % 16 == 0 && (uintptr_t)dst % 16 == 0;
        const dim3 grid4((unsigned)((work / 4 + 255) / 256));
        if (dwords && aligned16)
            hipLaunchKernelGGL(reorder_to_fsv4_x4_kernel<true>, grid4, dim3(256), 0, s, a, (const uint8_t*)src, (uint8_t*)dst);
        else if (dwords)
            hipLaunchKernelGGL(reorder_to_fsv4_x4_kernel<false>, grid4, dim3(256), 0, s, a, (const uint8_t*)src, (uint8_t*)dst);
        else if (a.dst.fsv == 4)
            hipLaunchKernelGGL(reorder_to_blocked_kernel<4>, dim3((unsigned)nb), dim3(256), 0, s, a, (const uint8_t*)src, (uint8_t*)dst);
        else
            hipLaunchKernelGGL(reorder_to_blocked_kernel<16>, dim3((unsigned)nb), dim3(256), 0, s, a, (const uint8_t*)src, (uint8_t*)dst);
        CHIP_CHECK(hipGetLastError());
        // feature slices the destination holds beyond ceil(F / fsv) do not exist in these formats
        return;
    }
    a.dst_fs_fill = a.dst.fsv > 1 ? a.dst.fs_count * a.dst.fsv - dt.f : 0;
    const int64_t total = (int64_t)a.B * (a.F + a.dst_fs_fill) * a.Y * a.X;
    const int64_t blocks = (total + 255) / 256;
    CHIP_REQUIRE(blocks < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "tensor too large for the reorder grid");
    hipLaunchKernelGGL(reorder_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, src, dst);
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
