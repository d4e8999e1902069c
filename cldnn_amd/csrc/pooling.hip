// Pooling for the layers between the convolutions of an int8 network (max / average over a sliding window).
// Arithmetic after the reference's kernels: kernel_selector/core/cl_kernels/pooling_gpu_int8_ref.cl:15-140 (int8:
// int accumulator, average = round(sum / count) half away from zero) and pooling_gpu_ref.cl (float: accumulator in
// the unit type, no rounding).  Window taps outside the input are skipped; a window that lies outside the input
// altogether leaves its output untouched (the buffer's zero).
#include "common.h"
#include "epilogue.h"
#include "kernels.h"
#include "conv_mfma_kernel.h"  // FastDiv

namespace chip {

struct PoolArgs {
    Pitch in, out;
    int B, F, IH, IW, OH, OW;
    int ky, kx, sy, sx, py, px;
    int mode;     // CLDNN_HIP_POOL_*
    int divider;  // CLDNN_HIP_POOL_DIV_*
    int dt;
};

__device__ __forceinline__ int window_count(const PoolArgs& a, int oy0, int ox0, int valid)
{
    if (a.divider == CLDNN_HIP_POOL_DIV_FIXED) return a.ky * a.kx;
    if (a.divider == CLDNN_HIP_POOL_DIV_VALID) return valid > 0 ? valid : 1;
    // window clipped to the input plus its padding (pooling_gpu_int8_ref.cl:104-108)
    const int hend = min(oy0 + a.ky, a.IH + a.py), wend = min(ox0 + a.kx, a.IW + a.px);
    const int n = (hend - oy0) * (wend - ox0);
    return n > 0 ? n : 1;
}

// one work-item per output element, any layout
__global__ void __launch_bounds__(256) pooling_kernel(PoolArgs a, const void* __restrict__ in, void* __restrict__ out)
{
    const int64_t total = (int64_t)a.B * a.F * a.OH * a.OW;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    int b, f, y, x;
    if (a.out.fsv > 1 || a.out.pf == 1) {  // features innermost in memory
        f = (int)(idx % a.F);
        int64_t r = idx / a.F;
        x = (int)(r % a.OW);
        r /= a.OW;
        y = (int)(r % a.OH);
        b = (int)(r / a.OH);
    } else {
        x = (int)(idx % a.OW);
        int64_t r = idx / a.OW;
        y = (int)(r % a.OH);
        r /= a.OH;
        f = (int)(r % a.F);
        b = (int)(r / a.F);
    }
    const int oy0 = y * a.sy - a.py, ox0 = x * a.sx - a.px;
    if (oy0 + a.ky < 0 || oy0 >= a.IH || ox0 + a.kx < 0 || ox0 >= a.IW) {
        // A window that lies wholly outside the input: the reference's kernel leaves such an output untouched, i.e. at
        // the zero its buffers are created with (pooling_gpu_int8_ref.cl:62-68).  A buffer handed over by the memory
        // pool is not zero, so the zero is written.
        EpiOut z;
        z.f = 0.0f, z.i = 0;
        store_out(out, a.dt, a.out.at(b, f, y, x), z);
        return;
    }
    const bool is_max = a.mode == CLDNN_HIP_POOL_MAX;
    int valid = 0;
    EpiOut o;
    if (a.dt == CLDNN_HIP_F32) {
        float r = is_max ? -3.402823466e+38f : 0.0f;  // UNIT_VAL_MIN of float
        for (int j = 0; j < a.ky; ++j) {
            const int iy = oy0 + j;
            if (iy < 0 || iy >= a.IH) continue;
            for (int i = 0; i < a.kx; ++i) {
                const int ix = ox0 + i;
                if (ix < 0 || ix >= a.IW) continue;
                const float v = ((const float*)in)[a.in.at(b, f, iy, ix)];
                r = is_max ? fmaxf(r, v) : r + v;
                ++valid;
            }
        }
        if (!is_max) r = r / (float)window_count(a, oy0, ox0, valid);
        o.f = r, o.i = 0;
    } else {
        int r = is_max ? -128 : 0;  // CHAR_MIN also for unsigned data, as in the reference
        for (int j = 0; j < a.ky; ++j) {
            const int iy = oy0 + j;
            if (iy < 0 || iy >= a.IH) continue;
            for (int i = 0; i < a.kx; ++i) {
                const int ix = ox0 + i;
                if (ix < 0 || ix >= a.IW) continue;
                const int64_t at = a.in.at(b, f, iy, ix);
                const int v = a.dt == CLDNN_HIP_U8 ? (int)((const uint8_t*)in)[at] : (int)((const int8_t*)in)[at];
                r = is_max ? max(r, v) : r + v;
                ++valid;
            }
        }
        if (!is_max) r = (int)round_half_away((float)r / (float)window_count(a, oy0, ox0, valid));
        o.i = r, o.f = (float)r;
    }
    store_out(out, a.dt, a.out.at(b, f, y, x), o);
}

// int8 in the blocked layout: one work-item per (pixel, slice of 16 features), 16-byte loads and one 16-byte store.
// 32-bit index arithmetic with precomputed reciprocals; windows that lie inside the input skip the per-tap tests.
struct PoolFastArgs {
    PoolArgs a;
    FastDiv div_ow, div_oh, div_b;
    uint32_t total;
    int32_t in_off, in_pb, in_pf, in_py, out_off, out_pb, out_pf, out_py;
};

// SPLIT > 1: the taps of one window are shared out over SPLIT adjacent lanes and combined with lane shuffles (large
// windows over few outputs, e.g. the global average in front of a classifier: 49 taps, 4096 outputs x slices).
template <bool UNSIGNED, bool MAX, int SPLIT>
__global__ void __launch_bounds__(256) pooling_fsv16_kernel(PoolFastArgs p, const uint8_t* __restrict__ in, uint8_t* __restrict__ out)
{
    const PoolArgs& a = p.a;
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    const uint32_t idx = gid / SPLIT;
    const int part = (int)(gid % SPLIT);
    if (idx >= p.total) return;  // whole groups of SPLIT lanes leave together
    uint32_t r = p.div_ow.div(idx);
    const int x = (int)(idx - r * (uint32_t)a.OW);
    uint32_t r2 = p.div_oh.div(r);
    const int y = (int)(r - r2 * (uint32_t)a.OH);
    const uint32_t fs = p.div_b.div(r2);
    const int b = (int)(r2 - fs * (uint32_t)a.B);
    const int oy0 = y * a.sy - a.py, ox0 = x * a.sx - a.px;
    if (oy0 + a.ky < 0 || oy0 >= a.IH || ox0 + a.kx < 0 || ox0 >= a.IW) {
        // a window wholly outside the input: zero, as a freshly created buffer of the reference holds (see pooling_kernel);
        // the lanes of a SPLIT group share the window and leave together
        if (part == 0)
            *reinterpret_cast<uint4*>(out + (p.out_off + b * p.out_pb + (int)fs * p.out_pf + y * p.out_py + x * 16)) = make_uint4(0, 0, 0, 0);
        return;
    }
    int acc[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) acc[c] = MAX ? -128 : 0;
    const uint8_t* src = in + (p.in_off + b * p.in_pb + (int)fs * p.in_pf);
    auto tap = [&](int iy, int ix) {
        const uint4 v = *reinterpret_cast<const uint4*>(src + (iy * p.in_py + ix * 16));
        const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const unsigned byte = (w[c >> 2] >> (8 * (c & 3))) & 255u;
            const int e = UNSIGNED ? (int)byte : (int)(int8_t)byte;
            acc[c] = MAX ? max(acc[c], e) : acc[c] + e;
        }
    };
    int valid = 0;
    if constexpr (SPLIT > 1) {
        const int taps = a.ky * a.kx;
        for (int t = part; t < taps; t += SPLIT) {
            const int j = t / a.kx, i = t - j * a.kx;
            const int iy = oy0 + j, ix = ox0 + i;
            if (iy < 0 || iy >= a.IH || ix < 0 || ix >= a.IW) continue;
            tap(iy, ix);
            ++valid;
        }
#pragma unroll
        for (int m = 1; m < SPLIT; m *= 2) {
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                const int o = __shfl_xor(acc[c], m, 64);
                acc[c] = MAX ? max(acc[c], o) : acc[c] + o;
            }
            valid += __shfl_xor(valid, m, 64);
        }
        if (part != 0) return;
    } else if (oy0 >= 0 && ox0 >= 0 && oy0 + a.ky <= a.IH && ox0 + a.kx <= a.IW) {
        for (int j = 0; j < a.ky; ++j)
            for (int i = 0; i < a.kx; ++i) tap(oy0 + j, ox0 + i);
        valid = a.ky * a.kx;
    } else {
        for (int j = 0; j < a.ky; ++j) {
            const int iy = oy0 + j;
            if (iy < 0 || iy >= a.IH) continue;
            for (int i = 0; i < a.kx; ++i) {
                const int ix = ox0 + i;
                if (ix < 0 || ix >= a.IW) continue;
                tap(iy, ix);
                ++valid;
            }
        }
    }
    if (!MAX) {
        const float n = (float)window_count(a, oy0, ox0, valid);
#pragma unroll
        for (int c = 0; c < 16; ++c) acc[c] = (int)round_half_away((float)acc[c] / n);
    }
    unsigned w[4] = {0, 0, 0, 0};
    const int live = a.F - (int)fs * 16;  // features past the end of the tensor stay zero
#pragma unroll
    for (int c = 0; c < 16; ++c)
        if (c < live) w[c >> 2] |= ((unsigned)acc[c] & 255u) << (8 * (c & 3));
    *reinterpret_cast<uint4*>(out + (p.out_off + b * p.out_pb + (int)fs * p.out_pf + y * p.out_py + x * 16)) = make_uint4(w[0], w[1], w[2], w[3]);
}

void launch_pooling(hipStream_t s, const cldnn_hip_pooling_desc& d, const void* in, void* out)
{
    const cldnn_hip_tensor &it = d.input, &ot = d.output;
    CHIP_REQUIRE(d.mode == CLDNN_HIP_POOL_MAX || d.mode == CLDNN_HIP_POOL_AVERAGE, CLDNN_HIP_INVALID_ARG, "pooling: unknown mode");
    CHIP_REQUIRE(d.divider >= CLDNN_HIP_POOL_DIV_FIXED && d.divider <= CLDNN_HIP_POOL_DIV_PADDED, CLDNN_HIP_INVALID_ARG,
                 "pooling: unknown divider mode");
    CHIP_REQUIRE(d.size_y > 0 && d.size_x > 0 && d.stride_y > 0 && d.stride_x > 0 && d.pad_y >= 0 && d.pad_x >= 0,
                 CLDNN_HIP_INVALID_ARG, "pooling: window and stride must be positive, padding non-negative");
    CHIP_REQUIRE(it.dtype == ot.dtype, CLDNN_HIP_INVALID_ARG, "pooling keeps the data type");
    CHIP_REQUIRE(it.dtype == CLDNN_HIP_S8 || it.dtype == CLDNN_HIP_U8 || it.dtype == CLDNN_HIP_F32, CLDNN_HIP_INVALID_ARG,
                 "pooling: data must be s8, u8 or f32");
    CHIP_REQUIRE(it.b == ot.b && it.f == ot.f, CLDNN_HIP_DIMENSION_MISMATCH, "pooling keeps batch and feature counts");
    CHIP_REQUIRE(ot.y > 0 && ot.x > 0, CLDNN_HIP_DIMENSION_MISMATCH, "pooling: empty output");
    PoolArgs a{};
    a.in = make_pitch(it), a.out = make_pitch(ot);
    a.B = it.b, a.F = it.f, a.IH = it.y, a.IW = it.x, a.OH = ot.y, a.OW = ot.x;
    a.ky = d.size_y, a.kx = d.size_x, a.sy = d.stride_y, a.sx = d.stride_x, a.py = d.pad_y, a.px = d.pad_x;
    a.mode = d.mode, a.divider = d.divider, a.dt = it.dtype;
    const bool blocked = it.format == CLDNN_HIP_FMT_FS_B_YX_FSV16 && ot.format == CLDNN_HIP_FMT_FS_B_YX_FSV16 && it.dtype != CLDNN_HIP_F32;
    const int64_t total = blocked ? (int64_t)((a.F + 15) / 16) * a.B * a.OH * a.OW : (int64_t)a.B * a.F * a.OH * a.OW;
    const int64_t blocks = (total + 255) / 256;
    CHIP_REQUIRE(blocks < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "tensor too large for the pooling grid");
    if (blocked) {
        CHIP_REQUIRE(tensor_elems(it) < (1ull << 31) && tensor_elems(ot) < (1ull << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "tensor of 2 GiB or more");
        PoolFastArgs p{};
        p.a = a;
        p.div_ow = make_fast_div((uint32_t)a.OW), p.div_oh = make_fast_div((uint32_t)a.OH), p.div_b = make_fast_div((uint32_t)a.B);
        p.total = (uint32_t)total;
        p.in_off = (int32_t)a.in.off, p.in_pb = (int32_t)a.in.pb, p.in_pf = (int32_t)a.in.pf, p.in_py = (int32_t)a.in.py;
        p.out_off = (int32_t)a.out.off, p.out_pb = (int32_t)a.out.pb, p.out_pf = (int32_t)a.out.pf, p.out_py = (int32_t)a.out.py;
        const bool u = it.dtype == CLDNN_HIP_U8, mx = d.mode == CLDNN_HIP_POOL_MAX;
        // few outputs with many taps each: 16 lanes per window
        const bool split = a.ky * a.kx >= 16 && total * 16 < (1ll << 31) && total < 256 * 1024;
        const dim3 grid((unsigned)(split ? (total * 16 + 255) / 256 : blocks)), block(256);
        const uint8_t* src = (const uint8_t*)in;
        uint8_t* dst = (uint8_t*)out;
        if (split) {
            if (u && mx) hipLaunchKernelGGL((pooling_fsv16_kernel<true, true, 16>), grid, block, 0, s, p, src, dst);
            else if (u) hipLaunchKernelGGL((pooling_fsv16_kernel<true, false, 16>), grid, block, 0, s, p, src, dst);
            else if (mx) hipLaunchKernelGGL((pooling_fsv16_kernel<false, true, 16>), grid, block, 0, s, p, src, dst);
            else hipLaunchKernelGGL((pooling_fsv16_kernel<false, false, 16>), grid, block, 0, s, p, src, dst);
        } else if (u && mx) hipLaunchKernelGGL((pooling_fsv16_kernel<true, true, 1>), grid, block, 0, s, p, src, dst);
        else if (u) hipLaunchKernelGGL((pooling_fsv16_kernel<true, false, 1>), grid, block, 0, s, p, src, dst);
        else if (mx) hipLaunchKernelGGL((pooling_fsv16_kernel<false, true, 1>), grid, block, 0, s, p, src, dst);
        else hipLaunchKernelGGL((pooling_fsv16_kernel<false, false, 1>), grid, block, 0, s, p, src, dst);
    } else {
        hipLaunchKernelGGL(pooling_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, in, out);
    }
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
