// Pooling for the layers between the convolutions of an int8 network (max / average over a sliding window).
// Arithmetic after the reference's kernels: kernel_selector/core/cl_kernels/pooling_gpu_int8_ref.cl:15-140 (int8:
// int accumulator, average = round(sum / count) half away from zero) and pooling_gpu_ref.cl (float: accumulator in
// the unit type, no rounding).  Window taps outside the input are skipped; a window that lies outside the input
// altogether leaves its output untouched (the buffer's zero).
#include "common.h"
#include "epilogue.h"
#include "kernels.h"

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
    if (oy0 + a.ky < 0 || oy0 >= a.IH || ox0 + a.kx < 0 || ox0 >= a.IW) return;
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

// int8 in the blocked layout: one work-item per (pixel, slice of 16 features), 16-byte loads and one 16-byte store
template <bool UNSIGNED>
__global__ void __launch_bounds__(256) pooling_fsv16_kernel(PoolArgs a, const uint8_t* __restrict__ in, uint8_t* __restrict__ out)
{
    const int slices = (a.F + 15) / 16;
    const int64_t total = (int64_t)slices * a.B * a.OH * a.OW;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int x = (int)(idx % a.OW);
    int64_t r = idx / a.OW;
    const int y = (int)(r % a.OH);
    r /= a.OH;
    const int b = (int)(r % a.B), fs = (int)(r / a.B);
    const int oy0 = y * a.sy - a.py, ox0 = x * a.sx - a.px;
    if (oy0 + a.ky < 0 || oy0 >= a.IH || ox0 + a.kx < 0 || ox0 >= a.IW) return;
    const bool is_max = a.mode == CLDNN_HIP_POOL_MAX;
    int acc[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) acc[c] = is_max ? -128 : 0;
    int valid = 0;
    const int64_t base = a.in.off + (int64_t)b * a.in.pb + (int64_t)fs * a.in.pf;
    for (int j = 0; j < a.ky; ++j) {
        const int iy = oy0 + j;
        if (iy < 0 || iy >= a.IH) continue;
        for (int i = 0; i < a.kx; ++i) {
            const int ix = ox0 + i;
            if (ix < 0 || ix >= a.IW) continue;
            const uint4 v = *reinterpret_cast<const uint4*>(in + base + (int64_t)iy * a.in.py + (int64_t)ix * 16);
            const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                const unsigned byte = (w[c >> 2] >> (8 * (c & 3))) & 255u;
                const int e = UNSIGNED ? (int)byte : (int)(int8_t)byte;
                acc[c] = is_max ? max(acc[c], e) : acc[c] + e;
            }
            ++valid;
        }
    }
    if (!is_max) {
        const float n = (float)window_count(a, oy0, ox0, valid);
#pragma unroll
        for (int c = 0; c < 16; ++c) acc[c] = (int)round_half_away((float)acc[c] / n);
    }
    unsigned w[4] = {0, 0, 0, 0};
    const int live = a.F - fs * 16;  // features past the end of the tensor stay zero
#pragma unroll
    for (int c = 0; c < 16; ++c)
        if (c < live) w[c >> 2] |= ((unsigned)acc[c] & 255u) << (8 * (c & 3));
    *reinterpret_cast<uint4*>(out + a.out.off + (int64_t)b * a.out.pb + (int64_t)fs * a.out.pf + (int64_t)y * a.out.py + (int64_t)x * 16) =
        make_uint4(w[0], w[1], w[2], w[3]);
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
    if (blocked && it.dtype == CLDNN_HIP_U8)
        hipLaunchKernelGGL(pooling_fsv16_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, s, a, (const uint8_t*)in, (uint8_t*)out);
    else if (blocked)
        hipLaunchKernelGGL(pooling_fsv16_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, s, a, (const uint8_t*)in, (uint8_t*)out);
    else
        hipLaunchKernelGGL(pooling_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a, in, out);
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
