// General element-wise primitive: up to four inputs combined left to right with one operation, inputs read through
// strides and broadcast by size, int8 data either in the 8-bit type (wrap-around after every step) or, quantized, in
// int followed by round(r * factor), saturation to signed char and the activation.
//
// Follows the reference's generic kernel: indexing kernel_selector/core/cl_kernels/generic_eltwise_ref.cl:106-135,
// the operation chain kernel_selector/core/actual_kernels/eltwise/eltwise_kernel_base.cpp:236-352, the quantized
// tail generic_eltwise_ref.cl:311-330.  One work-item per output element, any layout; the residual sums of a
// network are normally fused into the convolution before them and never reach this kernel.
#include "epilogue.h"
#include "kernels.h"
#include "conv_mfma_kernel.h"  // FastDiv

namespace chip {

struct EltwiseArgs {
    Pitch in[CLDNN_HIP_ELTWISE_MAX_INPUTS];
    Pitch dst;
    const void* src[CLDNN_HIP_ELTWISE_MAX_INPUTS];
    int B[CLDNN_HIP_ELTWISE_MAX_INPUTS], F[CLDNN_HIP_ELTWISE_MAX_INPUTS], Y[CLDNN_HIP_ELTWISE_MAX_INPUTS],
        X[CLDNN_HIP_ELTWISE_MAX_INPUTS];
    int sy[CLDNN_HIP_ELTWISE_MAX_INPUTS], sx[CLDNN_HIP_ELTWISE_MAX_INPUTS], dt[CLDNN_HIP_ELTWISE_MAX_INPUTS];
    float coef[CLDNN_HIP_ELTWISE_MAX_INPUTS];
    int count, mode, has_coef;
    int OB, OF, OY, OX, dst_dt;
    int quantized;
    const float* calib;
    float oqf;
    int act;
    float m, n;
};

__device__ __forceinline__ int eltwise_op_int(int mode, int a, int b)
{
    switch (mode) {
    case CLDNN_HIP_ELTWISE_SUB: return a - b;
    case CLDNN_HIP_ELTWISE_MAX: return a > b ? a : b;
    case CLDNN_HIP_ELTWISE_PROD: return a * b;
    case CLDNN_HIP_ELTWISE_DIV: return b ? a / b : 0;
    case CLDNN_HIP_ELTWISE_MIN: return a < b ? a : b;
    case CLDNN_HIP_ELTWISE_MOD: return b ? a % b : 0;
    default: return a + b;
    }
}

__device__ __forceinline__ float eltwise_op_float(int mode, float a, float b)
{
    switch (mode) {
    case CLDNN_HIP_ELTWISE_SUB: return a - b;
    case CLDNN_HIP_ELTWISE_MAX: return fmaxf(a, b);
    case CLDNN_HIP_ELTWISE_PROD: return a * b;
    case CLDNN_HIP_ELTWISE_DIV: return a / b;
    case CLDNN_HIP_ELTWISE_MIN: return fminf(a, b);
    case CLDNN_HIP_ELTWISE_POW: return powf(a, b);
    case CLDNN_HIP_ELTWISE_MOD: return fmodf(a, b);
    default: return a + b;
    }
}

__global__ void __launch_bounds__(256) eltwise_kernel(EltwiseArgs p, void* __restrict__ dst)
{
    const int64_t total = (int64_t)p.OB * p.OF * p.OY * p.OX;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    // the destination's innermost axis runs fastest over the lanes, so that the stores coalesce
    int bi, f, y, x;
    if (p.dst.fsv > 1 || p.dst.pf == 1) {
        f = (int)(idx % p.OF);
        int64_t r = idx / p.OF;
        x = (int)(r % p.OX);
        r /= p.OX;
        y = (int)(r % p.OY);
        bi = (int)(r / p.OY);
    } else {
        x = (int)(idx % p.OX);
        int64_t r = idx / p.OX;
        y = (int)(r % p.OY);
        r /= p.OY;
        f = (int)(r % p.OF);
        bi = (int)(r / p.OF);
    }
    auto at = [&](int i) {
        return p.in[i].at(bi % p.B[i], f % p.F[i], (y * p.sy[i]) % p.Y[i], (x * p.sx[i]) % p.X[i]);
    };
    EpiOut o;
    if (p.dt[0] == CLDNN_HIP_F32) {
        float v = ((const float*)p.src[0])[at(0)];
        if (p.has_coef) v *= p.coef[0];
        for (int i = 1; i < p.count; ++i) {
            float w = load_as_float(p.src[i], p.dt[i], at(i));
            if (p.has_coef) w *= p.coef[i];
            v = eltwise_op_float(p.mode, v, w);
        }
        v = act_f(p.act, p.m, p.n, v);
        o.f = v;
        o.i = p.dst_dt == CLDNN_HIP_U8 ? sat_u8(round_half_away(v)) : sat_s8(round_half_away(v));
    } else {
        const bool is_unsigned = p.dt[0] == CLDNN_HIP_U8;
        auto load = [&](int i) {
            const int64_t a = at(i);
            if (p.dt[i] == CLDNN_HIP_U8) return (int)((const uint8_t*)p.src[i])[a];
            if (p.dt[i] == CLDNN_HIP_S8) return (int)((const int8_t*)p.src[i])[a];
            // a float operand of int8 data is cast to the 8-bit type first (toward zero)
            const int t = (int)((const float*)p.src[i])[a];
            return is_unsigned ? (int)(unsigned char)t : (int)(signed char)t;
        };
        int v = load(0);
        for (int i = 1; i < p.count; ++i) {
            v = eltwise_op_int(p.mode, v, load(i));
            // outside the quantized form every intermediate has the data's own 8-bit type
            if (!p.quantized) v = is_unsigned ? (int)(unsigned char)v : (int)(signed char)v;
        }
        if (p.quantized) {
            const float s = p.calib ? p.calib[f] : p.oqf;
            v = (int)round_half_away((float)v * s);
            v = v < -128 ? -128 : (v > 127 ? 127 : v);  // convert_char_sat
        }
        v = act_i(p.act, p.m, p.n, v);
        o.f = (float)v;
        // the value is assigned to the output's 8-bit type: conversion between the integer types wraps
        o.i = p.dst_dt == CLDNN_HIP_U8 ? (int)(unsigned char)v : (p.dst_dt == CLDNN_HIP_S8 ? (int)(signed char)v : v);
    }
    store_out(dst, p.dst_dt, p.dst.at(bi, f, y, x), o);
}

// The form a quantized network meets between its convolutions: every operand 8-bit in fs_b_yx_fsv16, same logical size
// (strides allowed, no broadcast).  One lane = one pixel of one 16-feature slice: a 16-byte load per input, the same
// arithmetic as above on 16 values, one 16-byte store; the padding features of the last slice are written as zero.
struct EltwiseBlockedArgs {
    const uint8_t* src[CLDNN_HIP_ELTWISE_MAX_INPUTS];
    int off[CLDNN_HIP_ELTWISE_MAX_INPUTS], pb[CLDNN_HIP_ELTWISE_MAX_INPUTS], pf[CLDNN_HIP_ELTWISE_MAX_INPUTS],
        py[CLDNN_HIP_ELTWISE_MAX_INPUTS], px[CLDNN_HIP_ELTWISE_MAX_INPUTS];  // bytes; the strides are folded into py / px
    int is_u8[CLDNN_HIP_ELTWISE_MAX_INPUTS];
    int count, mode;
    int doff, dpb, dpf, dpy;
    int B, F, Y, X, slices;
    FastDiv div_x;
    int quantized, calib_vec4;
    const float* calib;
    float oqf;
    int act;
    float m, n;
};

// MODE: the operation fixed at compile time (the sum of a residual block: the common case), or -1 = read it from the
// arguments.  Left to the run-time value alone, the sixteen switch statements of a lane stay sixteen chains of scalar
// branches, each with the division sequences of the div and mod modes behind them.
template <int MODE>
__global__ void __launch_bounds__(256) eltwise_blocked_kernel(EltwiseBlockedArgs p, uint8_t* __restrict__ dst)
{
    const int mode = MODE >= 0 ? MODE : p.mode;
    // grid: x over the pixels of a plane, y = batch, z = feature slice
    const unsigned pixel = blockIdx.x * blockDim.x + threadIdx.x;
    if (pixel >= (unsigned)(p.Y * p.X)) return;
    const int y = (int)p.div_x.div(pixel), x = (int)(pixel - (unsigned)y * p.X);
    const int b = (int)blockIdx.y, fs = (int)blockIdx.z;
    int v[16];
    {
        const uint4 w = *reinterpret_cast<const uint4*>(p.src[0] + p.off[0] + b * p.pb[0] + fs * p.pf[0] + y * p.py[0] + x * p.px[0]);
        const unsigned ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const unsigned byte = (ww[c >> 2] >> (8 * (c & 3))) & 255u;
            v[c] = p.is_u8[0] ? (int)byte : (int)(signed char)byte;
        }
    }
    const bool wrap_unsigned = p.is_u8[0] != 0;
    for (int i = 1; i < p.count; ++i) {
        const uint4 w = *reinterpret_cast<const uint4*>(p.src[i] + p.off[i] + b * p.pb[i] + fs * p.pf[i] + y * p.py[i] + x * p.px[i]);
        const unsigned ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const unsigned byte = (ww[c >> 2] >> (8 * (c & 3))) & 255u;
            int o = p.is_u8[i] ? (int)byte : (int)(signed char)byte;
            // an operand of the other 8-bit type is cast to the first input's type first
            if (p.is_u8[i] != p.is_u8[0]) o = wrap_unsigned ? (int)(unsigned char)o : (int)(signed char)o;
            int t = eltwise_op_int(mode, v[c], o);
            if (!p.quantized) t = wrap_unsigned ? (int)(unsigned char)t : (int)(signed char)t;
            v[c] = t;
        }
    }
    unsigned out[4] = {0, 0, 0, 0};
    const int f0 = fs * 16;
    float scale[16];
    if (p.quantized) {
        if (p.calib && p.calib_vec4) {  // whole slices and an aligned vector: four 16-byte loads
#pragma unroll
            for (int d4 = 0; d4 < 4; ++d4) {
                const float4 c4 = *reinterpret_cast<const float4*>(p.calib + f0 + d4 * 4);
                scale[d4 * 4 + 0] = c4.x, scale[d4 * 4 + 1] = c4.y, scale[d4 * 4 + 2] = c4.z, scale[d4 * 4 + 3] = c4.w;
            }
        } else {
#pragma unroll
            for (int c = 0; c < 16; ++c) scale[c] = p.calib ? p.calib[f0 + c < p.F ? f0 + c : 0] : p.oqf;
        }
    }
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        int t = v[c];
        if (p.quantized) {
            const float s = scale[c];
            t = (int)round_half_away((float)t * s);
            t = t < -128 ? -128 : (t > 127 ? 127 : t);
        }
        t = act_i(p.act, p.m, p.n, t);
        if (f0 + c < p.F) out[c >> 2] |= ((unsigned)t & 255u) << (8 * (c & 3));
    }
    *reinterpret_cast<uint4*>(dst + p.doff + b * p.dpb + fs * p.dpf + y * p.dpy + x * 16) = make_uint4(out[0], out[1], out[2], out[3]);
}

// true when the blocked kernel was launched
static bool launch_eltwise_blocked(hipStream_t s, const cldnn_hip_eltwise_desc& d, const void* const* inputs, const float* calib, void* dst)
{
    const cldnn_hip_tensor& o = d.output;
    auto byte_type = [](int dt) { return dt == CLDNN_HIP_S8 || dt == CLDNN_HIP_U8; };
    if (o.format != CLDNN_HIP_FMT_FS_B_YX_FSV16 || !byte_type(o.dtype) || d.has_coefficients) return false;
    if (tensor_elems(o) >= (1ull << 31)) return false;
    EltwiseBlockedArgs p{};
    for (int i = 0; i < d.n_inputs; ++i) {
        const cldnn_hip_tensor& t = d.inputs[i];
        const int sy = d.stride_y[i] > 0 ? d.stride_y[i] : 1, sx = d.stride_x[i] > 0 ? d.stride_x[i] : 1;
        if (!inputs[i] || t.format != CLDNN_HIP_FMT_FS_B_YX_FSV16 || !byte_type(t.dtype) || tensor_elems(t) >= (1ull << 31)) return false;
        // same features and batch, spatial size covered exactly: nothing wraps around
        if (t.b != o.b || t.f != o.f || t.y / sy != o.y || t.x / sx != o.x) return false;
        const Pitch q = make_pitch(t);
        p.src[i] = (const uint8_t*)inputs[i];
        p.off[i] = (int)q.off, p.pb[i] = (int)q.pb, p.pf[i] = (int)q.pf, p.py[i] = (int)q.py * sy, p.px[i] = (int)q.px * sx;
        p.is_u8[i] = t.dtype == CLDNN_HIP_U8;
    }
    const Pitch q = make_pitch(o);
    p.count = d.n_inputs, p.mode = d.mode;
    p.doff = (int)q.off, p.dpb = (int)q.pb, p.dpf = (int)q.pf, p.dpy = (int)q.py;
    p.B = o.b, p.F = o.f, p.Y = o.y, p.X = o.x, p.slices = (o.f + 15) / 16;
    // (the stored value is the low byte of the result for either output type: conversion between the 8-bit types wraps)
    p.quantized = d.quantized, p.calib = calib, p.oqf = d.output_quantization_factor;
    p.act = d.activation, p.m = d.m, p.n = d.n;
    p.calib_vec4 = calib && o.f % 16 == 0 && (uintptr_t)calib % 16 == 0;
    const int64_t plane = (int64_t)p.Y * p.X;
    if (plane == 0 || p.B == 0) return true;
    if (p.B > 65535 || p.slices > 65535) return false;
    p.div_x = make_fast_div((uint32_t)p.X);
    const dim3 grid((unsigned)((plane + 255) / 256), (unsigned)p.B, (unsigned)p.slices);
    if (p.mode == CLDNN_HIP_ELTWISE_SUM) hipLaunchKernelGGL(eltwise_blocked_kernel<CLDNN_HIP_ELTWISE_SUM>, grid, dim3(256), 0, s, p, (uint8_t*)dst);
    else hipLaunchKernelGGL(eltwise_blocked_kernel<-1>, grid, dim3(256), 0, s, p, (uint8_t*)dst);
    CHIP_CHECK(hipGetLastError());
    return true;
}

void launch_eltwise(hipStream_t s, const cldnn_hip_eltwise_desc& d, const void* const* inputs, const float* calib, void* dst)
{
    CHIP_REQUIRE(d.n_inputs >= 2 && d.n_inputs <= CLDNN_HIP_ELTWISE_MAX_INPUTS, CLDNN_HIP_INVALID_ARG,
                 "eltwise: between 2 and 4 inputs");
    CHIP_REQUIRE(d.mode >= CLDNN_HIP_ELTWISE_SUM && d.mode <= CLDNN_HIP_ELTWISE_MOD, CLDNN_HIP_INVALID_ARG,
                 "eltwise: unknown mode (the comparison and logic modes are not part of this library)");
    const int dt0 = d.inputs[0].dtype;
    const bool int_data = dt0 == CLDNN_HIP_S8 || dt0 == CLDNN_HIP_U8;
    CHIP_REQUIRE(int_data || dt0 == CLDNN_HIP_F32, CLDNN_HIP_INVALID_ARG, "eltwise: data must be int8, uint8 or float");
    // reference src/eltwise.cpp:38-46
    CHIP_REQUIRE(!(int_data && d.mode == CLDNN_HIP_ELTWISE_POW), CLDNN_HIP_INVALID_ARG,
                 "Requested eltwise mode is not supported for integer types.");
    CHIP_REQUIRE(!d.quantized || int_data, CLDNN_HIP_INVALID_ARG, "eltwise: the quantized form needs int8 inputs");
    CHIP_REQUIRE(!d.has_coefficients || (!int_data && d.mode == CLDNN_HIP_ELTWISE_SUM), CLDNN_HIP_INVALID_ARG,
                 "eltwise: coefficients belong to a float sum");
    const cldnn_hip_tensor& o = d.output;
    if (int_data && launch_eltwise_blocked(s, d, inputs, calib, dst)) return;
    EltwiseArgs p{};
    p.count = d.n_inputs, p.mode = d.mode, p.has_coef = d.has_coefficients;
    for (int i = 0; i < d.n_inputs; ++i) {
        const cldnn_hip_tensor& t = d.inputs[i];
        CHIP_REQUIRE(inputs[i], CLDNN_HIP_INVALID_ARG, "eltwise: null input");
        const bool ti = t.dtype == CLDNN_HIP_S8 || t.dtype == CLDNN_HIP_U8;
        CHIP_REQUIRE(ti || t.dtype == CLDNN_HIP_F32, CLDNN_HIP_INVALID_ARG, "eltwise: data must be int8, uint8 or float");
        p.in[i] = make_pitch(t), p.src[i] = inputs[i], p.dt[i] = t.dtype;
        p.B[i] = t.b, p.F[i] = t.f, p.Y[i] = t.y, p.X[i] = t.x;
        p.sy[i] = d.stride_y[i] > 0 ? d.stride_y[i] : 1, p.sx[i] = d.stride_x[i] > 0 ? d.stride_x[i] : 1;
        p.coef[i] = d.coefficients[i];
        CHIP_REQUIRE(t.b > 0 && t.f > 0 && t.y > 0 && t.x > 0, CLDNN_HIP_INVALID_ARG, "eltwise: empty input");
        // a strided input covers the output exactly; an unstrided one repeats (index modulo its size)
        auto fits = [](int in, int stride, int out) { return stride > 1 ? in / stride == out : in <= out; };
        CHIP_REQUIRE(fits(t.b, 1, o.b) && fits(t.f, 1, o.f) && fits(t.y, p.sy[i], o.y) && fits(t.x, p.sx[i], o.x),
                     CLDNN_HIP_DIMENSION_MISMATCH, "eltwise: an input does not cover the output");
    }
    p.dst = make_pitch(o), p.dst_dt = o.dtype;
    p.OB = o.b, p.OF = o.f, p.OY = o.y, p.OX = o.x;
    p.quantized = d.quantized, p.calib = calib, p.oqf = d.output_quantization_factor;
    p.act = d.activation, p.m = d.m, p.n = d.n;
    const int64_t total = (int64_t)p.OB * p.OF * p.OY * p.OX;
    if (total == 0) return;
    const int64_t blocks = (total + 255) / 256;
    CHIP_REQUIRE(blocks < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "tensor too large for the eltwise grid");
    hipLaunchKernelGGL(eltwise_kernel, dim3((unsigned)blocks), dim3(256), 0, s, p, dst);
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
