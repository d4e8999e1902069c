// Device-side epilogue of the quantized convolution: int32 accumulator -> stored value.
// Every float operation below is a separately rounded IEEE operation (the library is built
// with -ffp-contract=off); the sequence follows the reference semantic kernel
// kernel_selector/core/cl_kernels/fused_conv_eltwise_gpu_ref.cl:148-232.
#pragma once
#include "common.h"

namespace chip {

// OpenCL round(): halfway cases away from zero.  0.49999997f is the largest float below one half;
// trunc(x + copysign(0.49999997f, x)) equals round-half-away(x) for every finite float (checked
// exhaustively on the host over all 2^32 bit patterns).
__device__ __forceinline__ float round_half_away(float x)
{
    return truncf(x + copysignf(0.49999997f, x));
}

__device__ __forceinline__ float round_sel(float x, int even)
{
    return even ? rintf(x) : round_half_away(x);
}

// jitter.cpp:373-396 (float instantiation)
__device__ __forceinline__ float act_f(int act, float m, float n, float x)
{
    switch (act) {
    case CLDNN_HIP_ACT_RELU: return fmaxf(0.0f, x);
    case CLDNN_HIP_ACT_RELU_SLOPE:
        if (isinf(m)) return x >= 0.0f ? x : -m;
        return fmaxf(x, 0.0f) + (m * fminf(x, 0.0f));
    case CLDNN_HIP_ACT_CLAMP: return fmaxf(m, fminf(n, x));
    default: return x;
    }
}

__device__ __forceinline__ int act_i(int act, float m, float n, int x)
{
    switch (act) {
    case CLDNN_HIP_ACT_RELU: return x > 0 ? x : 0;
    case CLDNN_HIP_ACT_RELU_SLOPE: {
        int s = (int)m;
        return (x > 0 ? x : 0) + s * (x < 0 ? x : 0);
    }
    case CLDNN_HIP_ACT_CLAMP: {
        int lo = (int)m;
        float t = (float)x < n ? (float)x : n;
        int ti = (int)t;
        return ti > lo ? ti : lo;
    }
    default: return x;
    }
}

// convert_char_sat / convert_uchar_sat of a float that is already integral (or NaN -> 0)
__device__ __forceinline__ int sat_s8(float v)
{
    if (v != v) return 0;  // convert_char_sat(NaN) == 0
    v = fminf(fmaxf(v, -128.0f), 127.0f);
    return (int)v;
}
__device__ __forceinline__ int sat_u8(float v)
{
    if (v != v) return 0;
    v = fminf(fmaxf(v, 0.0f), 255.0f);
    return (int)v;
}

struct EpiOut {
    float f;  // value when the output type is float
    int i;    // value when the output type is s8/u8 (already saturated)
};

__device__ __forceinline__ float load_as_float(const void* p, int dt, int64_t i)
{
    switch (dt) {
    case CLDNN_HIP_S8: return (float)((const int8_t*)p)[i];
    case CLDNN_HIP_U8: return (float)((const uint8_t*)p)[i];
    case CLDNN_HIP_I32: return (float)((const int32_t*)p)[i];
    default: return ((const float*)p)[i];
    }
}

__device__ __forceinline__ EpiOut finish(const Epilogue& e, float o)
{
    EpiOut r;
    r.f = o;
    r.i = 0;
    if (e.out_dt == CLDNN_HIP_S8) r.i = sat_s8(o);
    else if (e.out_dt == CLDNN_HIP_U8) r.i = sat_u8(o);
    return r;
}

// acc: int32 accumulator WITHOUT bias; eltw: residual value already widened to float
// (exact for int8 / int32 below 2^24 / float).
__device__ __forceinline__ EpiOut epilogue_generic(const Epilogue& e, int acc, int f, float eltw)
{
    const bool out_fp = e.out_dt == CLDNN_HIP_F32;
    if (e.mode == MODE_Q && e.fc) {
        int v = acc;
        if (e.bias) {
            const float bv = e.bias_dt == CLDNN_HIP_F32 ? ((const float*)e.bias)[f] : (float)((const int*)e.bias)[f];
            float x = (float)acc * e.wqf[f];
            x = x * e.iqf;
            x = x + bv;
            x = x * (e.calib ? e.calib[f] : e.oqf);
            v = (int)(signed char)(int)round_sel(x, e.round_even);
        }
        const int c = act_i(e.act, e.act_m, e.act_n, (int)(signed char)v);
        EpiOut r;
        r.i = (int)(signed char)c, r.f = (float)r.i;
        if (e.out_dt == CLDNN_HIP_U8) r.i = r.i < 0 ? 0 : r.i;
        return r;
    }
    if (e.mode == MODE_Q) {
        if (e.bias && !e.bias_after) {
            int bv = e.bias_dt == CLDNN_HIP_F32 ? (int)((const float*)e.bias)[f] : ((const int*)e.bias)[f];
            acc = (int)((unsigned)acc + (unsigned)bv);
        }
        float deq = (float)acc;
        if (e.wqf) {
            deq = deq * e.wqf[f];
            deq = deq * e.iqf;
        }
        if (e.bias_after) deq = deq + ((const float*)e.bias)[f];
        const bool second = e.split_f > 0 && f >= e.split_f;  // the sibling convolution's features
        float a = second ? act_f(e.act2, e.act2_m, e.act2_n, deq) : act_f(e.act, e.act_m, e.act_n, deq);
        float cal = a;
        if (e.calib) cal = a * e.calib[f];
        else if (e.oqf_on) cal = a * e.oqf;
        if (!e.fused) {
            if (!out_fp) cal = round_sel(cal, e.round_even);
            return finish(e, cal);
        }
        cal = round_sel(cal, e.round_even);
        if (e.conv_sat) cal = (float)(e.conv_sat == 1 ? sat_s8(cal) : sat_u8(cal));  // what an int8 tensor in between would hold
        float ev = e.ncs_on ? eltw * e.ncs : eltw;
        float s = cal + ev;
        float ea = act_f(e.eltw_act, e.eltw_m, e.eltw_n, s);
        float o = ea;
        if (e.eltw_calib) o = ea * e.eltw_calib[f];
        if (!out_fp) o = round_sel(o, e.round_even);
        return finish(e, o);
    }
    // MODE_FINT: integer activation, float only in the final calibration
    if (e.bias) {
        int bv = e.bias_dt == CLDNN_HIP_F32 ? (int)((const float*)e.bias)[f] : ((const int*)e.bias)[f];
        acc = (int)((unsigned)acc + (unsigned)bv);
    }
    int a = act_i(e.act, e.act_m, e.act_n, acc);
    int s;
    if (e.ncs_on) s = (int)((float)a + eltw * e.ncs);
    else s = a + (int)eltw;
    int ea = act_i(e.eltw_act, e.eltw_m, e.eltw_n, s);
    if (e.eltw_calib) {
        float o = (float)ea * e.eltw_calib[f];
        if (!out_fp) o = round_sel(o, e.round_even);
        ea = (int)o;
    }
    EpiOut r;
    r.f = (float)ea;
    r.i = ea;
    if (e.out_dt == CLDNN_HIP_S8) r.i = ea < -128 ? -128 : (ea > 127 ? 127 : ea);
    else if (e.out_dt == CLDNN_HIP_U8) r.i = ea < 0 ? 0 : (ea > 255 ? 255 : ea);
    return r;
}

__device__ __forceinline__ void store_out(void* out, int dt, int64_t i, const EpiOut& v)
{
    switch (dt) {
    case CLDNN_HIP_S8: ((int8_t*)out)[i] = (int8_t)v.i; break;
    case CLDNN_HIP_U8: ((uint8_t*)out)[i] = (uint8_t)v.i; break;
    case CLDNN_HIP_I32: ((int32_t*)out)[i] = v.i; break;
    default: ((float*)out)[i] = v.f; break;
    }
}

}  // namespace chip
