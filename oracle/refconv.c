/*
 * refconv -- CPU oracle (test infrastructure; see refconv.h for scope and citations).
 *
 * Arithmetic modes, selected exactly as the reference kernel's preprocessor does
 * (fused_conv_eltwise_gpu_ref.cl:18-48):
 *   MODE_Q    quantisation / calibration / output factor present:
 *             int32 accumulator, float epilogue.
 *   MODE_FINT fused form on int8 data with none of those: int32 accumulator,
 *             int activation, float only for the final eltwise calibration.
 *   MODE_NAT  otherwise: accumulator and activation have the INPUT element
 *             type (char wraps modulo 256, float accumulates in tap order).
 *
 * Build with -ffp-contract=off: the epilogue is a chain of separately rounded
 * float operations.
 */
#include "refconv.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { MODE_Q = 0, MODE_FINT = 1, MODE_NAT = 2 };

int rc_threads_available(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* sliding_window_utils.h:113-126 -- (in + 2*pad - ((k-1)*dil+1)) / stride + 1, degenerate -> 1 */
int rc_out_extent(int in, int pad, int filt, int dil, int stride)
{
    int wnd = (filt - 1) * dil + 1;
    int span = in + 2 * pad;
    if (wnd > span) return 1;
    return (span - wnd) / stride + 1;
}

void rc_dense_bfyx(rc_pitch* p, int F, int H, int W)
{
    p->off = 0;
    p->px = 1;
    p->py = W;
    p->pf = (int64_t)W * H;
    p->pb = (int64_t)W * H * F;
}

/* OpenCL round(): nearest, halfway cases away from zero (fused_conv_eltwise_gpu_ref.cl:33). */
float rc_round_half_away(float x)
{
    return roundf(x);
}

/*
 * The HIP epilogue rounds with trunc(x + copysign(0.49999997f, x)) (0.49999997f is the largest float
 * below one half).  Count the finite floats for which that differs from roundf: must be zero.
 */
long rc_count_round_trick_mismatches(void)
{
    long bad = 0;
#ifdef _OPENMP
#pragma omp parallel for reduction(+ : bad) schedule(static)
#endif
    for (int64_t u = 0; u < ((int64_t)1 << 32); ++u) {
        uint32_t b = (uint32_t)u;
        float x;
        memcpy(&x, &b, 4);
        if (!(x == x) || isinf(x)) continue;
        if (roundf(x) != truncf(x + copysignf(0.49999997f, x))) ++bad;
    }
    return bad;
}

static float rnd(const rc_desc* d, float x)
{
    return d->round_even ? nearbyintf(x) : roundf(x);
}

/* jitter.cpp:373-396, float instantiation (fmax/fmin) */
static float act_f(int act, float m, float n, float x)
{
    switch (act) {
    case RC_ACT_RELU: return fmaxf(0.0f, x);
    case RC_ACT_RELU_SLOPE:
        if (isinf(m)) return x >= 0.0f ? x : -m;
        return fmaxf(x, 0.0f) + (m * fminf(x, 0.0f));
    case RC_ACT_CLAMP: return fmaxf(m, fminf(n, x));
    default: return x;
    }
}

/* same formulas instantiated for int (convert_int of the float parameters truncates) */
static int act_i(int act, float m, float n, int x)
{
    switch (act) {
    case RC_ACT_RELU: return x > 0 ? x : 0;
    case RC_ACT_RELU_SLOPE: {
        int s = (int)m;
        return (x > 0 ? x : 0) + s * (x < 0 ? x : 0);
    }
    case RC_ACT_CLAMP: {
        int lo = (int)m;
        float t = (float)x < n ? (float)x : n; /* min(n, input) */
        int ti = (int)t;
        return ti > lo ? ti : lo;
    }
    default: return x;
    }
}

/* same formulas instantiated for char */
static signed char act_c(int act, float m, float n, signed char x)
{
    (void)n;
    switch (act) {
    case RC_ACT_RELU: return x > 0 ? x : 0;
    case RC_ACT_RELU_SLOPE: {
        signed char s = (signed char)(int)m;
        return (signed char)((x > 0 ? x : 0) + s * (x < 0 ? x : 0));
    }
    default: return x;
    }
}

static double load_val(const void* p, int dt, int64_t i)
{
    switch (dt) {
    case RC_S8: return ((const int8_t*)p)[i];
    case RC_U8: return ((const uint8_t*)p)[i];
    case RC_I32: return ((const int32_t*)p)[i];
    default: return ((const float*)p)[i];
    }
}

/* convert_T_sat for integer targets, plain conversion for float (jitter.cpp:477-560) */
static double store_sat(void* out, int dt, int64_t i, double v, int v_is_float)
{
    switch (dt) {
    case RC_S8: {
        double c = v;
        if (v_is_float && isnan(v)) c = 0;
        if (c > 127) c = 127;
        if (c < -128) c = -128;
        int8_t r = (int8_t)c; /* v is already integral or truncation toward zero applies */
        if (out) ((int8_t*)out)[i] = r;
        return r;
    }
    case RC_U8: {
        double c = v;
        if (v_is_float && isnan(v)) c = 0;
        if (c > 255) c = 255;
        if (c < 0) c = 0;
        uint8_t r = (uint8_t)c;
        if (out) ((uint8_t*)out)[i] = r;
        return r;
    }
    case RC_I32: {
        double c = v;
        if (c > 2147483647.0) c = 2147483647.0;
        if (c < -2147483648.0) c = -2147483648.0;
        int32_t r = (int32_t)c;
        if (out) ((int32_t*)out)[i] = r;
        return r;
    }
    default: {
        float r = (float)v;
        if (out) ((float*)out)[i] = r;
        return r;
    }
    }
}

static int is_int8(int dt) { return dt == RC_S8 || dt == RC_U8; }

static int pick_mode(const rc_desc* d)
{
    if (d->fused) {
        /* fused_conv_eltwise_kernel_base.cpp:141-154: CALIBRATION_TERM / O_QF only exist under quantisation */
        if (d->has_wqf) return MODE_Q;
        if (is_int8(d->in_dt) || is_int8(d->out_dt) || is_int8(d->eltw_dt)) return MODE_FINT;
        return MODE_NAT;
    }
    /* convolution_kernel_base.cpp:66-100 */
    if (d->has_wqf || d->has_calib || d->oqf != 1.0f) return MODE_Q;
    return MODE_NAT;
}

/* float-side epilogue after the int32 accumulator (bias NOT yet added) */
static double epilogue_q(const rc_desc* d, int32_t acc, int f, const void* bias, const float* wqf,
                         const float* calib, double eltw_val, const float* eltw_calib, void* out, int64_t oi)
{
    /* convolution_kernel_ref.cpp:89-91: f32 bias under quantisation is added after dequantisation
       (plain convolution only; the fused host class never sets the flag) */
    int bias_after = (!d->fused) && d->has_wqf && bias && d->bias_dt == RC_F32;
    int calib_on = d->fused ? (d->has_wqf && d->has_calib) : d->has_calib;
    int oqf_on = d->fused ? 1 : (d->oqf != 1.0f);
    int out_fp = d->out_dt == RC_F32;

    if (bias && !bias_after) {
        int32_t bv = d->bias_dt == RC_F32 ? (int32_t)((const float*)bias)[f] : ((const int32_t*)bias)[f];
        acc = (int32_t)((uint32_t)acc + (uint32_t)bv);
    }
    float deq = (float)acc;
    if (d->has_wqf) {
        deq = deq * wqf[f];
        deq = deq * d->iqf;
    }
    if (bias_after) deq = deq + ((const float*)bias)[f];
    float a = act_f(d->act, d->act_m, d->act_n, deq);
    float cal = a;
    if (calib_on) cal = a * calib[f];
    else if (oqf_on) cal = a * d->oqf;

    if (!d->fused) {
        if (!out_fp) cal = rnd(d, cal);
        return store_sat(out, d->out_dt, oi, cal, 1);
    }
    cal = rnd(d, cal); /* the fused form rounds the conv result even for float output (.cl:27-34) */
    float e;
    if (d->non_conv_scale != 1.0f) e = (float)eltw_val * d->non_conv_scale;
    else e = (float)eltw_val;
    float s = cal + e;
    float ea = act_f(d->eltw_act, d->eltw_m, d->eltw_n, s);
    float o = ea;
    if (d->has_eltw_calib) o = ea * eltw_calib[f];
    if (!out_fp) o = rnd(d, o);
    return store_sat(out, d->out_dt, oi, o, 1);
}

/* quantized fully_connected (see rc_desc.fc) */
static double epilogue_fc_q(const rc_desc* d, int32_t acc, int f, const void* bias, const float* wqf, const float* calib,
                            void* out, int64_t oi)
{
    int32_t v = acc;
    if (bias) {
        float bv = d->bias_dt == RC_F32 ? ((const float*)bias)[f] : (float)((const int32_t*)bias)[f];
        float x = (float)acc * wqf[f];
        x = x * d->iqf;
        x = x + bv;
        x = x * (d->has_calib ? calib[f] : d->oqf);
        v = (int32_t)(signed char)(int32_t)rnd(d, x); /* (UNIT_TYPE)round(...) */
    }
    signed char c = (signed char)v; /* convert_char: the low byte */
    c = act_c(d->act, d->act_m, d->act_n, c);
    return store_sat(out, d->out_dt, oi, c, 0);
}

/* MODE_FINT: int activation, float only in the last calibration (.cl:35-42, 199-232) */
static double epilogue_fint(const rc_desc* d, int32_t acc, int f, const void* bias, double eltw_val,
                            const float* eltw_calib, void* out, int64_t oi)
{
    if (bias) {
        int32_t bv = d->bias_dt == RC_F32 ? (int32_t)((const float*)bias)[f] : ((const int32_t*)bias)[f];
        acc = (int32_t)((uint32_t)acc + (uint32_t)bv);
    }
    int a = act_i(d->act, d->act_m, d->act_n, acc);
    int s;
    if (d->non_conv_scale != 1.0f) {
        float e = (float)eltw_val * d->non_conv_scale;
        s = (int)((float)a + e); /* int + float -> float, stored to an int */
    } else {
        s = a + (int)eltw_val; /* convert_int_sat of an int8/int32 value is the value */
    }
    int ea = act_i(d->eltw_act, d->eltw_m, d->eltw_n, s);
    if (d->has_eltw_calib) {
        float o = (float)ea * eltw_calib[f];
        if (d->out_dt != RC_F32) o = rnd(d, o);
        ea = (int)o; /* the kernel assigns the rounded float back to its int variable */
        if (d->out_dt == RC_F32) return store_sat(out, d->out_dt, oi, (double)(int)o, 0);
    }
    return store_sat(out, d->out_dt, oi, ea, 0);
}

double rc_epilogue(const rc_desc* d, int32_t acc, int f, const void* bias, const float* wqf,
                   const float* calib, double eltw_val, const float* eltw_calib)
{
    int mode = pick_mode(d);
    if (mode == MODE_Q) return epilogue_q(d, acc, f, bias, wqf, calib, eltw_val, eltw_calib, NULL, 0);
    if (mode == MODE_FINT) return epilogue_fint(d, acc, f, bias, eltw_val, eltw_calib, NULL, 0);
    return NAN;
}

/* valid output range [lo, hi) along one axis for tap offset t = k*dil - pad */
static void valid_range(int out_n, int in_n, int stride, int t, int* lo, int* hi)
{
    /* need 0 <= o*stride + t < in_n */
    int l = 0, h = out_n;
    if (t < 0) l = (-t + stride - 1) / stride;
    /* o*stride + t <= in_n - 1  ->  o <= (in_n - 1 - t) / stride */
    if (in_n - 1 - t < 0) h = 0;
    else {
        int m = (in_n - 1 - t) / stride + 1;
        if (m < h) h = m;
    }
    if (l > h) l = h;
    *lo = l;
    *hi = h;
}

/*
 * Integer accumulation of one (b, f) output plane.  Integer addition is exact
 * and order-free, so the loop is arranged plane-at-a-time (tap outermost) for
 * speed; every in-range tap of fused_conv_eltwise_gpu_ref.cl:113-146 is
 * visited exactly once and out-of-range taps are skipped.
 */
static void acc_plane_int(const rc_desc* d, const void* in, const int8_t* w, int b, int f, int32_t* acc)
{
    int ifm_g = d->IFM / d->groups;
    int ofm_g = d->OFM / d->groups;
    int g = f / ofm_g;
    int OH = d->OH, OW = d->OW;
    memset(acc, 0, sizeof(int32_t) * (size_t)OH * OW);
    for (int k = 0; k < ifm_g; ++k) {
        int64_t in_base = d->in_p.off + (int64_t)b * d->in_p.pb + (int64_t)(g * ifm_g + k) * d->in_p.pf;
        for (int j = 0; j < d->FY; ++j) {
            int ylo, yhi;
            valid_range(OH, d->IH, d->sy, j * d->dy - d->pad_y, &ylo, &yhi);
            for (int i = 0; i < d->FX; ++i) {
                int xlo, xhi;
                valid_range(OW, d->IW, d->sx, i * d->dx - d->pad_x, &xlo, &xhi);
                int32_t wv = w[(((int64_t)f * ifm_g + k) * d->FY + j) * d->FX + i];
                if (wv == 0) continue;
                for (int y = ylo; y < yhi; ++y) {
                    int iy = y * d->sy - d->pad_y + j * d->dy;
                    int64_t row = in_base + (int64_t)iy * d->in_p.py
                                  + (int64_t)(i * d->dx - d->pad_x) * d->in_p.px;
                    int32_t* arow = acc + (size_t)y * OW;
                    int64_t step = (int64_t)d->sx * d->in_p.px;
                    if (d->in_dt == RC_U8) {
                        const uint8_t* p = (const uint8_t*)in + row;
                        for (int x = xlo; x < xhi; ++x)
                            arow[x] = (int32_t)((uint32_t)arow[x] + (uint32_t)((int32_t)p[x * step] * wv));
                    } else {
                        const int8_t* p = (const int8_t*)in + row;
                        for (int x = xlo; x < xhi; ++x)
                            arow[x] = (int32_t)((uint32_t)arow[x] + (uint32_t)((int32_t)p[x * step] * wv));
                    }
                }
            }
        }
    }
}

/* MODE_NAT, float data: per-pixel accumulation in the reference's k -> j -> i order */
static void acc_plane_f32(const rc_desc* d, const float* in, const float* w, int b, int f, float* acc)
{
    int ifm_g = d->IFM / d->groups;
    int ofm_g = d->OFM / d->groups;
    int g = f / ofm_g;
    int OH = d->OH, OW = d->OW;
    for (int i = 0; i < OH * OW; ++i) acc[i] = 0.0f;
    for (int k = 0; k < ifm_g; ++k) {
        int64_t in_base = d->in_p.off + (int64_t)b * d->in_p.pb + (int64_t)(g * ifm_g + k) * d->in_p.pf;
        for (int j = 0; j < d->FY; ++j) {
            int ylo, yhi;
            valid_range(OH, d->IH, d->sy, j * d->dy - d->pad_y, &ylo, &yhi);
            for (int i = 0; i < d->FX; ++i) {
                int xlo, xhi;
                valid_range(OW, d->IW, d->sx, i * d->dx - d->pad_x, &xlo, &xhi);
                float wv = w[(((int64_t)f * ifm_g + k) * d->FY + j) * d->FX + i];
                for (int y = ylo; y < yhi; ++y) {
                    int iy = y * d->sy - d->pad_y + j * d->dy;
                    for (int x = xlo; x < xhi; ++x) {
                        int ix = x * d->sx - d->pad_x + i * d->dx;
                        float v = in[in_base + (int64_t)iy * d->in_p.py + (int64_t)ix * d->in_p.px];
                        acc[(size_t)y * OW + x] = acc[(size_t)y * OW + x] + v * wv;
                    }
                }
            }
        }
    }
}

int rc_conv(const rc_desc* d, const void* in, const void* weights, const void* bias, const float* wqf,
            const float* calib, const void* eltw, const float* eltw_calib, void* out, int32_t* acc_out,
            int nthreads)
{
    int mode = pick_mode(d);
    if (d->groups < 1 || d->IFM % d->groups || d->OFM % d->groups) return -1;
    if (mode != MODE_NAT && d->w_dt != RC_S8 && !(d->in_dt == RC_F32 && d->w_dt == RC_F32)) return -1;
    if (mode == MODE_NAT && d->in_dt == RC_F32 && d->w_dt != RC_F32) return -1;
    if (mode == MODE_NAT && is_int8(d->in_dt) && d->w_dt != RC_S8) return -1;
    if (d->fused && !eltw) return -1;
    if (nthreads < 1) nthreads = 1;

    const int OH = d->OH, OW = d->OW;
    const int64_t planes = (int64_t)d->B * d->OFM;
    int rc = 0;

#ifdef _OPENMP
#pragma omp parallel num_threads(nthreads)
#endif
    {
        int32_t* acc = (int32_t*)malloc(sizeof(int32_t) * (size_t)OH * OW + 64);
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 1)
#endif
        for (int64_t pl = 0; pl < planes; ++pl) {
            int b = (int)(pl / d->OFM), f = (int)(pl % d->OFM);
            int64_t obase = d->out_p.off + (int64_t)b * d->out_p.pb + (int64_t)f * d->out_p.pf;
            int64_t ebase = d->eltw_p.off + (int64_t)b * d->eltw_p.pb + (int64_t)f * d->eltw_p.pf;

            if (mode == MODE_NAT && d->in_dt == RC_F32) {
                float* facc = (float*)acc;
                acc_plane_f32(d, (const float*)in, (const float*)weights, b, f, facc);
                for (int y = 0; y < OH; ++y)
                    for (int x = 0; x < OW; ++x) {
                        float v = facc[(size_t)y * OW + x];
                        if (bias) v = v + (float)load_val(bias, d->bias_dt, f);
                        v = act_f(d->act, d->act_m, d->act_n, v);
                        int64_t oi = obase + (int64_t)y * d->out_p.py + (int64_t)x * d->out_p.px;
                        if (d->fused) {
                            float e = (float)load_val(eltw, d->eltw_dt,
                                                      ebase + (int64_t)y * d->esy * d->eltw_p.py
                                                          + (int64_t)x * d->esx * d->eltw_p.px);
                            if (d->non_conv_scale != 1.0f) e = e * d->non_conv_scale;
                            float s = act_f(d->eltw_act, d->eltw_m, d->eltw_n, v + e);
                            if (d->has_eltw_calib) s = s * eltw_calib[f];
                            if (d->out_dt != RC_F32) s = rnd(d, s);
                            store_sat(out, d->out_dt, oi, s, 1);
                        } else {
                            store_sat(out, d->out_dt, oi, v, 1);
                        }
                    }
                continue;
            }

            if (d->in_dt == RC_F32) {
                /* quantised form on float data: operands go through convert_int (truncation), .cl:21,140 */
                int ifm_g = d->IFM / d->groups, g = f / (d->OFM / d->groups);
                for (int y = 0; y < OH; ++y)
                    for (int x = 0; x < OW; ++x) {
                        int32_t a = 0;
                        for (int k = 0; k < ifm_g; ++k)
                            for (int j = 0; j < d->FY; ++j)
                                for (int i = 0; i < d->FX; ++i) {
                                    int iy = y * d->sy - d->pad_y + j * d->dy, ix = x * d->sx - d->pad_x + i * d->dx;
                                    if (iy < 0 || iy >= d->IH || ix < 0 || ix >= d->IW) continue;
                                    float v = ((const float*)in)[d->in_p.off + (int64_t)b * d->in_p.pb
                                                                 + (int64_t)(g * ifm_g + k) * d->in_p.pf
                                                                 + (int64_t)iy * d->in_p.py + (int64_t)ix * d->in_p.px];
                                    float wv = ((const float*)weights)[(((int64_t)f * ifm_g + k) * d->FY + j) * d->FX + i];
                                    a += (int32_t)v * (int32_t)wv;
                                }
                        acc[(size_t)y * OW + x] = a;
                    }
            } else {
                acc_plane_int(d, in, (const int8_t*)weights, b, f, acc);
            }

            if (acc_out) memcpy(acc_out + (size_t)pl * OH * OW, acc, sizeof(int32_t) * (size_t)OH * OW);

            for (int y = 0; y < OH; ++y)
                for (int x = 0; x < OW; ++x) {
                    int32_t a = acc[(size_t)y * OW + x];
                    int64_t oi = obase + (int64_t)y * d->out_p.py + (int64_t)x * d->out_p.px;
                    double ev = 0;
                    if (d->fused)
                        ev = load_val(eltw, d->eltw_dt,
                                      ebase + (int64_t)y * d->esy * d->eltw_p.py + (int64_t)x * d->esx * d->eltw_p.px);
                    if (mode == MODE_Q && d->fc) {
                        epilogue_fc_q(d, a, f, bias, wqf, calib, out, oi);
                    } else if (mode == MODE_Q) {
                        epilogue_q(d, a, f, bias, wqf, calib, ev, eltw_calib, out, oi);
                    } else if (mode == MODE_FINT) {
                        epilogue_fint(d, a, f, bias, ev, eltw_calib, out, oi);
                    } else {
                        /* MODE_NAT on int8: accumulator, bias and activation all in the input's char type */
                        signed char c = (signed char)a; /* sum of products wrapped modulo 256 */
                        if (bias) {
                            double bv = load_val(bias, d->bias_dt, f);
                            c = (signed char)(c + (signed char)(int)bv);
                        }
                        c = act_c(d->act, d->act_m, d->act_n, c);
                        store_sat(out, d->out_dt, oi, c, 0);
                    }
                }
        }
        free(acc);
    }
    return rc;
}

/* ------------------------------------------------------------------------------------------------ pooling */
int rc_pool_out_extent(int in, int pad, int size, int stride)
{
    int off = -pad; /* the primitive's input_offset */
    int extend = size > stride ? size : stride;
    int once = 2 * off + extend <= in + stride - 1 ? (in - 2 * off - extend + stride - 1) / stride + 1 : 1;
    int any = off <= in - 1 ? (in - off - 1) / stride + 1 : 1;
    return once < any ? once : any;
}

int rc_pool(const rc_pool_desc* d, const void* in, void* out)
{
    if (!(d->dt == RC_S8 || d->dt == RC_U8 || d->dt == RC_F32) || d->mode < 0 || d->mode > 1) return -1;
    for (int b = 0; b < d->B; ++b)
        for (int f = 0; f < d->F; ++f) {
            int64_t ib = ((int64_t)b * d->F + f) * d->IH * d->IW, ob = ((int64_t)b * d->F + f) * d->OH * d->OW;
            for (int y = 0; y < d->OH; ++y)
                for (int x = 0; x < d->OW; ++x) {
                    int oy = y * d->sy - d->pad_y, ox = x * d->sx - d->pad_x;
                    if (oy + d->ky < 0 || oy >= d->IH || ox + d->kx < 0 || ox >= d->IW) continue;
                    int valid = 0;
                    int ri = d->mode == 0 ? -128 : 0;
                    float rf = d->mode == 0 ? -3.402823466e+38f : 0.0f;
                    for (int j = 0; j < d->ky; ++j) {
                        int iy = oy + j;
                        if (iy < 0 || iy >= d->IH) continue;
                        for (int i = 0; i < d->kx; ++i) {
                            int ix = ox + i;
                            if (ix < 0 || ix >= d->IW) continue;
                            int64_t at = ib + (int64_t)iy * d->IW + ix;
                            if (d->dt == RC_F32) {
                                float v = ((const float*)in)[at];
                                rf = d->mode == 0 ? (v > rf ? v : rf) : rf + v;
                            } else {
                                int v = d->dt == RC_U8 ? (int)((const uint8_t*)in)[at] : (int)((const int8_t*)in)[at];
                                ri = d->mode == 0 ? (v > ri ? v : ri) : ri + v;
                            }
                            ++valid;
                        }
                    }
                    int n = d->ky * d->kx;
                    if (d->divider == 1) n = valid > 0 ? valid : 1;
                    if (d->divider == 2) {
                        int hend = oy + d->ky < d->IH + d->pad_y ? oy + d->ky : d->IH + d->pad_y;
                        int wend = ox + d->kx < d->IW + d->pad_x ? ox + d->kx : d->IW + d->pad_x;
                        n = (hend - oy) * (wend - ox);
                        if (n < 1) n = 1;
                    }
                    int64_t oi = ob + (int64_t)y * d->OW + x;
                    if (d->dt == RC_F32) {
                        ((float*)out)[oi] = d->mode == 0 ? rf : rf / (float)n;
                    } else {
                        if (d->mode == 1) ri = (int)rc_round_half_away((float)ri / (float)n);
                        if (d->dt == RC_U8) ((uint8_t*)out)[oi] = (uint8_t)ri;
                        else ((int8_t*)out)[oi] = (int8_t)ri;
                    }
                }
        }
    return 0;
}
