/*
 * refconv -- CPU oracle for the quantized convolution path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the arithmetic
 * of the reference semantic kernel, used as the checker by tests/, by
 * __graft_entry__.smoke() and by bench.py's cpu_baseline leg.  Nothing in the
 * product library links, loads or calls it.
 *
 * What it follows (paths relative to the reference tree):
 *   kernel_selector/core/cl_kernels/fused_conv_eltwise_gpu_ref.cl:18-63   arithmetic-type selection
 *   kernel_selector/core/cl_kernels/fused_conv_eltwise_gpu_ref.cl:93-198  convolution + epilogue
 *   kernel_selector/core/cl_kernels/fused_conv_eltwise_gpu_ref.cl:199-233 eltwise tail
 *   kernel_selector/core/common/jitter.cpp:363-396                        activation formulas
 *   kernel_selector/core/common/jitter.cpp:462-583                        which converts saturate
 *   kernel_selector/core/actual_kernels/convolution/convolution_kernel_ref.cpp:64-94  f32 bias added after dequantisation
 *   kernel_selector/core/actual_kernels/convolution/convolution_kernel_base.cpp:51-124 QUANTIZATION/CALIBRATION/O_QF flags
 *   kernel_selector/core/actual_kernels/fused_conv_eltwise/fused_conv_eltwise_kernel_base.cpp:122-176 fused flags
 *   src/include/sliding_window_utils.h:90-129                             output size
 *   tests/test_cases/convolution_gpu_test.cpp:5582-5705                   host loop skeleton
 *
 * Parity pinning: every function here is pinned by the reference's own
 * known-answer tables (tests/golden/conv_kat.json, taken from
 * tests/test_cases/convolution_gpu_test.cpp and
 * tests/test_cases/fused_conv_eltwise_gpu_test.cpp) and by closed-form /
 * brute-force checks in tests/test_oracle.py.  The reference itself cannot be
 * executed (it needs an Intel OpenCL device), so there is no oracle/_ref build.
 */
#ifndef REFCONV_H
#define REFCONV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { RC_S8 = 0, RC_U8 = 1, RC_I32 = 2, RC_F32 = 3, RC_NONE = -1 };

/* activation codes (subset of cldnn_activation_func that the path uses) */
enum { RC_ACT_NONE = 0, RC_ACT_RELU = 1, RC_ACT_RELU_SLOPE = 2, RC_ACT_CLAMP = 3 };

/* strides are in elements; offset is the element index of (b=0,f=0,y=0,x=0) */
typedef struct {
    int64_t off, pb, pf, py, px;
} rc_pitch;

typedef struct {
    /* data types */
    int in_dt, w_dt, bias_dt, out_dt, eltw_dt;
    /* logical sizes */
    int B, IFM, IH, IW;          /* IFM = total input features (all groups) */
    int OFM, OH, OW;             /* OFM = total output features (all groups) */
    int FY, FX;
    int sy, sx, dy, dx;
    int pad_y, pad_x;            /* = max(-input_offset, 0) */
    int groups;
    /* quantisation */
    int has_wqf;                 /* weights_quantization_factors given  -> QUANTIZATION_TERM */
    int has_calib;               /* output_calibration_factors given    -> CALIBRATION_TERM */
    float iqf;                   /* input_quantization_factor  */
    float oqf;                   /* output_quantization_factor */
    /* conv activation */
    int act; float act_m, act_n;
    /* fused_conv_eltwise part */
    int fused;
    float non_conv_scale;
    int eltw_act; float eltw_m, eltw_n;
    int has_eltw_calib;
    int esy, esx;                /* eltwise input stride */
    /* memory pitches */
    rc_pitch in_p, out_p, eltw_p;
    /* 1 = round half to even instead of half away from zero (documented variant, not the reference) */
    int round_even;
    /* 1 = the epilogue of the reference's quantized fully_connected kernels
       (fully_connected_gpu_bfyx_ref.cl:63-84, fully_connected_gpu_MMAD.cl:103-118): with a bias
       (char)round(((float)acc * wqf * iqf + bias) * (calib or oqf)), without one the raw accumulator; converted to
       char by dropping the upper bits; the activation acts on that char */
    int fc;
} rc_desc;

/* Output extent along one axis (sliding_window_utils.h:113-126; degenerate value 1). */
int rc_out_extent(int in, int pad, int filt, int dil, int stride);

/* Fill *p with dense bfyx pitches for (F,H,W). */
void rc_dense_bfyx(rc_pitch* p, int F, int H, int W);

/*
 * Full reference convolution.  weights: [OFM][IFM/groups][FY][FX] dense.
 * bias/wqf/calib/eltw_calib: [OFM] or NULL.  acc_out (optional): dense
 * [B][OFM][OH][OW] int32 accumulators before the bias is added (only written
 * in the integer-accumulator modes).  Returns 0, or -1 on an unsupported
 * combination.  Uses OpenMP over (b, f) when nthreads > 1.
 */
int rc_conv(const rc_desc* d, const void* in, const void* weights, const void* bias,
            const float* wqf, const float* calib, const void* eltw, const float* eltw_calib,
            void* out, int32_t* acc_out, int nthreads);

/*
 * Epilogue alone for the integer-accumulator modes: takes the int32
 * accumulator (without bias) of one output element of feature f and returns
 * the stored value widened to double (exact for s8/u8/f32).
 */
double rc_epilogue(const rc_desc* d, int32_t acc, int f, const void* bias, const float* wqf,
                   const float* calib, double eltw_val, const float* eltw_calib);

/*
 * Pooling over dense bfyx tensors (the layers between the convolutions of an int8 network).  Follows
 * kernel_selector/core/cl_kernels/pooling_gpu_int8_ref.cl:15-140 for s8 / u8 (int accumulator starting at CHAR_MIN
 * for the maximum, average = round(sum / count) half away from zero) and pooling_gpu_ref.cl for f32 (float
 * accumulator, plain division); taps outside the input are skipped, a window wholly outside leaves the output as it
 * is.  mode: 0 max, 1 average.  divider: 0 window size, 1 taps inside the input, 2 window clipped to input + padding
 * (src/gpu/pooling_gpu.cpp:36-52,100-108).
 */
typedef struct {
    int dt;
    int B, F, IH, IW, OH, OW;
    int ky, kx, sy, sx, pad_y, pad_x;
    int mode, divider;
} rc_pool_desc;
int rc_pool(const rc_pool_desc* d, const void* in, void* out);
/* Output extent of a pooling window along one axis (sliding_window_utils.h:135-186, swor_mode::exceed_once_data;
 * src/pooling.cpp:110-116): min(the last window may overhang the padded input once, every window starts inside
 * input + leading padding); degenerate value 1. */
int rc_pool_out_extent(int in, int pad, int size, int stride);

/* Helpers exposed for tests. */
float rc_round_half_away(float x);
int   rc_threads_available(void);
long  rc_count_round_trick_mismatches(void);

#ifdef __cplusplus
}
#endif
#endif
