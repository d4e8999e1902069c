/*
 * cldnn_hip.h -- thin C-ABI HIP layer underneath the clDNN-compatible host
 * library.  It stands where the reference's OpenCL "gpu toolkit" stands
 * (engine, buffers, events, kernel enqueue) and additionally exposes the
 * quantized convolution as a directly callable operator.
 *
 * Plain C: opaque handles, pointers and sizes only.  Every function returns
 * a cldnn_hip_status (0 = success) unless stated otherwise; the message of
 * the last failure on the calling thread is available from
 * cldnn_hip_last_error() (same contract as cldnn_get_last_error_message,
 * reference src/cldnn.cpp:27-33).
 *
 * The library never falls back to host computation: without a usable HIP
 * device every compute entry point fails with CLDNN_HIP_DEVICE_ERROR.
 */
#ifndef CLDNN_HIP_H
#define CLDNN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t cldnn_hip_status;
/* values mirror reference api/C/cldnn.h:70-79 */
#define CLDNN_HIP_SUCCESS 0
#define CLDNN_HIP_ERROR -1
#define CLDNN_HIP_INVALID_ARG -2
#define CLDNN_HIP_OUT_OF_RESOURCES -3
#define CLDNN_HIP_DEVICE_ERROR -4
#define CLDNN_HIP_UNSUPPORTED_SIZE -5
#define CLDNN_HIP_UNSUPPORTED_FORMAT -6
#define CLDNN_HIP_DIMENSION_MISMATCH -7

typedef struct cldnn_hip_engine_s* cldnn_hip_engine;
typedef struct cldnn_hip_buffer_s* cldnn_hip_buffer;
typedef struct cldnn_hip_event_s* cldnn_hip_event;
typedef struct cldnn_hip_conv_s* cldnn_hip_conv;
typedef struct cldnn_hip_conv_chain_s* cldnn_hip_conv_chain;

const char* cldnn_hip_last_error(void);

/* ------------------------------------------------------------------ engine
 * replaces gpu_toolkit construction / device pick
 * (reference src/gpu/ocl_toolkit.cpp:104-151, src/gpu/ocl_builder.cpp:79-160)
 * and engine_info (reference src/gpu/engine_info.cpp, api/C/cldnn.h:167-188). */
typedef struct {
    uint32_t cores_count;        /* compute units */
    uint32_t core_frequency;     /* MHz */
    uint64_t max_work_group_size;
    uint64_t max_local_mem_size; /* LDS bytes per workgroup */
    uint64_t max_global_mem_size;
    uint64_t max_alloc_mem_size;
    uint32_t wavefront_size;
    uint32_t xcd_count;          /* accelerator dies (each with its own L2) */
    char name[64];
    char arch[32];               /* e.g. "gfx950" */
} cldnn_hip_engine_info;

uint32_t cldnn_hip_device_count(void);
cldnn_hip_status cldnn_hip_engine_create(uint32_t device, uint32_t enable_profiling, cldnn_hip_engine* out);
cldnn_hip_status cldnn_hip_engine_retain(cldnn_hip_engine e);
cldnn_hip_status cldnn_hip_engine_release(cldnn_hip_engine e);
cldnn_hip_status cldnn_hip_engine_get_info(cldnn_hip_engine e, cldnn_hip_engine_info* info);
/* the engine's HIP stream as a void* (hipStream_t); all work of an engine is ordered on it */
void* cldnn_hip_engine_stream(cldnn_hip_engine e);
/* replaces gpu_toolkit::flush / finish (reference src/gpu/ocl_toolkit.cpp:291-300) */
cldnn_hip_status cldnn_hip_engine_flush(cldnn_hip_engine e);
cldnn_hip_status cldnn_hip_engine_finish(cldnn_hip_engine e);
/* bytes currently / at most allocated through this engine (reference src/include/engine_impl.h:123-124) */
int64_t cldnn_hip_engine_used_memory(cldnn_hip_engine e);
int64_t cldnn_hip_engine_max_used_memory(cldnn_hip_engine e);

/* ------------------------------------------------------------------ buffers
 * replaces gpu_buffer (reference src/gpu/memory_gpu.cpp:37-90): zero-filled at
 * allocation; lock() hands out a host pointer valid for read AND write,
 * reference-counted; the first lock copies device -> pinned shadow, the last
 * unlock copies the shadow back to the device. */
cldnn_hip_status cldnn_hip_buffer_alloc(cldnn_hip_engine e, size_t bytes, cldnn_hip_buffer* out);
cldnn_hip_status cldnn_hip_buffer_retain(cldnn_hip_buffer b);
cldnn_hip_status cldnn_hip_buffer_release(cldnn_hip_buffer b);
void* cldnn_hip_buffer_lock(cldnn_hip_buffer b);     /* NULL on failure */
cldnn_hip_status cldnn_hip_buffer_unlock(cldnn_hip_buffer b);
/* gpu_buffer::fill (reference src/gpu/memory_gpu.cpp:87-90) */
cldnn_hip_status cldnn_hip_buffer_fill(cldnn_hip_buffer b, uint8_t pattern);
void* cldnn_hip_buffer_device_ptr(cldnn_hip_buffer b);
size_t cldnn_hip_buffer_size(cldnn_hip_buffer b);
/* direct copies ordered on the engine stream (blocking) */
cldnn_hip_status cldnn_hip_buffer_write(cldnn_hip_buffer b, size_t offset, const void* host, size_t bytes);
cldnn_hip_status cldnn_hip_buffer_read(cldnn_hip_buffer b, size_t offset, void* host, size_t bytes);

/* ------------------------------------------------------------------ events
 * replaces base_event / user_event / events_pool
 * (reference src/gpu/ocl_base_event.cpp:23-159, src/gpu/ocl_user_event.cpp, src/gpu/events_pool.h:25-139). */
typedef void (*cldnn_hip_event_handler)(void*);
cldnn_hip_status cldnn_hip_event_create_user(cldnn_hip_engine e, uint32_t set, cldnn_hip_event* out);
/* marker after everything enqueued so far (gpu_toolkit::enqueue_marker, reference src/gpu/ocl_toolkit.cpp:197-230) */
cldnn_hip_status cldnn_hip_event_record(cldnn_hip_engine e, cldnn_hip_event* out);
/* bracket the work enqueued between the two calls; with profiling enabled the event then carries
 * its execution time (reference src/gpu/ocl_toolkit.cpp:170-178 returns such an event per kernel) */
cldnn_hip_status cldnn_hip_event_record_begin(cldnn_hip_engine e, cldnn_hip_event* out);
cldnn_hip_status cldnn_hip_event_record_end(cldnn_hip_event ev);
/* An event for work that will be submitted LATER (reference: an OpenCL command enqueued behind a user event exists, and
 * can be waited for, before that user event is set -- src/gpu/ocl_toolkit.cpp:153-195 with deps).  create_deferred makes
 * the event; record_deferred, called once when the work has been enqueued on the event's engine, records it.  Until then
 * is_set is 0 and wait / add_handler / elapsed_ns block (or call back) only after the recording AND the work are done. */
cldnn_hip_status cldnn_hip_event_create_deferred(cldnn_hip_engine e, cldnn_hip_event* out);
cldnn_hip_status cldnn_hip_event_record_deferred(cldnn_hip_event ev);
cldnn_hip_status cldnn_hip_event_retain(cldnn_hip_event ev);
cldnn_hip_status cldnn_hip_event_release(cldnn_hip_event ev);
cldnn_hip_status cldnn_hip_event_wait(cldnn_hip_event ev);
int32_t cldnn_hip_event_is_set(cldnn_hip_event ev);
int32_t cldnn_hip_event_is_user(cldnn_hip_event ev);
cldnn_hip_status cldnn_hip_event_set(cldnn_hip_event ev);
cldnn_hip_status cldnn_hip_event_add_handler(cldnn_hip_event ev, cldnn_hip_event_handler h, void* param);
/* "executing" interval in ns (reference src/gpu/ocl_base_event.cpp:68-96); 0 when profiling is off */
cldnn_hip_status cldnn_hip_event_elapsed_ns(cldnn_hip_event ev, uint64_t* ns);
/* make the engine stream wait for events before later work (gpu_toolkit::sync_events, reference src/gpu/ocl_toolkit.cpp:313-346).
 * A stream cannot wait for a host flag: for a user event that is not set yet the CALLING THREAD is held until it is.  A
 * caller that must not block looks at cldnn_hip_event_is_user / cldnn_hip_event_is_set first and postpones its
 * submission (libclDNN does: cldnn_execute_network behind an unset user event returns at once and submits from
 * cldnn_hip_event_set). */
cldnn_hip_status cldnn_hip_engine_wait_events(cldnn_hip_engine e, const cldnn_hip_event* evs, size_t n);

/* ------------------------------------------------------------------ tensors */
enum { CLDNN_HIP_S8 = 0, CLDNN_HIP_U8 = 1, CLDNN_HIP_I32 = 2, CLDNN_HIP_F32 = 3, CLDNN_HIP_NO_TYPE = -1 };

enum {
    CLDNN_HIP_FMT_BFYX = 0,
    CLDNN_HIP_FMT_YXFB = 1,
    CLDNN_HIP_FMT_BYXF = 2,
    /* [fs][b][y][x][16 features]: the 16-byte feature slice of one pixel is one lane's
       int8 MFMA K-fragment and one 128-bit load.  Chosen by the layout rule that replaces
       byxf_af32 / fs_bs_yx_bsv4_fsv32 (reference src/layout_optimizer.cpp:187-291,
       kernel_selector/core/cl_kernels/include/fetch.cl:126-196). */
    CLDNN_HIP_FMT_FS_B_YX_FSV16 = 3,
    /* [b][fs][y][x][4 features] (reference fetch.cl:453-476) */
    CLDNN_HIP_FMT_B_FS_YX_FSV4 = 4
};

/* logical size + physical spatial/feature padding (reference api/CPP/layout.hpp:387-433) */
typedef struct {
    int32_t dtype;
    int32_t format;
    int32_t b, f, y, x;
    int32_t pad_lo_b, pad_lo_f, pad_lo_y, pad_lo_x;
    int32_t pad_hi_b, pad_hi_f, pad_hi_y, pad_hi_x;
} cldnn_hip_tensor;

/* bytes a buffer for this tensor must have */
size_t cldnn_hip_tensor_bytes(const cldnn_hip_tensor* t);
/* element index of logical (b,f,y,x) inside the buffer (get_linear_offset, reference api/CPP/layout.hpp:407-433) */
int64_t cldnn_hip_tensor_offset(const cldnn_hip_tensor* t, int32_t b, int32_t f, int32_t y, int32_t x);

/* layout / precision change; replaces the reorder kernels the path needs
 * (reference src/gpu/reorder_gpu.cpp, kernel_selector/core/cl_kernels/reorder_data.cl).
 * f32 -> integer conversions go towards zero like the reference's convert_char (kernel_selector/core/common/jitter.cpp:483)
 * and saturate where OpenCL leaves the result undefined; padding of dst is left untouched. */
cldnn_hip_status cldnn_hip_reorder(cldnn_hip_engine e, const void* src_dev, const cldnn_hip_tensor* src,
                                   void* dst_dev, const cldnn_hip_tensor* dst);

enum { CLDNN_HIP_ACT_NONE = 0, CLDNN_HIP_ACT_RELU = 1, CLDNN_HIP_ACT_RELU_SLOPE = 2, CLDNN_HIP_ACT_CLAMP = 3 };

/* One input of a concatenation copied to its place in the output: the source's element (0, 0, 0, 0) lands at the given
 * logical offset of the destination; any two layouts, same element size (reference
 * kernel_selector/core/cl_kernels/concatenation_gpu_ref.cl:18-46 and src/gpu/concatenation_gpu.cpp:64-90: one kernel per
 * input).  Asynchronous on the engine stream. */
cldnn_hip_status cldnn_hip_copy_region(cldnn_hip_engine e, const void* src_dev, const cldnn_hip_tensor* src, void* dst_dev,
                                       const cldnn_hip_tensor* dst, int32_t offset_b, int32_t offset_f, int32_t offset_y, int32_t offset_x);

/* stand-alone activation and element-wise sum (what the convolution epilogue fuses when it can);
 * replace the reference's activation / eltwise kernels for the cases a convolution topology needs
 * (reference src/gpu/activation_gpu.cpp, src/gpu/eltwise_gpu.cpp,
 *  kernel_selector/core/cl_kernels/generic_eltwise_ref.cl:311-328).
 * activation codes: CLDNN_HIP_ACT_*.  quantized != 0: integer sum, round(sum * factor) with the factor
 * per feature (calib_dev) or per tensor, saturate to int8, then the activation. */
cldnn_hip_status cldnn_hip_activation(cldnn_hip_engine e, const void* src_dev, const cldnn_hip_tensor* src,
                                      void* dst_dev, const cldnn_hip_tensor* dst, int32_t activation, float m, float n);
cldnn_hip_status cldnn_hip_eltwise_sum(cldnn_hip_engine e, const void* a_dev, const cldnn_hip_tensor* a,
                                       const void* b_dev, const cldnn_hip_tensor* b, void* dst_dev,
                                       const cldnn_hip_tensor* dst, int32_t quantized, const float* calib_dev,
                                       float output_quantization_factor, int32_t activation, float m, float n);

/* General element-wise primitive: 2..CLDNN_HIP_ELTWISE_MAX_INPUTS inputs combined left to right,
 * r = op(...op(op(in0, in1), in2)..., inN-1)  (reference src/gpu/eltwise_gpu.cpp:80-140,
 * kernel_selector/core/actual_kernels/eltwise/eltwise_kernel_base.cpp:236-352,
 * kernel_selector/core/cl_kernels/generic_eltwise_ref.cl:106-135 and 311-330).
 * Input i is read at (b % B_i, f % F_i, (y * stride_y[i]) % Y_i, (x * stride_x[i]) % X_i): strides shrink, sizes of
 * one broadcast.  The arithmetic type follows the first input: float data in float; int8 data in the 8-bit type with
 * wrap-around after every step, unless `quantized`: then in int, followed by round(r * factor) (calib_dev[f] or
 * output_quantization_factor), saturation to signed char and the activation.  Integer division and modulo by zero
 * give 0 here (undefined in the reference).  Coefficients multiply the inputs of a float sum. */
enum {
    CLDNN_HIP_ELTWISE_SUM = 0, CLDNN_HIP_ELTWISE_SUB = 1, CLDNN_HIP_ELTWISE_MAX = 2, CLDNN_HIP_ELTWISE_PROD = 3,
    CLDNN_HIP_ELTWISE_DIV = 4, CLDNN_HIP_ELTWISE_MIN = 5, CLDNN_HIP_ELTWISE_POW = 6, CLDNN_HIP_ELTWISE_MOD = 7
};  /* the values of cldnn_eltwise_mode (reference api/C/eltwise.h:33-67); POW for float data only */
#define CLDNN_HIP_ELTWISE_MAX_INPUTS 4
typedef struct {
    int32_t mode;                 /* CLDNN_HIP_ELTWISE_* */
    int32_t n_inputs;
    cldnn_hip_tensor inputs[CLDNN_HIP_ELTWISE_MAX_INPUTS];
    int32_t stride_y[CLDNN_HIP_ELTWISE_MAX_INPUTS], stride_x[CLDNN_HIP_ELTWISE_MAX_INPUTS];  /* 0 = 1 */
    int32_t has_coefficients;     /* float sum only */
    float coefficients[CLDNN_HIP_ELTWISE_MAX_INPUTS];
    cldnn_hip_tensor output;
    int32_t quantized;
    float output_quantization_factor;
    int32_t activation;           /* CLDNN_HIP_ACT_* */
    float m, n;
} cldnn_hip_eltwise_desc;
/* asynchronous on the engine stream; device pointers; calib_dev may be NULL */
cldnn_hip_status cldnn_hip_eltwise(cldnn_hip_engine e, const cldnn_hip_eltwise_desc* desc, const void* const* inputs_dev,
                                   const float* calib_dev, void* output_dev);

/* ------------------------------------------------------------------ pooling
 * The layers between the convolutions of an int8 network: sliding-window maximum / average.  Replaces the pooling
 * kernels (reference src/gpu/pooling_gpu.cpp:60-160, kernel_selector/core/cl_kernels/pooling_gpu_int8_ref.cl:15-140,
 * pooling_gpu_ref.cl): int8 data accumulate in int and an average is round(sum / count), half away from zero; float
 * data accumulate in float.  Taps outside the input are skipped; the data type and the feature count are kept. */
enum { CLDNN_HIP_POOL_MAX = 0, CLDNN_HIP_POOL_AVERAGE = 1 };
enum {
    CLDNN_HIP_POOL_DIV_FIXED = 0,  /* average divides by the window size (pooling_mode::average) */
    CLDNN_HIP_POOL_DIV_VALID = 1,  /* ... by the number of taps inside the input (average_no_padding) */
    CLDNN_HIP_POOL_DIV_PADDED = 2  /* ... by the window clipped to input + padding (average whose last window overhangs) */
};
typedef struct {
    cldnn_hip_tensor input, output;
    int32_t mode;                 /* CLDNN_HIP_POOL_* */
    int32_t divider;              /* CLDNN_HIP_POOL_DIV_* */
    int32_t size_y, size_x;
    int32_t stride_y, stride_x;
    int32_t pad_y, pad_x;         /* = max(-input_offset, 0) */
} cldnn_hip_pooling_desc;
/* asynchronous on the engine stream; device pointers */
cldnn_hip_status cldnn_hip_pooling(cldnn_hip_engine e, const cldnn_hip_pooling_desc* desc, const void* input_dev,
                                   void* output_dev);
/* output extent along one axis: the last window may overhang the padded input once but must start inside the data
 * (reference src/include/sliding_window_utils.h:135-186, swor_mode::exceed_once_data; src/pooling.cpp:110-116) */
int32_t cldnn_hip_pooling_out_extent(int32_t in, int32_t pad, int32_t size, int32_t stride);

/* ------------------------------------------------------------------ convolution
 * One object per convolution / fused_conv_eltwise node; replaces
 * convolution_gpu::create + kernel selection + weight reordering
 * (reference src/gpu/convolution_gpu.cpp:71-162, src/gpu/fused_conv_eltwise_gpu.cpp:70-200,
 *  kernel_selector/core/kernel_selector.cpp:80-207, src/graph_optimizer/post_optimize_weights.cpp:36-66)
 * and, at run time, execute_impl (reference src/gpu/primitive_gpu_base.h:117-168).
 * Arithmetic follows the reference semantic kernel
 * (kernel_selector/core/cl_kernels/fused_conv_eltwise_gpu_ref.cl:93-233). */
/* which kernel family may be used */
enum {
    CLDNN_HIP_IMPL_AUTO = 0,      /* tile-config table decides */
    CLDNN_HIP_IMPL_REF = 1,       /* one work-item per output, any layout */
    CLDNN_HIP_IMPL_MFMA = 2,      /* implicit GEMM on int8 MFMA, fs_b_yx_fsv16 */
    CLDNN_HIP_IMPL_DEPTHWISE = 3  /* bandwidth kernel, fs_b_yx_fsv16, groups == features */
};

typedef struct {
    cldnn_hip_tensor input;       /* activations */
    cldnn_hip_tensor output;      /* logical size must equal the computed output size */
    cldnn_hip_tensor eltw;        /* second input of fused_conv_eltwise (ignored unless fused) */
    int32_t weights_dtype;        /* CLDNN_HIP_S8 (or F32 for the float reference path) */
    int32_t bias_dtype;           /* CLDNN_HIP_I32 / F32 / NO_TYPE */
    int32_t ofm, ifm;             /* totals over all groups */
    int32_t fy, fx;
    int32_t stride_y, stride_x;
    int32_t dilation_y, dilation_x;
    int32_t pad_y, pad_x;         /* = max(-input_offset, 0) */
    int32_t groups;
    int32_t has_wqf;              /* weights_quantization_factors given */
    int32_t has_calib;            /* output_calibration_factors given */
    float input_quantization_factor;
    float output_quantization_factor;
    int32_t activation;           /* CLDNN_HIP_ACT_* applied to the dequantised conv result */
    float activation_m, activation_n;
    /* fused_conv_eltwise part */
    int32_t fused;
    float non_conv_scale;
    int32_t eltw_activation;
    float eltw_activation_m, eltw_activation_n;
    int32_t has_eltw_calib;
    int32_t eltw_stride_y, eltw_stride_x;
    int32_t second_input_in_output; /* residual is read from the output buffer itself */
    int32_t round_to_even;        /* 0 = reference behaviour (half away from zero) */
    int32_t impl;                 /* CLDNN_HIP_IMPL_* */
    int32_t tile_override;        /* 0 = table decides; otherwise row + 1 of the tile-config table (tuning / tests) */
    /* zero padding on the high side MINUS the padding on the low side (pad_y / pad_x); 0 = symmetric.  Asymmetric
     * padding_above / padding_below of the primitive, which the reference realises with a border primitive
     * (src/graph_optimizer/handle_input_padding.cpp:43-77). */
    int32_t pad_end_delta_y, pad_end_delta_x;
    /* 1: the epilogue of the reference's quantized fully_connected kernels instead of the convolution's
     * (kernel_selector/core/cl_kernels/fully_connected_gpu_bfyx_ref.cl:63-84, fully_connected_gpu_MMAD.cl:103-118):
     * with a bias (char)round(((float)acc * wqf * iqf + bias) * (calib or output factor)), without one the raw
     * accumulator; conversion to char keeps the low byte; the activation acts on that char.  A fully_connected layer
     * is the convolution whose filter covers the whole input plane; this flag only matters when has_wqf is set. */
    int32_t fully_connected;
    /* fused form only, needs has_wqf.  1: the convolution's rounded result is saturated to the s8 range before the
     * second input is added (2: to the u8 range) -- the arithmetic of a convolution that writes int8 followed by a
     * stand-alone quantized eltwise sum (reference generic_eltwise_ref.cl:318-330 behind convolution_gpu_ref), which
     * fused_conv_eltwise itself does not have: it adds to the unsaturated value (fused_conv_eltwise_gpu_ref.cl:199-233).
     * Lets a sum the reference leaves stand-alone run inside the convolution with unchanged results. */
    int32_t conv_saturate;
    /* Two convolutions of the same input in one launch ("siblings": same filter size, stride, padding and dilation, e.g.
     * a residual block's shortcut projection and its opening 1x1).  sibling_split > 0: output features [0, sibling_split)
     * belong to the first convolution and take `activation`, features [sibling_split, ofm) belong to the second and take
     * sibling_activation; weights, bias and per-feature factors are the two convolutions' concatenated.  In
     * fs_b_yx_fsv16 the second convolution's result is the contiguous tail of the output buffer (feature slices are the
     * outermost axis), so a reader takes it as a tensor of its own.  Needs a multiple of 16, one group, the quantized
     * non-fused form; not for fully_connected.  The reference enqueues the two primitives one after the other
     * (src/gpu/primitive_gpu_base.h:117-168); the results per feature are the same. */
    int32_t sibling_split;
    int32_t sibling_activation;
    float sibling_activation_m, sibling_activation_n;
} cldnn_hip_conv_desc;

/* Host pointers: weights [ofm][ifm/groups][fy][fx] dense, bias/wqf/calib/eltw_calib [ofm] or NULL.
 * Everything is copied / pre-packed into device memory owned by the object. */
cldnn_hip_status cldnn_hip_conv_create(cldnn_hip_engine e, const cldnn_hip_conv_desc* desc, const void* weights,
                                       const void* bias, const float* wqf, const float* calib,
                                       const float* eltw_calib, cldnn_hip_conv* out);
cldnn_hip_status cldnn_hip_conv_release(cldnn_hip_conv c);
/* asynchronous on the engine stream; device pointers */
cldnn_hip_status cldnn_hip_conv_enqueue(cldnn_hip_conv c, const void* input_dev, void* output_dev,
                                        const void* eltw_dev);
/* cldnn_hip_conv_enqueue for callers that must not allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and
 * results as cldnn_hip_conv_enqueue; the one kernel family with a scratch buffer -- the small-batch kernel, which
 * gathers the activations of a filter wider than one tap into fragment order -- takes that buffer from a fixed
 * array of 4 MiB inside the library's code object (one copy per device, held until the process ends) instead of
 * the object's own allocation.  Calls no hipMalloc / hipFree.  A convolution whose gather needs more than 4 MiB is
 * refused with CLDNN_HIP_UNSUPPORTED_SIZE.  Every call on a device shares that device's array: calls that overlap
 * on one device (two streams) race; calls on one stream are ordered.  Nothing in the array has to start at zero. */
cldnn_hip_status cldnn_hip_conv_enqueue_static_scratch(cldnn_hip_conv c, const void* input_dev, void* output_dev,
                                                       const void* eltw_dev);
/* raw int32 accumulators (before bias), dense [b][ofm][oy][ox]; test / verification hook */
cldnn_hip_status cldnn_hip_conv_accumulators(cldnn_hip_conv c, const void* input_dev, int32_t* acc_dev);

typedef struct {
    int32_t impl;                 /* CLDNN_HIP_IMPL_* actually chosen */
    int32_t tile_index;           /* row of the tile-config table (-1 when not applicable) */
    int32_t tile_pixels, tile_ofm;
    int32_t grid, block;
    int32_t lds_bytes;
    int64_t ops;                  /* 2*B*OY*OX*OFM*(IFM/groups)*FY*FX */
    int64_t bytes;                /* algorithmic bytes: input + output + weights + per-ofm vectors (+ residual) */
    char kernel_name[96];
} cldnn_hip_conv_info;
cldnn_hip_status cldnn_hip_conv_get_info(cldnn_hip_conv c, cldnn_hip_conv_info* info);

/* ------------------------------------------------------------------ convolution chain
 * Two or three convolution / fused_conv_eltwise nodes of which every one after the first is a 1x1 / stride-1 /
 * unpadded convolution that reads its predecessor's result, executed as ONE launch: the requantised int8 tile of a
 * stage is handed to the next stage in registers.  The reference runs such nodes one launch each
 * (src/gpu/primitive_gpu_base.h:117-168); the results are the same bits.  Typical use: the tail of a ResNet bottleneck,
 * 3x3 -> 1x1 expansion with the residual sum -> the next block's 1x1 reduction.
 * descs / weights / bias / wqf / calib / eltw_calib: `count` entries each, as for cldnn_hip_conv_create (the arrays
 * bias, wqf, calib, eltw_calib and their entries may be NULL).  descs[k + 1].input must describe the same logical
 * tensor as descs[k].output.  keep_output[k] == 0: nobody else reads stage k's result and it is never written
 * (NULL: every result is written).  Fails with CLDNN_HIP_UNSUPPORTED_FORMAT when the convolutions cannot run as one
 * chain (layout, epilogue form, weights that do not fit into LDS ...): the caller then runs them one by one. */
cldnn_hip_status cldnn_hip_conv_chain_create(cldnn_hip_engine e, int32_t count, const cldnn_hip_conv_desc* descs,
                                             const void* const* weights, const void* const* bias, const float* const* wqf,
                                             const float* const* calib, const float* const* eltw_calib,
                                             const int32_t* keep_output, cldnn_hip_conv_chain* out);
cldnn_hip_status cldnn_hip_conv_chain_release(cldnn_hip_conv_chain chain);
/* asynchronous on the engine stream; outputs_dev / eltw_dev: `count` device pointers (entries of stages that are not
 * kept / not fused are ignored and may be NULL; eltw_dev itself may be NULL when no stage is fused) */
cldnn_hip_status cldnn_hip_conv_chain_enqueue(cldnn_hip_conv_chain chain, const void* input_dev, void* const* outputs_dev,
                                              const void* const* eltw_dev);
/* ops = sum over the stages; bytes = what crosses the memory interface (intermediate tensors that are neither kept
 * nor re-read are left out) */
cldnn_hip_status cldnn_hip_conv_chain_get_info(cldnn_hip_conv_chain chain, cldnn_hip_conv_info* info);

/* computed output extent along one axis (reference src/include/sliding_window_utils.h:90-129) */
int32_t cldnn_hip_conv_out_extent(int32_t in, int32_t pad, int32_t filt, int32_t dil, int32_t stride);

/* Kernel runner for tuning: times the table's own choice and every row of the tile-config table that accepts this
 * convolution, on scratch tensors of the descriptor's shapes filled with pseudo-random bytes, and reports the fastest.
 * Replaces the reference's kernel_runner (src/gpu/kernel_runner.cpp:106-190, used by tuning_mode tune_and_cache through
 * kernel_selector/core/kernel_selector.cpp GetAutoTuneBestKernel): the device is kept busy for 150 ms first (the
 * clocks of an idle device rise over tens of milliseconds, and the candidates timed first would lose to the later ones),
 * then each candidate is created, run for 20 ms untimed and `runs` times back to back on the engine's stream between
 * two events; the best of three such batches counts.
 * best_tile_index = -1 when the table's own choice is the fastest (or no row applies: depthwise, plain layouts).
 * row_us (may be NULL) receives cldnn_hip_tile_config_count() entries, negative where a row does not apply.
 * Blocks until done; allocates and frees its scratch tensors. */
cldnn_hip_status cldnn_hip_conv_tune(cldnn_hip_engine e, const cldnn_hip_conv_desc* desc, const void* weights,
                                     const void* bias, const float* wqf, const float* calib, const float* eltw_calib,
                                     int32_t runs, int32_t* best_tile_index, float* best_us, float* default_us,
                                     float* row_us);

/* number of rows of the gfx950 tile-config table and a printable description of one row */
int32_t cldnn_hip_tile_config_count(void);
const char* cldnn_hip_tile_config_name(int32_t index);

#ifdef __cplusplus
}
#endif
#endif
