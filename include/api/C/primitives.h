/*
 * Descriptor structures ("dto") of the primitives a convolution topology needs.  Field order and
 * meaning follow the reference headers: api/C/input_layout.h, data.h, reorder.h, activation.h,
 * eltwise.h, pooling.h, concatenation.h, convolution.h:36-74 and api_extension/C/fused_conv_eltwise.h:35-97.
 */
#ifndef CLDNN_PRIMITIVES_H
#define CLDNN_PRIMITIVES_H
#include "cldnn.h"

#ifdef __cplusplus
extern "C" {
#endif

CLDNN_BEGIN_PRIMITIVE_DESC(input_layout)
cldnn_layout layout;
CLDNN_END_PRIMITIVE_DESC(input_layout)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(input_layout);

CLDNN_BEGIN_PRIMITIVE_DESC(data)
cldnn_memory mem;
CLDNN_END_PRIMITIVE_DESC(data)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(data);

CLDNN_BEGIN_PRIMITIVE_DESC(reorder)
cldnn_format_type output_format;
cldnn_primitive_id mean_subtract;          /* not supported: must be empty */
cldnn_float_arr subtract_per_feature;      /* not supported: must be empty */
cldnn_reorder_mean_mode mean_mode;
CLDNN_END_PRIMITIVE_DESC(reorder)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(reorder);

CLDNN_BEGIN_PRIMITIVE_DESC(activation)
cldnn_activation_func activation_func;
cldnn_activation_additional_params additional_params;
cldnn_primitive_id additional_params_input; /* not supported: must be empty */
CLDNN_END_PRIMITIVE_DESC(activation)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(activation);

/* pooling (reference api/C/pooling.h:33-69); the argmax and bilinear modes are not implemented */
typedef enum {
    cldnn_pooling_max,
    cldnn_pooling_average,
    cldnn_pooling_average_no_padding,
    cldnn_pooling_max_with_argmax,
    cldnn_pooling_bilinear
} cldnn_pooling_mode;

CLDNN_BEGIN_PRIMITIVE_DESC(pooling)
cldnn_primitive_id argmax;    /* not supported: must be empty */
int32_t mode;                 /* cldnn_pooling_mode */
int8_t global_pooling;        /* window = the whole input plane */
cldnn_tensor input_offset;    /* negative = zero padding */
cldnn_tensor stride;
cldnn_tensor size;
uint32_t with_output_size;
cldnn_tensor output_size;
CLDNN_END_PRIMITIVE_DESC(pooling)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(pooling);

/* concatenation (reference api/C/concatenation.h:31-50): the inputs side by side along one axis; every other axis must
 * agree.  along_z belongs to five-dimensional tensors, which this library does not have. */
typedef enum {
    cldnn_concatenation_along_b = 0,
    cldnn_concatenation_along_f = CLDNN_TENSOR_BATCH_DIM_MAX,
    cldnn_concatenation_along_x = CLDNN_TENSOR_BATCH_DIM_MAX + CLDNN_TENSOR_FEATURE_DIM_MAX,
    cldnn_concatenation_along_y = cldnn_concatenation_along_x + 1,
    cldnn_concatenation_along_z = cldnn_concatenation_along_y + 1
} cldnn_concatenation_axis;

CLDNN_BEGIN_PRIMITIVE_DESC(concatenation)
cldnn_concatenation_axis axis;
CLDNN_END_PRIMITIVE_DESC(concatenation)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(concatenation);

/* fully_connected (reference api/C/fully_connected.h:33-59): the convolution whose filter covers the whole input
 * plane; weights [ofm][ifm][y][x] in bfyx.  Quantized (weights_quantization_factors given) it has the epilogue of the
 * reference's int8 fully_connected kernels, not the convolution's. */
CLDNN_BEGIN_PRIMITIVE_DESC(fully_connected)
uint32_t with_activation;
float activation_negative_slope;
cldnn_primitive_id weights;
cldnn_primitive_id bias;
cldnn_primitive_id weights_quantization_factors;
cldnn_primitive_id output_calibration_factors;
float input_quantization_factor;
float output_quantization_factor;
CLDNN_END_PRIMITIVE_DESC(fully_connected)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(fully_connected);

typedef enum {
    cldnn_eltwise_sum,
    cldnn_eltwise_sub,
    cldnn_eltwise_max,
    cldnn_eltwise_prod,
    cldnn_eltwise_div,
    cldnn_eltwise_min,
    cldnn_eltwise_pow,
    cldnn_eltwise_mod
} cldnn_eltwise_mode; /* the reference's comparison and logic modes (eq ... or) are not part of this library */

CLDNN_BEGIN_PRIMITIVE_DESC(eltwise)
cldnn_primitive_id output_calibration_factors;
float output_quantization_factor;
int32_t mode; /* cldnn_eltwise_mode */
cldnn_float_arr coefficients;
uint32_t with_activation;
float activation_negative_slope;
cldnn_tensor_arr stride;
CLDNN_END_PRIMITIVE_DESC(eltwise)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(eltwise);

CLDNN_BEGIN_PRIMITIVE_DESC(convolution)
cldnn_tensor input_offset;   /* negative spatial values = zero padding; positive = that many elements left out on both sides */
cldnn_tensor stride;
cldnn_tensor dilation;
uint32_t with_activation;
float activation_negative_slope;
uint32_t split;              /* number of weight / bias / factor primitives; executed as groups = split in one launch */
uint32_t with_output_size;
cldnn_tensor output_size;
cldnn_primitive_id_arr weights;
cldnn_primitive_id_arr bias;
cldnn_primitive_id_arr weights_quantization_factors;
cldnn_primitive_id_arr output_calibration_factors;
float input_quantization_factor;
float output_quantization_factor;
uint32_t groups;
cldnn_tensor padding_above;  /* zero padding in front of / behind the data, each side on its own (may differ) */
cldnn_tensor padding_below;
CLDNN_END_PRIMITIVE_DESC(convolution)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(convolution);

CLDNN_BEGIN_PRIMITIVE_DESC(fused_conv_eltwise)
struct conv_data {
    cldnn_tensor input_offset;
    cldnn_tensor stride;
    cldnn_tensor dilation;
    uint32_t with_activation;
    float activation_negative_slope;
    uint32_t split;
    uint32_t with_output_size;
    cldnn_tensor output_size;
    cldnn_primitive_id_arr weights;
    cldnn_primitive_id_arr bias;
    cldnn_primitive_id_arr weights_quantization_factors;
    cldnn_primitive_id_arr output_calibration_factors;
    float input_quantization_factor;
    float output_quantization_factor;
} conv;
struct eltw_data {
    cldnn_primitive_id output_calibration_factors;
    float output_quantization_factor;
    int32_t mode;
    cldnn_float_arr coefficients;
    uint32_t with_activation;
    float activation_negative_slope;
    cldnn_tensor_arr stride;
} eltw;
float non_conv_scale;
uint8_t second_input_in_output;
CLDNN_END_PRIMITIVE_DESC(fused_conv_eltwise)
CLDNN_DECLARE_PRIMITIVE_TYPE_ID(fused_conv_eltwise);

#ifdef __cplusplus
}
#endif
#endif
