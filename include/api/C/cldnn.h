/*
 * cldnn.h -- C API of the clDNN-compatible host library (libclDNN.so) for the quantized
 * convolution path, backed by the HIP layer of include/cldnn_hip.h instead of OpenCL.
 *
 * Names, argument meaning, enumerator values and structure layouts follow the reference's
 * api/C/cldnn.h (status codes :70-79, engine configuration :149-164, engine info :167-188,
 * build options :207-227, formats :253-301, tensor / padding / layout :311-351, primitive
 * descriptor macros :497-520, functions :537-805), so code written against that header compiles
 * and links against this one.  Only what a convolution topology needs is present: the primitives
 * input_layout, data, reorder, activation, eltwise, convolution and fused_conv_eltwise, and the
 * formats yxfb, byxf, bfyx, b_fs_yx_fsv4 plus the new fs_b_yx_fsv16.
 *
 * Every function reports through its trailing cldnn_status*; the text of the last failure on the
 * calling thread is returned by cldnn_get_last_error_message().
 */
#ifndef CLDNN_H
#define CLDNN_H

#include <stddef.h>
#include <stdint.h>

#if defined(_WIN32)
#define CLDNN_API __declspec(dllexport)
#else
#define CLDNN_API __attribute__((visibility("default")))
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status */
#define CLDNN_SUCCESS 0
#define CLDNN_ERROR -1
#define CLDNN_INVALID_ARG -2
#define CLDNN_OUT_OF_RESOURCES -3
#define CLDNN_DEVICE_ERROR -4
#define CLDNN_UNSUPPORTED_SIZE -5
#define CLDNN_UNSUPPORTED_FORMAT -6
#define CLDNN_DIMENSION_MISMATCH -7
#define CLDNN_ALLOC_SIZE_EXCEEDED -8
#define CLDNN_GLOBAL_SIZE_EXCEEDED -9
typedef int32_t cldnn_status;

typedef struct { int32_t major, minor, build, revision; } cldnn_version;

/* ---- opaque handles (intrusively reference counted: create/build/allocate/get return +1) */
typedef struct cldnn_engine_impl* cldnn_engine;
typedef struct cldnn_event_impl* cldnn_event;
typedef struct cldnn_topology_impl* cldnn_topology;
typedef struct cldnn_program_impl* cldnn_program;
typedef struct cldnn_network_impl* cldnn_network;
typedef struct cldnn_memory_impl* cldnn_memory;

/* ---- engine.  The single engine type keeps the value 0 ("the default device engine"); here it is HIP. */
typedef enum { cldnn_engine_ocl = 0 } cldnn_engine_type;
typedef enum { cldnn_priority_disabled, cldnn_priority_low, cldnn_priority_med, cldnn_priority_high } cldnn_priority_mode_type;
typedef enum { cldnn_throttle_disabled, cldnn_throttle_low, cldnn_throttle_med, cldnn_throttle_high } cldnn_throttle_mode_type;

typedef struct {
    uint32_t enable_profiling;         /* per-primitive timing through hipEvent pairs */
    uint32_t meaningful_kernels_names; /* accepted, no effect (kernels are precompiled) */
    uint32_t dump_custom_program;      /* accepted, no effect */
    const char* compiler_options;      /* accepted, no effect */
    const char* single_kernel_name;    /* accepted, no effect */
    uint32_t enable_parallelisation;   /* a second stream runs convolutions whose only user comes later (shortcut branches) */
    const char* engine_log;            /* accepted, no effect */
    const char* sources_dumps_dir;     /* accepted, no effect */
    int16_t priority_mode;             /* must stay disabled: one stream at default priority */
    int16_t throttle_mode;
    uint32_t enable_memory_pool;       /* networks reuse buffers between intermediate tensors of identical layout */
    void* context;                     /* must be NULL */
    const char* tuning_cache_path;     /* tuning cache file of a tuning_config that names none (default "cache.json") */
} cldnn_engine_configuration;

typedef struct {
    uint32_t cores_count;
    uint32_t core_frequency;
    uint64_t max_work_group_size;
    uint64_t max_local_mem_size;
    uint64_t max_global_mem_size;
    uint64_t max_alloc_mem_size;
    uint64_t max_image2d_width;
    uint64_t max_image2d_height;
    uint8_t supports_fp16;
    uint8_t supports_fp16_denorms;
    uint8_t supports_subgroups_short;
    uint8_t supports_image;
    uint8_t supports_imad;   /* 1: packed int8 dot products are native */
    uint8_t supports_immad;  /* 1: int8 matrix instructions (MFMA) are native */
} cldnn_engine_info;

/* ---- events */
typedef void (*cldnn_event_handler)(void*);
typedef struct { const char* name; uint64_t nanoseconds; } cldnn_profiling_interval;

/* ---- build options */
typedef enum {
    cldnn_build_option_fusing,
    cldnn_build_option_optimize_data,
    cldnn_build_option_debug,
    cldnn_build_option_outputs,
    cldnn_build_option_tuning_config,
    cldnn_build_option_graph_dumps_dir,
    cldnn_build_option_learning_config,
    cldnn_build_option_detection_output_gpu
} cldnn_build_option_type;
typedef enum { cldnn_tuning_disabled, cldnn_tuning_use_cache, cldnn_tuning_tune_and_cache } cldnn_tuning_mode_type;
struct cldnn_tuning_config { const int32_t mode; const char* cache_file_path; };
struct cldnn_learning_params { const float momentum; const float weights_decay; };
typedef struct { int32_t type; const void* data; } cldnn_build_option;
typedef struct { cldnn_event event; cldnn_memory memory; } cldnn_network_output;

/* ---- memory description.  Enumerator values are the reference's. */
typedef enum {
    cldnn_format_yxfb = 0,
    cldnn_format_byxf = 1,
    cldnn_format_bfyx = 2,
    cldnn_format_fyxb = 3,             /* listed for completeness; not accepted by this library */
    cldnn_format_b_fs_yx_fsv4 = 31,
    cldnn_format_fs_b_yx_fsv16 = 35,   /* NEW: [fs][b][y][x][16 features], the int8 MFMA layout */
    cldnn_format_format_num = 36,
    cldnn_format_any = -1
} cldnn_format_type;

#define CLDNN_FLOAT_TYPE_MASK 0x80
#define CLDNN_UINT_TYPE_MASK 0x40
#define CLDNN_TENSOR_BATCH_DIM_MAX 1
#define CLDNN_TENSOR_FEATURE_DIM_MAX 1
#define CLDNN_TENSOR_SPATIAL_DIM_MAX 3
#define CLDNN_TENSOR_LOCAL_DIM_MAX 2
#define CLDNN_TENSOR_DIM_MAX 8

/* sizes[] = { batch, feature, x, y, z, local x, local y, - } */
typedef struct {
    size_t batch_num, feature_num, spatial_num, local_num;
    int32_t sizes[CLDNN_TENSOR_DIM_MAX];
} cldnn_tensor;

typedef struct { cldnn_tensor lower_size, upper_size; float filling_value; } cldnn_padding;

typedef enum {
    cldnn_i8 = sizeof(int8_t),
    cldnn_f16 = sizeof(int16_t) | CLDNN_FLOAT_TYPE_MASK, /* not accepted by this library */
    cldnn_f32 = sizeof(float) | CLDNN_FLOAT_TYPE_MASK,
    cldnn_u8 = sizeof(uint8_t) | CLDNN_UINT_TYPE_MASK,
    cldnn_i32 = sizeof(int32_t),
    cldnn_i64 = sizeof(int64_t)                          /* not accepted by this library */
} cldnn_data_type;

typedef struct {
    size_t data_type;   /* cldnn_data_type */
    int32_t format;     /* cldnn_format_type */
    cldnn_tensor size;  /* logical size, padding excluded */
    cldnn_padding padding;
} cldnn_layout;

typedef struct { const float* data; size_t size; } cldnn_float_arr;
typedef struct { const uint16_t* data; size_t size; } cldnn_uint16_t_arr;
typedef struct { const cldnn_tensor* data; size_t size; } cldnn_tensor_arr;
typedef const struct cldnn_primitive_type* cldnn_primitive_type_id;
typedef const char* cldnn_primitive_id;
typedef struct { const cldnn_primitive_id* data; size_t size; } cldnn_primitive_id_arr;
typedef struct { cldnn_data_type data_type; char enabled; } cldnn_optional_data_type;

/* activation functions: values of the reference enum; this library implements none, relu,
 * relu_negative_slope and clamp (the ones a quantized convolution topology uses); the others
 * are refused when the program is built */
typedef enum cldnn_activation_func_t {
    activation_none = 0,
    activation_logistic = 1,
    activation_hyperbolic_tan = 2,
    activation_relu = 3,
    activation_relu_negative_slope = 4,
    activation_clamp = 5,
    activation_softrelu = 6,
    activation_abs = 7,
    activation_linear = 8,
    activation_square = 9,
    activation_sqrt = 10,
    activation_elu = 11,
    activation_negative = 25
} cldnn_activation_func;
typedef struct cldnn_activation_additional_params_t { float a, b; } cldnn_activation_additional_params;
typedef enum cldnn_reorder_mean_mode_t { mean_none, mean_subtract, mean_mul, mean_div } cldnn_reorder_mean_mode;

/* ---- primitive descriptors: every descriptor starts with these five fields */
#define CLDNN_BEGIN_PRIMITIVE_DESC(PType)          \
    struct cldnn_##PType##_desc {                  \
        cldnn_primitive_type_id type;              \
        cldnn_primitive_id id;                     \
        cldnn_primitive_id_arr input;              \
        cldnn_padding output_padding;              \
        cldnn_optional_data_type output_data_type;
#define CLDNN_END_PRIMITIVE_DESC(PType) };
#define CLDNN_PRIMITIVE_DESC(PType) cldnn_##PType##_desc
CLDNN_BEGIN_PRIMITIVE_DESC(primitive)
CLDNN_END_PRIMITIVE_DESC(primitive)

CLDNN_API cldnn_version cldnn_get_version(cldnn_status* status);

/* ---- topology */
CLDNN_API cldnn_topology cldnn_create_topology(cldnn_status* status);
CLDNN_API void cldnn_add_primitive(cldnn_topology topology, const struct CLDNN_PRIMITIVE_DESC(primitive)* dto, cldnn_status* status);
CLDNN_API void cldnn_change_input_layout(cldnn_topology topology, cldnn_primitive_id id, cldnn_layout new_layout, cldnn_status* status);
CLDNN_API void cldnn_get_primitive_ids(cldnn_topology topology, char* ids, size_t size, size_t* size_ret, cldnn_status* status);
CLDNN_API void cldnn_retain_topology(cldnn_topology topology, cldnn_status* status);
CLDNN_API void cldnn_release_topology(cldnn_topology topology, cldnn_status* status);

/* ---- engine */
CLDNN_API uint32_t cldnn_get_engine_count(int32_t type, cldnn_status* status);
CLDNN_API void cldnn_release_pending_memory(cldnn_engine engine, cldnn_status* status);
CLDNN_API cldnn_engine cldnn_create_engine(int32_t type, uint32_t engine_num, const cldnn_engine_configuration* configuration, cldnn_status* status);
CLDNN_API void cldnn_retain_engine(cldnn_engine engine, cldnn_status* status);
CLDNN_API void cldnn_release_engine(cldnn_engine engine, cldnn_status* status);
CLDNN_API cldnn_engine_info cldnn_get_engine_info(cldnn_engine engine, cldnn_status* status);
CLDNN_API int32_t cldnn_get_engine_type(cldnn_engine engine, cldnn_status* status);
CLDNN_API int64_t cldnn_get_temp_used_device_memory_size(cldnn_engine engine, cldnn_status* status);
CLDNN_API int64_t cldnn_get_max_used_device_memory_size(cldnn_engine engine, cldnn_status* status);

/* ---- events */
CLDNN_API cldnn_event cldnn_create_user_event(cldnn_engine engine, cldnn_status* status);
CLDNN_API int32_t cldnn_is_user_event(cldnn_event event, cldnn_status* status);
CLDNN_API void cldnn_retain_event(cldnn_event event, cldnn_status* status);
CLDNN_API void cldnn_release_event(cldnn_event event, cldnn_status* status);
CLDNN_API void cldnn_wait_for_event(cldnn_event event, cldnn_status* status);
CLDNN_API void cldnn_set_event(cldnn_event event, cldnn_status* status);
CLDNN_API void cldnn_add_event_handler(cldnn_event event, cldnn_event_handler handler, void* param, cldnn_status* status);
CLDNN_API void cldnn_get_event_profiling_info(cldnn_event event, cldnn_profiling_interval* profiling, size_t size, size_t* size_ret, cldnn_status* status);

/* ---- program / network */
CLDNN_API cldnn_program cldnn_build_program(cldnn_engine engine, cldnn_topology topology, cldnn_build_option* options, size_t options_num, cldnn_status* status);
CLDNN_API void cldnn_retain_program(cldnn_program program, cldnn_status* status);
CLDNN_API void cldnn_release_program(cldnn_program program, cldnn_status* status);
CLDNN_API cldnn_network cldnn_build_network(cldnn_engine engine, cldnn_topology topology, cldnn_build_option* options, size_t options_num, cldnn_status* status);
CLDNN_API cldnn_network cldnn_allocate_network(cldnn_program program, cldnn_status* status);
CLDNN_API void cldnn_retain_network(cldnn_network network, cldnn_status* status);
CLDNN_API void cldnn_release_network(cldnn_network network, cldnn_status* status);
CLDNN_API void cldnn_set_network_input(cldnn_network network, cldnn_primitive_id id, cldnn_memory mem, cldnn_status* status);
CLDNN_API void cldnn_get_primitive_info(cldnn_network network, cldnn_primitive_id id, char* info, size_t size, size_t* size_ret, cldnn_status* status);
CLDNN_API cldnn_engine cldnn_get_network_engine(cldnn_network network, cldnn_status* status);
CLDNN_API cldnn_program cldnn_get_network_program(cldnn_network network, cldnn_status* status);
CLDNN_API void cldnn_get_network_output_names(cldnn_network network, char* names, size_t size, size_t* size_ret, cldnn_status* status);
CLDNN_API void cldnn_get_network_executed_primitive_names(cldnn_network network, char* names, size_t size, size_t* size_ret, cldnn_status* status);
CLDNN_API void cldnn_get_network_all_primitive_names(cldnn_network network, char* names, size_t size, size_t* size_ret, cldnn_status* status);
CLDNN_API void cldnn_get_network_all_primitive_org_names(cldnn_network network, char* names, size_t size, size_t* size_ret, cldnn_status* status);
CLDNN_API void cldnn_execute_network(cldnn_network network, cldnn_event* dependencies, size_t deps_num, cldnn_status* status);
CLDNN_API cldnn_network_output cldnn_get_network_output(cldnn_network network, const char* name, cldnn_status* status);
CLDNN_API cldnn_memory cldnn_get_network_output_memory(cldnn_network network, const char* name, cldnn_status* status);
CLDNN_API cldnn_event cldnn_get_network_output_event(cldnn_network network, const char* name, cldnn_status* status);

/* ---- memory */
CLDNN_API cldnn_memory cldnn_allocate_memory(cldnn_engine engine, cldnn_layout layout, cldnn_status* status);
CLDNN_API cldnn_memory cldnn_attach_memory(cldnn_layout layout, void* pointer, size_t size, cldnn_status* status);
CLDNN_API int32_t cldnn_is_the_same_buffer(cldnn_memory mem1, cldnn_memory mem2, cldnn_status* status);
CLDNN_API void cldnn_retain_memory(cldnn_memory memory, cldnn_status* status);
CLDNN_API void cldnn_release_memory(cldnn_memory memory, cldnn_status* status);
CLDNN_API void* cldnn_lock_memory(cldnn_memory memory, cldnn_status* status);
CLDNN_API void cldnn_unlock_memory(cldnn_memory memory, cldnn_status* status);
CLDNN_API cldnn_layout cldnn_get_memory_layout(cldnn_memory memory, cldnn_status* status);
CLDNN_API cldnn_engine cldnn_get_memory_engine(cldnn_memory memory, cldnn_status* status);

CLDNN_API const char* cldnn_get_last_error_message();

/* ---- addition (no counterpart in the reference API; the reference offers graph dumps to files through
 * cldnn_build_option_graph_dumps_dir instead).  Runs the graph passes of cldnn_build_program on the
 * topology without an engine and returns the resulting graph in execution order as a JSON array: per
 * node id, type, org_id, deps, is_output, format, data_type, size / pad_lower / pad_upper as
 * [b, f, x, y], and for convolutions the stride and folded activation.  Nothing is compiled or run. */
CLDNN_API void cldnn_plan_topology(cldnn_topology topology, cldnn_build_option* options, size_t options_num, char* json, size_t size, size_t* size_ret, cldnn_status* status);

#ifdef __cplusplus
}
#endif

#ifdef __cplusplus
#define CLDNN_DECLARE_PRIMITIVE_TYPE_ID(PType) extern "C" CLDNN_API cldnn_primitive_type_id cldnn_##PType##_type_id(cldnn_status* status)
#else
#define CLDNN_DECLARE_PRIMITIVE_TYPE_ID(PType) CLDNN_API cldnn_primitive_type_id cldnn_##PType##_type_id(cldnn_status* status)
#endif

#endif /* CLDNN_H */
