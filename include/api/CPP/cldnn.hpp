// Header-only C++ wrappers over the C API of include/api/C/cldnn.h for the convolution path.
//
// Class names, method names and constructor argument order follow the reference's C++ API
// (api/CPP/cldnn_defs.h, tensor.hpp, layout.hpp, memory.hpp, engine.hpp, event.hpp, topology.hpp,
// program.hpp, network.hpp, primitive.hpp, input_layout.hpp, data.hpp, reorder.hpp, activation.hpp,
// eltwise.hpp, convolution.hpp:38-882 and api_extension/CPP/fused_conv_eltwise.hpp:37-160), so code written
// against those headers compiles against this one.  The headers of those names in this directory
// forward here.  Every failing C call is re-thrown as cldnn::error carrying the status and the
// library's message.
#pragma once
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../C/primitives.h"

namespace cldnn {

using status_t = ::cldnn_status;

struct error : std::runtime_error {
    error(const std::string& msg, status_t st = CLDNN_ERROR) : std::runtime_error(msg), _status(st) {}
    status_t status() const { return _status; }

private:
    status_t _status;
};

// runs a C call that takes a trailing cldnn_status* and throws on failure
template <class F>
auto check_status(const char* what, F&& f) -> decltype(f((status_t*)nullptr))
{
    status_t st = CLDNN_SUCCESS;
    auto r = f(&st);
    if (st != CLDNN_SUCCESS) throw error(std::string(what) + ": " + ::cldnn_get_last_error_message(), st);
    return r;
}

enum class data_types : size_t { i8 = cldnn_i8, f16 = cldnn_f16, f32 = cldnn_f32, u8 = cldnn_u8, i32 = cldnn_i32, i64 = cldnn_i64 };

template <class T> struct type_to_data_type;
template <> struct type_to_data_type<int8_t> { static const data_types value = data_types::i8; };
template <> struct type_to_data_type<uint8_t> { static const data_types value = data_types::u8; };
template <> struct type_to_data_type<int32_t> { static const data_types value = data_types::i32; };
template <> struct type_to_data_type<float> { static const data_types value = data_types::f32; };

struct data_type_traits {
    static size_t size_of(data_types t) { return static_cast<size_t>(t) & ~(CLDNN_FLOAT_TYPE_MASK | CLDNN_UINT_TYPE_MASK); }
    static bool is_floating_point(data_types t) { return (static_cast<size_t>(t) & CLDNN_FLOAT_TYPE_MASK) != 0; }
};

struct optional_data_type {
    bool has = false;
    data_types value = data_types::f32;
    optional_data_type() {}
    optional_data_type(data_types v) : has(true), value(v) {}
    explicit operator bool() const { return has; }
    data_types operator*() const { return value; }
};

struct format {
    enum type : int32_t {
        yxfb = cldnn_format_yxfb,
        byxf = cldnn_format_byxf,
        bfyx = cldnn_format_bfyx,
        fyxb = cldnn_format_fyxb,
        b_fs_yx_fsv4 = cldnn_format_b_fs_yx_fsv4,
        fs_b_yx_fsv16 = cldnn_format_fs_b_yx_fsv16,
        format_num = cldnn_format_format_num,
        any = cldnn_format_any
    };
    type value;
    format(type t) : value(t) {}
    explicit format(int32_t t) : value(static_cast<type>(t)) {}
    operator type() const { return value; }
    // character order of the dimensions in memory, outermost first
    std::string order() const
    {
        switch (value) {
        case yxfb: return "yxfb";
        case byxf: return "byxf";
        case fyxb: return "fyxb";
        default: return "bfyx";
        }
    }
};

// N-dimensional size / offset: batch, feature, spatial x, y (z unused here).  Same storage as cldnn_tensor.
struct tensor {
    using value_type = int32_t;
    value_type batch[1], feature[1], spatial[3];
    value_type raw[CLDNN_TENSOR_DIM_MAX];

    explicit tensor(value_type default_size = 0) { fill(default_size); sync(); }
    tensor(value_type b, value_type f, value_type x, value_type y)
    {
        fill(1);
        raw[0] = b, raw[1] = f, raw[2] = x, raw[3] = y;
        sync();
    }
    tensor(value_type b, value_type f, value_type x, value_type y, value_type z)
    {
        fill(1);
        raw[0] = b, raw[1] = f, raw[2] = x, raw[3] = y, raw[4] = z;
        sync();
    }
    // sizes given in the order of `fmt` (e.g. format::bfyx, {b, f, y, x})
    tensor(format fmt, const std::vector<value_type>& sizes, value_type default_size = 1)
    {
        fill(default_size);
        const std::string o = fmt.order();
        if (sizes.size() != o.size()) throw std::invalid_argument("number of sizes does not match format");
        for (size_t i = 0; i < o.size(); ++i) raw[index_of(o[i])] = sizes[i];
        sync();
    }
    tensor(const cldnn_tensor& t)
    {
        for (int i = 0; i < CLDNN_TENSOR_DIM_MAX; ++i) raw[i] = t.sizes[i];
        sync();
    }
    operator cldnn_tensor() const
    {
        cldnn_tensor t{};
        t.batch_num = 1, t.feature_num = 1, t.spatial_num = 3, t.local_num = 2;
        // the named views are the writable ones
        value_type r[CLDNN_TENSOR_DIM_MAX];
        std::memcpy(r, raw, sizeof(r));
        r[0] = batch[0], r[1] = feature[0], r[2] = spatial[0], r[3] = spatial[1], r[4] = spatial[2];
        for (int i = 0; i < CLDNN_TENSOR_DIM_MAX; ++i) t.sizes[i] = r[i];
        return t;
    }
    size_t count() const { return (size_t)batch[0] * feature[0] * spatial[0] * spatial[1] * (spatial[2] > 0 ? spatial[2] : 1); }
    tensor negate() const
    {
        tensor r(*this);
        r.batch[0] = -batch[0], r.feature[0] = -feature[0];
        for (int i = 0; i < 3; ++i) r.spatial[i] = -spatial[i];
        return r;
    }
    bool operator==(const tensor& o) const
    {
        return batch[0] == o.batch[0] && feature[0] == o.feature[0] && spatial[0] == o.spatial[0] && spatial[1] == o.spatial[1];
    }
    bool operator!=(const tensor& o) const { return !(*this == o); }

private:
    void fill(value_type v)
    {
        for (auto& r : raw) r = v;
    }
    void sync() { batch[0] = raw[0], feature[0] = raw[1], spatial[0] = raw[2], spatial[1] = raw[3], spatial[2] = raw[4]; }
    static int index_of(char c) { return c == 'b' ? 0 : c == 'f' ? 1 : c == 'x' ? 2 : 3; }
};

// physical padding around a tensor; sizes in bfyx order like the reference's constructor
struct padding {
    tensor lower, upper;
    float fill;
    padding() : lower(0), upper(0), fill(0.f) {}
    padding(const std::vector<tensor::value_type>& lower_sizes, const std::vector<tensor::value_type>& upper_sizes, float filling_value = 0.f)
        : lower(format::bfyx, lower_sizes, 0), upper(format::bfyx, upper_sizes, 0), fill(filling_value) {}
    padding(const std::vector<tensor::value_type>& sizes, float filling_value = 0.f) : padding(sizes, sizes, filling_value) {}
    padding(const cldnn_padding& p) : lower(p.lower_size), upper(p.upper_size), fill(p.filling_value) {}
    tensor lower_size() const { return lower; }
    tensor upper_size() const { return upper; }
    float filling_value() const { return fill; }
    explicit operator bool() const { return !(lower == tensor(0) && upper == tensor(0)); }
    operator cldnn_padding() const { return cldnn_padding{lower, upper, fill}; }
};

struct layout {
    data_types data_type;
    cldnn::format format;
    tensor size;
    padding data_padding;
    layout(data_types dt, cldnn::format fmt, tensor sz, padding pad = padding()) : data_type(dt), format(fmt), size(sz), data_padding(pad) {}
    layout(const cldnn_layout& l) : data_type((data_types)l.data_type), format((cldnn::format::type)l.format), size(l.size), data_padding(l.padding) {}
    operator cldnn_layout() const { return cldnn_layout{(size_t)data_type, (int32_t)format.value, size, data_padding}; }
    size_t count() const { return size.count(); }
    tensor get_buffer_size() const
    {
        return tensor(size.batch[0] + data_padding.lower.batch[0] + data_padding.upper.batch[0],
                      size.feature[0] + data_padding.lower.feature[0] + data_padding.upper.feature[0],
                      size.spatial[0] + data_padding.lower.spatial[0] + data_padding.upper.spatial[0],
                      size.spatial[1] + data_padding.lower.spatial[1] + data_padding.upper.spatial[1]);
    }
    // bytes of the physical buffer (features rounded up to the block of a blocked format)
    size_t bytes_count() const
    {
        tensor b = get_buffer_size();
        size_t f = (size_t)b.feature[0];
        if (format == cldnn::format::fs_b_yx_fsv16) f = (f + 15) / 16 * 16;
        if (format == cldnn::format::b_fs_yx_fsv4) f = (f + 3) / 4 * 4;
        return data_type_traits::size_of(data_type) * b.batch[0] * f * b.spatial[0] * b.spatial[1];
    }
    layout with_padding(const padding& p) const
    {
        layout r(*this);
        r.data_padding = p;
        return r;
    }
    bool operator==(const layout& o) const { return data_type == o.data_type && format.value == o.format.value && size == o.size; }
};

// ------------------------------------------------------------------------------------------ handles
#define CLDNN_CPP_HANDLE(cls, what)                                                              \
    cls(const cls& o) : _impl(o._impl) { retain(); }                                             \
    cls& operator=(const cls& o)                                                                 \
    {                                                                                            \
        if (_impl != o._impl) {                                                                  \
            release();                                                                           \
            _impl = o._impl;                                                                     \
            retain();                                                                            \
        }                                                                                        \
        return *this;                                                                            \
    }                                                                                            \
    ~cls() { release(); }                                                                        \
    ::cldnn_##what get() const { return _impl; }                                                 \
    /* takes over one reference (what the C API's create / get functions return) */             \
    explicit cls(::cldnn_##what impl) : _impl(impl)                                              \
    {                                                                                            \
        if (!_impl) throw std::invalid_argument(#what " implementation is null");               \
    }                                                                                            \
    bool operator==(const cls& o) const { return _impl == o._impl; }                             \
                                                                                                 \
private:                                                                                         \
    ::cldnn_##what _impl;                                                                        \
    void retain()                                                                                \
    {                                                                                            \
        check_status("retain " #what, [&](status_t* s) { ::cldnn_retain_##what(_impl, s); return 0; }); \
    }                                                                                            \
    void release()                                                                               \
    {                                                                                            \
        if (_impl) {                                                                             \
            status_t s;                                                                          \
            ::cldnn_release_##what(_impl, &s);                                                   \
        }                                                                                        \
    }                                                                                            \
                                                                                                 \
public:

enum class engine_types : int32_t { ocl = cldnn_engine_ocl };
enum class priority_mode_types : int16_t { disabled = cldnn_priority_disabled, low, med, high };
enum class throttle_mode_types : int16_t { disabled = cldnn_throttle_disabled, low, med, high };

struct engine_configuration {
    bool enable_profiling;
    bool meaningful_kernels_names;
    bool dump_custom_program;
    std::string compiler_options;
    std::string single_kernel_name;
    bool enable_parallelisation;
    std::string engine_log;
    std::string sources_dumps_dir;
    priority_mode_types priority_mode;
    throttle_mode_types throttle_mode;
    bool enable_memory_pool;
    void* context;
    std::string tuning_cache_path;
    engine_configuration(bool profiling = false, bool decorate_kernel_names = false, bool dump_custom_program = false,
                         const std::string& options = std::string(), const std::string& single_kernel = std::string(),
                         bool primitives_parallelisation = false /* the reference's default is true; here the second stream costs more
                                                                    in cross-stream waits than it hides, so it is opt-in */,
                         const std::string& engine_log = std::string(),
                         const std::string& sources_dumps_dir = std::string(),
                         priority_mode_types priority_mode = priority_mode_types::disabled,
                         throttle_mode_types throttle_mode = throttle_mode_types::disabled, bool memory_pool = true,
                         void* context = nullptr, const std::string& tuning_cache = "cache.json")
        : enable_profiling(profiling), meaningful_kernels_names(decorate_kernel_names), dump_custom_program(dump_custom_program),
          compiler_options(options), single_kernel_name(single_kernel), enable_parallelisation(primitives_parallelisation),
          engine_log(engine_log), sources_dumps_dir(sources_dumps_dir), priority_mode(priority_mode), throttle_mode(throttle_mode),
          enable_memory_pool(memory_pool), context(context), tuning_cache_path(tuning_cache) {}
    operator ::cldnn_engine_configuration() const
    {
        return {enable_profiling, meaningful_kernels_names, dump_custom_program, compiler_options.c_str(), single_kernel_name.c_str(),
                enable_parallelisation, engine_log.c_str(), sources_dumps_dir.c_str(), (int16_t)priority_mode, (int16_t)throttle_mode,
                enable_memory_pool, context, tuning_cache_path.c_str()};
    }
};

using engine_info = ::cldnn_engine_info;

struct engine {
    engine(const engine_configuration& cfg = engine_configuration()) : engine(engine_types::ocl, 0, cfg) {}
    engine(engine_types type, uint32_t engine_num, const engine_configuration& cfg = engine_configuration())
        : _impl(check_status("create engine", [&](status_t* s) {
              ::cldnn_engine_configuration c = cfg;
              return ::cldnn_create_engine((int32_t)type, engine_num, &c, s);
          })) {}
    static uint32_t engine_count(engine_types type = engine_types::ocl)
    {
        return check_status("engine count", [&](status_t* s) { return ::cldnn_get_engine_count((int32_t)type, s); });
    }
    void release_pending_memory() const
    {
        check_status("release pending memory", [&](status_t* s) { ::cldnn_release_pending_memory(_impl, s); return 0; });
    }
    engine_info get_info() const
    {
        return check_status("engine info", [&](status_t* s) { return ::cldnn_get_engine_info(_impl, s); });
    }
    uint64_t get_max_used_device_memory_size() const
    {
        return (uint64_t)check_status("max used memory", [&](status_t* s) { return ::cldnn_get_max_used_device_memory_size(_impl, s); });
    }
    uint64_t get_temp_used_device_memory_size() const
    {
        return (uint64_t)check_status("used memory", [&](status_t* s) { return ::cldnn_get_temp_used_device_memory_size(_impl, s); });
    }
    engine_types get_type() const
    {
        return (engine_types)check_status("engine type", [&](status_t* s) { return ::cldnn_get_engine_type(_impl, s); });
    }
    CLDNN_CPP_HANDLE(engine, engine)
};

struct event {
    static event create_user_event(const engine& eng)
    {
        return event(check_status("create user event", [&](status_t* s) { return ::cldnn_create_user_event(eng.get(), s); }));
    }
    void wait() const
    {
        check_status("wait for event", [&](status_t* s) { ::cldnn_wait_for_event(_impl, s); return 0; });
    }
    void set() const
    {
        check_status("set event", [&](status_t* s) { ::cldnn_set_event(_impl, s); return 0; });
    }
    bool is_user_event() const
    {
        return check_status("is user event", [&](status_t* s) { return ::cldnn_is_user_event(_impl, s); }) != 0;
    }
    void set_event_handler(cldnn_event_handler handler, void* param) const
    {
        check_status("add event handler", [&](status_t* s) { ::cldnn_add_event_handler(_impl, handler, param, s); return 0; });
    }
    // (name, nanoseconds) of "submission", "starting", "executing"
    std::vector<std::pair<std::string, uint64_t>> get_profiling_info() const
    {
        cldnn_profiling_interval iv[8];
        size_t n = 0;
        check_status("profiling info", [&](status_t* s) { ::cldnn_get_event_profiling_info(_impl, iv, 8, &n, s); return 0; });
        std::vector<std::pair<std::string, uint64_t>> r;
        for (size_t i = 0; i < n; ++i) r.emplace_back(iv[i].name, iv[i].nanoseconds);
        return r;
    }
    CLDNN_CPP_HANDLE(event, event)
};

template <class T> struct pointer;

struct memory {
    static memory allocate(const engine& eng, const layout& l)
    {
        return memory(check_status("allocate memory", [&](status_t* s) { return ::cldnn_allocate_memory(eng.get(), l, s); }));
    }
    // wraps caller-owned host memory; `size` counts elements of T
    template <class T> static memory attach(const layout& l, T* ptr, size_t size)
    {
        if (!ptr) throw std::invalid_argument("pointer should not be null");
        if (size * sizeof(T) < l.bytes_count()) throw std::invalid_argument("buffer size mismatch - input size is less than layout size");
        return memory(check_status("attach memory", [&](status_t* s) { return ::cldnn_attach_memory(l, ptr, size * sizeof(T), s); }));
    }
    layout get_layout() const
    {
        return layout(check_status("memory layout", [&](status_t* s) { return ::cldnn_get_memory_layout(_impl, s); }));
    }
    size_t count() const { return get_layout().count(); }
    size_t size() const { return get_layout().bytes_count(); }
    bool is_allocated_by(const engine& eng) const
    {
        ::cldnn_engine e = check_status("memory engine", [&](status_t* s) { return ::cldnn_get_memory_engine(_impl, s); });
        if (!e) return false;
        status_t st;
        ::cldnn_release_engine(e, &st);
        return e == eng.get();
    }
    bool is_the_same_buffer(const memory& o) const
    {
        return check_status("same buffer", [&](status_t* s) { return ::cldnn_is_the_same_buffer(_impl, o._impl, s); }) != 0;
    }
    template <class T> cldnn::pointer<T> pointer() const;
    void* lock() const
    {
        return check_status("lock memory", [&](status_t* s) { return ::cldnn_lock_memory(_impl, s); });
    }
    void unlock() const
    {
        check_status("unlock memory", [&](status_t* s) { ::cldnn_unlock_memory(_impl, s); return 0; });
    }
    CLDNN_CPP_HANDLE(memory, memory)
};

// host view of a memory object for its lifetime: locks on construction, unlocks on destruction
template <class T> struct pointer {
    explicit pointer(const memory& mem) : _mem(mem), _size(mem.size() / sizeof(T)), _ptr(static_cast<T*>(mem.lock())) {}
    pointer(const pointer& o) : _mem(o._mem), _size(o._size), _ptr(static_cast<T*>(_mem.lock())) {}
    pointer& operator=(const pointer&) = delete;
    ~pointer()
    {
        try {
            _mem.unlock();
        } catch (...) {
        }
    }
    size_t size() const { return _size; }
    T* data() { return _ptr; }
    T* begin() { return _ptr; }
    T* end() { return _ptr + _size; }
    const T* begin() const { return _ptr; }
    const T* end() const { return _ptr + _size; }
    T& operator[](size_t i) { return _ptr[i]; }
    const T& operator[](size_t i) const { return _ptr[i]; }

private:
    memory _mem;
    size_t _size;
    T* _ptr;
};
template <class T> pointer<T> memory::pointer() const { return cldnn::pointer<T>(*this); }

// ------------------------------------------------------------------------------------------ primitives
using primitive_id = std::string;
using primitive_type_id = ::cldnn_primitive_type_id;

struct primitive {
    primitive_id id;
    std::vector<primitive_id> input;
    padding output_padding;
    optional_data_type output_data_type;
    virtual ~primitive() {}
    virtual const ::cldnn_primitive_desc* get_dto() const = 0;
    void set_output_data_type(data_types dt) { output_data_type = optional_data_type(dt); }

protected:
    primitive(const primitive_id& id, const std::vector<primitive_id>& in, const padding& pad, optional_data_type dt = optional_data_type())
        : id(id), input(in), output_padding(pad), output_data_type(dt) {}
    struct id_list {  // C view of a vector of ids
        std::vector<const char*> ptrs;
        cldnn_primitive_id_arr arr(const std::vector<primitive_id>& v)
        {
            ptrs.clear();
            for (auto& s : v) ptrs.push_back(s.c_str());
            return cldnn_primitive_id_arr{ptrs.data(), ptrs.size()};
        }
    };
    template <class Desc> void fill_base(Desc& d, primitive_type_id type, id_list& in) const
    {
        d.type = type;
        d.id = id.c_str();
        d.input = in.arr(input);
        d.output_padding = output_padding;
        d.output_data_type.enabled = output_data_type.has ? 1 : 0;
        d.output_data_type.data_type = (cldnn_data_type)output_data_type.value;
    }
};

#define CLDNN_CPP_TYPE_ID(name) \
    static primitive_type_id type_id() { return check_status(#name " type id", [&](status_t* s) { return ::cldnn_##name##_type_id(s); }); }

struct input_layout : primitive {
    cldnn::layout layout;
    input_layout(const primitive_id& id, const cldnn::layout& l) : primitive(id, {}, l.data_padding), layout(l) {}
    void change_layout(const cldnn::layout& l) { layout = l; }
    CLDNN_CPP_TYPE_ID(input_layout)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.layout = layout;
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    mutable cldnn_input_layout_desc _d{};
    mutable id_list _in;
};

struct data : primitive {
    memory mem;
    data(const primitive_id& id, const memory& m) : primitive(id, {}, padding()), mem(m) {}
    CLDNN_CPP_TYPE_ID(data)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.mem = mem.get();
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    mutable cldnn_data_desc _d{};
    mutable id_list _in;
};

struct reorder : primitive {
    format output_format;
    reorder(const primitive_id& id, const primitive_id& input, const layout& output_layout)
        : primitive(id, {input}, output_layout.data_padding, optional_data_type(output_layout.data_type)), output_format(output_layout.format) {}
    reorder(const primitive_id& id, const primitive_id& input, format output_format, data_types output_data_type,
            const padding& output_padding = padding())
        : primitive(id, {input}, output_padding, optional_data_type(output_data_type)), output_format(output_format) {}
    CLDNN_CPP_TYPE_ID(reorder)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.output_format = (cldnn_format_type)output_format.value;
        _d.mean_subtract = "";
        _d.subtract_per_feature = cldnn_float_arr{nullptr, 0};
        _d.mean_mode = mean_none;
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    mutable cldnn_reorder_desc _d{};
    mutable id_list _in;
};

struct activation : primitive {
    cldnn_activation_func activation_func;
    cldnn_activation_additional_params additional_params;
    activation(const primitive_id& id, const primitive_id& input, cldnn_activation_func func,
               cldnn_activation_additional_params params = {0.f, 0.f}, const padding& output_padding = padding())
        : primitive(id, {input}, output_padding), activation_func(func), additional_params(params) {}
    CLDNN_CPP_TYPE_ID(activation)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.activation_func = activation_func;
        _d.additional_params = additional_params;
        _d.additional_params_input = "";
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    mutable cldnn_activation_desc _d{};
    mutable id_list _in;
};

enum class pooling_mode : int32_t {
    max = cldnn_pooling_max,
    average = cldnn_pooling_average,
    average_no_padding = cldnn_pooling_average_no_padding,
    max_with_argmax = cldnn_pooling_max_with_argmax,
    bilinear = cldnn_pooling_bilinear
};

// pooling(id, input, mode, size, stride, input_offset), with a user-given output size, or global over the whole plane
// (reference api/CPP/pooling.hpp:59-190); the argmax forms are not implemented
struct pooling : primitive {
    pooling_mode mode;
    bool global_pooling;
    tensor input_offset{0}, stride{1}, size{0}, output_size{0};
    bool with_output_size = false;
    pooling(const primitive_id& id, const primitive_id& input, pooling_mode mode, const tensor& size, const tensor& stride,
            const tensor& input_offset = {0, 0, 0, 0}, const padding& output_padding = padding())
        : primitive(id, {input}, output_padding), mode(mode), global_pooling(false), input_offset(input_offset), stride(stride), size(size) {}
    pooling(const primitive_id& id, const primitive_id& input, pooling_mode mode, const tensor& size, const tensor& stride,
            const tensor& input_offset, tensor output_size, const padding& output_padding = padding())
        : primitive(id, {input}, output_padding), mode(mode), global_pooling(false), input_offset(input_offset), stride(stride), size(size),
          output_size(output_size), with_output_size(true) {}
    pooling(const primitive_id& id, const primitive_id& input, pooling_mode mode, const padding& output_padding = padding())
        : primitive(id, {input}, output_padding), mode(mode), global_pooling(true) {}
    static pooling create_with_output_size(const primitive_id& id, const primitive_id& input, tensor output_size, pooling_mode mode,
                                           const tensor& size, const tensor& stride, const tensor& input_offset = {0, 0, 0, 0},
                                           const padding& output_padding = padding())
    {
        return pooling(id, input, mode, size, stride, input_offset, output_size, output_padding);
    }
    CLDNN_CPP_TYPE_ID(pooling)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.argmax = "";
        _d.mode = static_cast<int32_t>(mode);
        _d.global_pooling = global_pooling;
        _d.input_offset = input_offset, _d.stride = stride, _d.size = size;
        _d.with_output_size = with_output_size, _d.output_size = output_size;
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    mutable cldnn_pooling_desc _d{};
    mutable id_list _in;
};

// concatenation(id, inputs, axis) (reference api/CPP/concatenation.hpp:54-92); along_z is not available
struct concatenation : primitive {
    enum concatenation_axis {
        along_b = cldnn_concatenation_along_b,
        along_f = cldnn_concatenation_along_f,
        along_x = cldnn_concatenation_along_x,
        along_y = cldnn_concatenation_along_y
    };
    concatenation_axis axis;
    concatenation(const primitive_id& id, const std::vector<primitive_id>& input, const concatenation_axis axis,
                  const padding& output_padding = padding())
        : primitive(id, input, output_padding), axis(axis) {}
    CLDNN_CPP_TYPE_ID(concatenation)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.axis = static_cast<cldnn_concatenation_axis>(axis);
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    mutable cldnn_concatenation_desc _d{};
    mutable id_list _in;
};

// fully_connected(id, input, weights, bias, with_activation, slope) and the quantized forms with
// w_quantization_factor [, output_calibration_factors], i_quantization_factor [, o_quantization_factor]
// (reference api/CPP/fully_connected.hpp:60-150)
struct fully_connected : primitive {
    primitive_id weights, bias, weights_quantization_factors, output_calibration_factors;
    float input_quantization_factor = 1.0f, output_quantization_factor = 1.0f;
    bool with_activation;
    float activation_negative_slope;
    fully_connected(const primitive_id& id, const primitive_id& input, const primitive_id& weights, const primitive_id& bias = "",
                    bool with_activation = false, float activation_slp = 0.0f, const padding& output_padding = padding())
        : primitive(id, {input}, output_padding), weights(weights), bias(bias), with_activation(with_activation),
          activation_negative_slope(activation_slp) {}
    fully_connected(const primitive_id& id, const primitive_id& input, const primitive_id& weights, const primitive_id& bias,
                    const primitive_id& w_quantization_factor, const float i_quantization_factor, const float o_quantization_factor,
                    bool with_activation = false, float activation_slp = 0.0f, const padding& output_padding = padding())
        : primitive(id, {input}, output_padding), weights(weights), bias(bias), weights_quantization_factors(w_quantization_factor),
          input_quantization_factor(i_quantization_factor), output_quantization_factor(o_quantization_factor),
          with_activation(with_activation), activation_negative_slope(activation_slp) {}
    fully_connected(const primitive_id& id, const primitive_id& input, const primitive_id& weights, const primitive_id& bias,
                    const primitive_id& w_quantization_factor, const primitive_id& output_calibration_factors,
                    const float i_quantization_factor, bool with_activation = false, float activation_slp = 0.0f,
                    const padding& output_padding = padding())
        : primitive(id, {input}, output_padding), weights(weights), bias(bias), weights_quantization_factors(w_quantization_factor),
          output_calibration_factors(output_calibration_factors), input_quantization_factor(i_quantization_factor),
          with_activation(with_activation), activation_negative_slope(activation_slp) {}
    CLDNN_CPP_TYPE_ID(fully_connected)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.with_activation = with_activation, _d.activation_negative_slope = activation_negative_slope;
        _d.weights = weights.c_str(), _d.bias = bias.c_str();
        _d.weights_quantization_factors = weights_quantization_factors.c_str();
        _d.output_calibration_factors = output_calibration_factors.c_str();
        _d.input_quantization_factor = input_quantization_factor, _d.output_quantization_factor = output_quantization_factor;
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    mutable cldnn_fully_connected_desc _d{};
    mutable id_list _in;
};

enum class eltwise_mode : int32_t { sum = cldnn_eltwise_sum, sub = cldnn_eltwise_sub, max = cldnn_eltwise_max, prod = cldnn_eltwise_prod,
                                    div = cldnn_eltwise_div, min = cldnn_eltwise_min, pow = cldnn_eltwise_pow, mod = cldnn_eltwise_mod };

struct eltwise : primitive {
    primitive_id output_calibration_factors;
    float output_quantization_factor = 1.0f;
    eltwise_mode mode;
    std::vector<float> coefficients;
    std::vector<tensor> stride;
    bool with_activation;
    float activation_negative_slope;
    // any number of inputs, combined left to right (reference api/CPP/eltwise.hpp:196-225 and 279-311)
    eltwise(const primitive_id& id, const std::vector<primitive_id>& inputs, eltwise_mode mode, bool with_activation = false,
            float activation_slp = 0.0f, const padding& output_padding = padding())
        : primitive(id, inputs, output_padding), mode(mode), with_activation(with_activation), activation_negative_slope(activation_slp) {}
    eltwise(const primitive_id& id, const std::vector<primitive_id>& inputs, eltwise_mode mode, const std::vector<float>& coefficients,
            bool with_activation = false, float activation_slp = 0.0f, const padding& output_padding = padding())
        : primitive(id, inputs, output_padding), mode(mode), coefficients(coefficients), with_activation(with_activation),
          activation_negative_slope(activation_slp)
    {
        if (mode == eltwise_mode::sum && !coefficients.empty() && coefficients.size() != inputs.size())
            throw std::invalid_argument("Invalid eltwise sum coefficients count (should be equal to 0 or input.size)");
        if (mode != eltwise_mode::sum && !coefficients.empty())
            throw std::invalid_argument("Only eltwise sum operation supports blob-wise coefficients");
    }
    eltwise(const primitive_id& id, const primitive_id& input, const primitive_id& input2, eltwise_mode mode, bool with_activation = false,
            float activation_slp = 0.0f, const padding& output_padding = padding())
        : primitive(id, {input, input2}, output_padding), mode(mode), with_activation(with_activation), activation_negative_slope(activation_slp) {}
    eltwise(const primitive_id& id, const primitive_id& input, const primitive_id& input2, std::vector<tensor> stride, eltwise_mode mode,
            bool with_activation = false, float activation_slp = 0.0f, const padding& output_padding = padding())
        : primitive(id, {input, input2}, output_padding), mode(mode), stride(std::move(stride)), with_activation(with_activation),
          activation_negative_slope(activation_slp) {}
    eltwise(const primitive_id& id, const primitive_id& input, const primitive_id& input2, const primitive_id& output_calibration_factors,
            eltwise_mode mode, bool with_activation = false, float activation_slp = 0.0f, const padding& output_padding = padding())
        : primitive(id, {input, input2}, output_padding), output_calibration_factors(output_calibration_factors), mode(mode),
          with_activation(with_activation), activation_negative_slope(activation_slp) {}
    eltwise(const primitive_id& id, const primitive_id& input, const primitive_id& input2, const float o_quantization_factor, eltwise_mode mode,
            bool with_activation = false, float activation_slp = 0.0f, const padding& output_padding = padding())
        : primitive(id, {input, input2}, output_padding), output_quantization_factor(o_quantization_factor), mode(mode),
          with_activation(with_activation), activation_negative_slope(activation_slp) {}
    CLDNN_CPP_TYPE_ID(eltwise)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.output_calibration_factors = output_calibration_factors.c_str();
        _d.output_quantization_factor = output_quantization_factor;
        _d.mode = (int32_t)mode;
        _d.coefficients = cldnn_float_arr{coefficients.data(), coefficients.size()};
        _d.with_activation = with_activation;
        _d.activation_negative_slope = activation_negative_slope;
        _strides.assign(stride.begin(), stride.end());
        _d.stride = cldnn_tensor_arr{_strides.data(), _strides.size()};
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    mutable cldnn_eltwise_desc _d{};
    mutable id_list _in;
    mutable std::vector<cldnn_tensor> _strides;
};

struct convolution : primitive {
    tensor input_offset, stride, dilation;
    bool with_activation;
    float activation_negative_slope;
    bool with_output_size = false;
    tensor output_size{0};
    uint32_t groups = 1;
    tensor padding_above{0}, padding_below{0};
    std::vector<primitive_id> weights, bias, weights_quantization_factors, output_calibration_factors;
    float input_quantization_factor = 1.0f, output_quantization_factor = 1.0f;

    // weights + bias
    convolution(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights, const std::vector<primitive_id>& bias,
                tensor stride = {1, 1, 1, 1}, tensor input_offset = {0, 0, 0, 0, 0}, tensor dilation = {1, 1, 1, 1}, bool with_activation = false,
                float activation_slp = 0.0f, const padding& output_padding = padding())
        : primitive(id, {input}, output_padding), input_offset(input_offset), stride(stride), dilation(dilation), with_activation(with_activation),
          activation_negative_slope(activation_slp), weights(weights), bias(bias) { validate(); }
    // weights + bias + explicit padding above / below
    convolution(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights, const std::vector<primitive_id>& bias,
                tensor stride, tensor input_offset, tensor dilation, tensor padding_above, tensor padding_below, bool with_activation = false,
                float activation_slp = 0.0f, const padding& output_padding = padding())
        : convolution(id, input, weights, bias, stride, input_offset, dilation, with_activation, activation_slp, output_padding)
    {
        this->padding_above = padding_above, this->padding_below = padding_below;
    }
    // grouped
    convolution(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights, const std::vector<primitive_id>& bias,
                uint32_t groups, tensor stride = {1, 1, 1, 1}, tensor input_offset = {0, 0, 0, 0, 0}, tensor dilation = {1, 1, 1, 1},
                bool with_activation = false, float activation_slp = 0.0f, const padding& output_padding = padding())
        : convolution(id, input, weights, bias, stride, input_offset, dilation, with_activation, activation_slp, output_padding)
    {
        this->groups = groups;
    }
    // quantized: per-feature weight factors, scalar input / output factors
    convolution(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights, const std::vector<primitive_id>& bias,
                const std::vector<primitive_id>& w_quantization_factor, const float i_quantization_factor, const float o_quantization_factor,
                tensor stride = {1, 1, 1, 1}, tensor input_offset = {0, 0, 0, 0, 0}, tensor dilation = {1, 1, 1, 1}, bool with_activation = false,
                float activation_slp = 0.0f, const padding& output_padding = padding())
        : convolution(id, input, weights, bias, stride, input_offset, dilation, with_activation, activation_slp, output_padding)
    {
        weights_quantization_factors = w_quantization_factor;
        input_quantization_factor = i_quantization_factor, output_quantization_factor = o_quantization_factor;
        validate();
    }
    // quantized with an explicit output type
    convolution(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights, const std::vector<primitive_id>& bias,
                const std::vector<primitive_id>& quantization_factors, data_types output_data_type, tensor stride = {1, 1, 1, 1},
                tensor input_offset = {0, 0, 0, 0}, tensor dilation = {1, 1, 1, 1}, bool with_activation = false, float activation_slp = 0.0f,
                const padding& output_padding = padding())
        : convolution(id, input, weights, bias, stride, input_offset, dilation, with_activation, activation_slp, output_padding)
    {
        weights_quantization_factors = quantization_factors;
        set_output_data_type(output_data_type);
        validate();
    }
    // quantized with per-feature output calibration
    convolution(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights, const std::vector<primitive_id>& bias,
                const std::vector<primitive_id>& w_quantization_factor, const std::vector<primitive_id>& output_calibration_factors,
                const float i_quantization_factor, tensor stride = {1, 1, 1, 1}, tensor input_offset = {0, 0, 0, 0, 0},
                tensor dilation = {1, 1, 1, 1}, bool with_activation = false, float activation_slp = 0.0f, const padding& output_padding = padding())
        : convolution(id, input, weights, bias, stride, input_offset, dilation, with_activation, activation_slp, output_padding)
    {
        weights_quantization_factors = w_quantization_factor;
        this->output_calibration_factors = output_calibration_factors;
        input_quantization_factor = i_quantization_factor;
        validate();
    }
    // no bias
    convolution(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights, tensor stride = {1, 1, 1, 1},
                tensor input_offset = {0, 0, 0, 0, 0}, tensor dilation = {1, 1, 1, 1}, bool with_activation = false, float activation_slp = 0.0f,
                const padding& output_padding = padding())
        : convolution(id, input, weights, std::vector<primitive_id>(), stride, input_offset, dilation, with_activation, activation_slp,
                      output_padding) {}
    // no bias, grouped
    convolution(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights, uint32_t groups,
                tensor stride = {1, 1, 1, 1}, tensor input_offset = {0, 0, 0, 0, 0}, tensor dilation = {1, 1, 1, 1}, bool with_activation = false,
                float activation_slp = 0.0f, const padding& output_padding = padding())
        : convolution(id, input, weights, std::vector<primitive_id>(), groups, stride, input_offset, dilation, with_activation, activation_slp,
                      output_padding) {}
    // user-defined output size
    convolution(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights, const std::vector<primitive_id>& bias,
                tensor stride, tensor input_offset, tensor dilation, bool with_activation, float activation_slp, tensor output_size,
                const padding& output_padding = padding())
        : convolution(id, input, weights, bias, stride, input_offset, dilation, with_activation, activation_slp, output_padding)
    {
        with_output_size = true;
        this->output_size = output_size;
    }
    static convolution create_with_output_size(const primitive_id& id, const primitive_id& input, const std::vector<primitive_id>& weights,
                                               const std::vector<primitive_id>& bias, tensor output_size, tensor stride = {1, 1, 1, 1},
                                               tensor input_offset = {0, 0, 0, 0, 0}, tensor dilation = {1, 1, 1, 1},
                                               bool with_activation = false, float activation_slp = 0.0f, const padding& output_padding = padding())
    {
        return convolution(id, input, weights, bias, stride, input_offset, dilation, with_activation, activation_slp, output_size, output_padding);
    }
    int32_t split() const { return static_cast<int32_t>(weights.size()); }
    CLDNN_CPP_TYPE_ID(convolution)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.input_offset = input_offset, _d.stride = stride, _d.dilation = dilation;
        _d.with_activation = with_activation, _d.activation_negative_slope = activation_negative_slope;
        _d.split = (uint32_t)weights.size();
        _d.with_output_size = with_output_size, _d.output_size = output_size;
        _d.weights = _w.arr(weights), _d.bias = _b.arr(bias);
        _d.weights_quantization_factors = _q.arr(weights_quantization_factors);
        _d.output_calibration_factors = _c.arr(output_calibration_factors);
        _d.input_quantization_factor = input_quantization_factor, _d.output_quantization_factor = output_quantization_factor;
        _d.groups = groups;
        _d.padding_above = padding_above, _d.padding_below = padding_below;
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    void validate() const
    {
        if (!bias.empty() && weights.size() != bias.size()) throw std::runtime_error("convolution's weights/bias count does not match");
        if (!output_calibration_factors.empty() && weights.size() != weights_quantization_factors.size())
            throw std::runtime_error("convolution's weights count does not match quantization factors count");
    }
    mutable cldnn_convolution_desc _d{};
    mutable id_list _in, _w, _b, _q, _c;
};

struct fused_conv_eltwise : primitive {
    struct conv_data {
        std::vector<primitive_id> weights, bias, weights_quantization_factors, output_calibration_factors;
        float input_quantization_factor = 1.0f, output_quantization_factor = 1.0f;
        tensor input_offset, stride, dilation;
        bool with_activation = false;
        float activation_negative_slope = 0.0f;
        bool with_output_size = false;
        tensor output_size{0};
    } conv;
    struct eltw_data {
        primitive_id output_calibration_factors;
        float output_quantization_factor = 1.0f;
        eltwise_mode mode = eltwise_mode::sum;
        bool with_activation = false;
        float activation_negative_slope = 0.0f;
        std::vector<tensor> stride;
    } eltw;
    float non_conv_scale = 1.0f;
    bool second_input_in_output = false;

    fused_conv_eltwise(const primitive_id& id, const primitive_id& input, const primitive_id& input2, eltwise_mode mode,
                       const std::vector<primitive_id>& weights, const std::vector<primitive_id>& bias,
                       const std::vector<primitive_id>& conv_w_quantization_factor,
                       const std::vector<primitive_id>& conv_output_calibration_factors, const float conv_i_quantization_factor,
                       const float non_conv_scale, const primitive_id& eltw_output_calibration_factors, const std::vector<tensor>& eltw_stride,
                       tensor stride = {1, 1, 1, 1}, tensor input_offset = {0, 0, 0, 0}, tensor dilation = {1, 1, 1, 1},
                       bool conv_with_activation = false, float conv_activation_slp = 0.0f, bool eltw_with_activation = false,
                       float eltw_activation_slp = 0.0f, const padding& output_padding = padding(),
                       optional_data_type output_data_type = optional_data_type())
        : primitive(id, {input, input2}, output_padding, output_data_type), non_conv_scale(non_conv_scale)
    {
        conv.weights = weights, conv.bias = bias;
        conv.weights_quantization_factors = conv_w_quantization_factor;
        conv.output_calibration_factors = conv_output_calibration_factors;
        conv.input_quantization_factor = conv_i_quantization_factor;
        conv.input_offset = input_offset, conv.stride = stride, conv.dilation = dilation;
        conv.with_activation = conv_with_activation, conv.activation_negative_slope = conv_activation_slp;
        eltw.output_calibration_factors = eltw_output_calibration_factors;
        eltw.mode = mode;
        eltw.with_activation = eltw_with_activation, eltw.activation_negative_slope = eltw_activation_slp;
        eltw.stride = eltw_stride;
        if (!bias.empty() && weights.size() != bias.size()) throw std::runtime_error("convolution's weights/bias count does not match");
        if (!conv.output_calibration_factors.empty() && weights.size() != conv.weights_quantization_factors.size())
            throw std::runtime_error("convolution's weights count does not match quantization factors count");
    }
    CLDNN_CPP_TYPE_ID(fused_conv_eltwise)
    const ::cldnn_primitive_desc* get_dto() const override
    {
        fill_base(_d, type_id(), _in);
        _d.conv.input_offset = conv.input_offset, _d.conv.stride = conv.stride, _d.conv.dilation = conv.dilation;
        _d.conv.with_activation = conv.with_activation, _d.conv.activation_negative_slope = conv.activation_negative_slope;
        _d.conv.split = (uint32_t)conv.weights.size();
        _d.conv.with_output_size = conv.with_output_size, _d.conv.output_size = conv.output_size;
        _d.conv.weights = _w.arr(conv.weights), _d.conv.bias = _b.arr(conv.bias);
        _d.conv.weights_quantization_factors = _q.arr(conv.weights_quantization_factors);
        _d.conv.output_calibration_factors = _c.arr(conv.output_calibration_factors);
        _d.conv.input_quantization_factor = conv.input_quantization_factor;
        _d.conv.output_quantization_factor = conv.output_quantization_factor;
        _d.eltw.output_calibration_factors = eltw.output_calibration_factors.c_str();
        _d.eltw.output_quantization_factor = eltw.output_quantization_factor;
        _d.eltw.mode = (int32_t)eltw.mode;
        _d.eltw.coefficients = cldnn_float_arr{nullptr, 0};
        _d.eltw.with_activation = eltw.with_activation, _d.eltw.activation_negative_slope = eltw.activation_negative_slope;
        _strides.assign(eltw.stride.begin(), eltw.stride.end());
        _d.eltw.stride = cldnn_tensor_arr{_strides.data(), _strides.size()};
        _d.non_conv_scale = non_conv_scale;
        _d.second_input_in_output = second_input_in_output;
        return reinterpret_cast<const ::cldnn_primitive_desc*>(&_d);
    }

private:
    mutable cldnn_fused_conv_eltwise_desc _d{};
    mutable id_list _in, _w, _b, _q, _c;
    mutable std::vector<cldnn_tensor> _strides;
};

// ------------------------------------------------------------------------------------------ topology / program / network
struct topology {
    topology() : _impl(check_status("create topology", [&](status_t* s) { return ::cldnn_create_topology(s); })) {}
    template <class... Args> explicit topology(const Args&... args) : topology() { add_all(args...); }
    template <class PType> void add(PType const& desc)
    {
        check_status("add primitive", [&](status_t* s) { ::cldnn_add_primitive(_impl, desc.get_dto(), s); return 0; });
    }
    template <class PType, class... Args> void add(PType const& desc, Args const&... args)
    {
        add(desc);
        add(args...);
    }
    void change_input_layout(const primitive_id& id, const layout& new_layout)
    {
        check_status("change input layout", [&](status_t* s) { ::cldnn_change_input_layout(_impl, id.c_str(), new_layout, s); return 0; });
    }
    std::vector<primitive_id> get_primitive_ids() const;
    CLDNN_CPP_HANDLE(topology, topology)
private:
    void add_all() {}
    template <class P, class... Args> void add_all(const P& p, const Args&... rest)
    {
        add(p);
        add_all(rest...);
    }
};

namespace detail {
// names returned as "a\0b\0\0" through the (buffer, size, size_ret) protocol of the C API
template <class F> std::vector<primitive_id> names(const char* what, F&& call)
{
    size_t need = 0;
    status_t st;
    call((char*)nullptr, (size_t)0, &need, &st);  // size query: reports the size through size_ret
    if (need == 0) throw error(std::string(what) + ": " + ::cldnn_get_last_error_message(), st);
    std::vector<char> buf(need);
    check_status(what, [&](status_t* s) { call(buf.data(), buf.size(), &need, s); return 0; });
    std::vector<primitive_id> r;
    for (size_t i = 0; i < need && buf[i];) {
        r.emplace_back(&buf[i]);
        i += r.back().size() + 1;
    }
    return r;
}
}  // namespace detail

inline std::vector<primitive_id> topology::get_primitive_ids() const
{
    return detail::names("primitive ids", [&](char* b, size_t n, size_t* r, status_t* s) { ::cldnn_get_primitive_ids(_impl, b, n, r, s); });
}

enum class build_option_type : int32_t {
    fusing = cldnn_build_option_fusing,
    optimize_data = cldnn_build_option_optimize_data,
    debug = cldnn_build_option_debug,
    outputs = cldnn_build_option_outputs,
    tuning_config = cldnn_build_option_tuning_config,
    graph_dumps_dir = cldnn_build_option_graph_dumps_dir,
    learning_config = cldnn_build_option_learning_config
};

// reference api/CPP/program.hpp:68-93
enum class tuning_mode : int32_t {
    tuning_disabled = cldnn_tuning_disabled,
    tuning_use_cache = cldnn_tuning_use_cache,
    tuning_tune_and_cache = cldnn_tuning_tune_and_cache
};
struct tuning_config_options {
    tuning_mode mode = tuning_mode::tuning_disabled;
    std::string cache_file_path;
};

struct build_option {
    build_option_type type;
    bool enabled = true;
    std::vector<primitive_id> ids;
    tuning_config_options tuning;
    static build_option tuning_config(const tuning_config_options& config = tuning_config_options())
    {
        return {build_option_type::tuning_config, true, {}, config};
    }
    static build_option fusing(bool enable = false) { return {build_option_type::fusing, enable, {}}; }
    static build_option optimize_data(bool enable = false) { return {build_option_type::optimize_data, enable, {}}; }
    static build_option debug(bool enable = false) { return {build_option_type::debug, enable, {}}; }
    static build_option outputs(const std::vector<primitive_id>& outs) { return {build_option_type::outputs, true, outs}; }
};

struct build_options {
    build_options() {}
    template <class... Args> build_options(const build_option& o, const Args&... rest) { set_option(o, rest...); }
    void set_option(const build_option& o)
    {
        for (auto& e : _opts)
            if (e.type == o.type) {
                e = o;
                return;
            }
        _opts.push_back(o);
    }
    template <class... Args> void set_option(const build_option& o, const Args&... rest)
    {
        set_option(o);
        set_option(rest...);
    }
    // C view; valid while this object and `keep` live
    struct c_view {
        std::vector<cldnn_build_option> opts;
        std::vector<std::vector<const char*>> ptrs;
        std::vector<cldnn_primitive_id_arr> arrs;
        std::vector<cldnn_tuning_config> tuning;
    };
    std::unique_ptr<c_view> get_refs() const
    {
        std::unique_ptr<c_view> v(new c_view());
        v->ptrs.reserve(_opts.size());
        v->arrs.reserve(_opts.size());
        v->tuning.reserve(_opts.size());
        for (auto& o : _opts) {
            if (!o.enabled) continue;
            if (o.type == build_option_type::tuning_config) {
                v->tuning.push_back(cldnn_tuning_config{(int32_t)o.tuning.mode, o.tuning.cache_file_path.c_str()});
                v->opts.push_back(cldnn_build_option{(int32_t)o.type, &v->tuning.back()});
            } else if (o.type == build_option_type::outputs) {
                v->ptrs.emplace_back();
                for (auto& s : o.ids) v->ptrs.back().push_back(s.c_str());
                v->arrs.push_back(cldnn_primitive_id_arr{v->ptrs.back().data(), v->ptrs.back().size()});
                v->opts.push_back(cldnn_build_option{(int32_t)o.type, &v->arrs.back()});
            } else {
                v->opts.push_back(cldnn_build_option{(int32_t)o.type, nullptr});
            }
        }
        return v;
    }

private:
    std::vector<build_option> _opts;
};

struct program {
    program(const engine& eng, const topology& topo, const build_options& options = build_options())
        : _impl(check_status("build program", [&](status_t* s) {
              auto v = options.get_refs();
              return ::cldnn_build_program(eng.get(), topo.get(), v->opts.data(), v->opts.size(), s);
          })) {}
    CLDNN_CPP_HANDLE(program, program)
};

struct network_output {
    event get_event() const { return _event; }
    memory get_memory() const
    {
        _event.wait();
        return _result;
    }
    network_output(::cldnn_event ev, ::cldnn_memory mem) : _event(ev), _result(mem) {}

private:
    event _event;
    memory _result;
};

struct network {
    network(const program& prog) : _impl(check_status("allocate network", [&](status_t* s) { return ::cldnn_allocate_network(prog.get(), s); })) {}
    network(const engine& eng, const topology& topo, const build_options& options = build_options())
        : _impl(check_status("build network", [&](status_t* s) {
              auto v = options.get_refs();
              return ::cldnn_build_network(eng.get(), topo.get(), v->opts.data(), v->opts.size(), s);
          })) {}
    engine get_engine() const
    {
        return engine(check_status("network engine", [&](status_t* s) { return ::cldnn_get_network_engine(_impl, s); }));
    }
    program get_program() const
    {
        return program(check_status("network program", [&](status_t* s) { return ::cldnn_get_network_program(_impl, s); }));
    }
    void set_input_data(const primitive_id& id, const memory& mem) const
    {
        check_status("set network input", [&](status_t* s) { ::cldnn_set_network_input(_impl, id.c_str(), mem.get(), s); return 0; });
    }
    std::string get_primitive_info(const primitive_id& id) const
    {
        size_t need = 0;
        status_t st;
        ::cldnn_get_primitive_info(_impl, id.c_str(), nullptr, 0, &need, &st);
        if (need == 0) throw error(std::string("primitive info: ") + ::cldnn_get_last_error_message(), st);
        std::vector<char> buf(need);
        check_status("primitive info", [&](status_t* s) { ::cldnn_get_primitive_info(_impl, id.c_str(), buf.data(), need, &need, s); return 0; });
        return std::string(buf.data());
    }
    std::vector<primitive_id> get_output_ids() const
    {
        return detail::names("output ids", [&](char* b, size_t n, size_t* r, status_t* s) { ::cldnn_get_network_output_names(_impl, b, n, r, s); });
    }
    std::vector<primitive_id> get_executed_primitive_ids() const
    {
        return detail::names("executed ids",
                             [&](char* b, size_t n, size_t* r, status_t* s) { ::cldnn_get_network_executed_primitive_names(_impl, b, n, r, s); });
    }
    std::vector<primitive_id> get_all_primitive_ids() const
    {
        return detail::names("all ids", [&](char* b, size_t n, size_t* r, status_t* s) { ::cldnn_get_network_all_primitive_names(_impl, b, n, r, s); });
    }
    std::vector<primitive_id> get_all_primitive_org_ids() const
    {
        return detail::names("all original ids",
                             [&](char* b, size_t n, size_t* r, status_t* s) { ::cldnn_get_network_all_primitive_org_names(_impl, b, n, r, s); });
    }
    network_output get_output(const primitive_id& id) const
    {
        cldnn_network_output o = check_status("network output", [&](status_t* s) { return ::cldnn_get_network_output(_impl, id.c_str(), s); });
        return network_output(o.event, o.memory);  // the wrappers take over the references the call returned
    }
    memory get_output_memory(const primitive_id& id) const
    {
        ::cldnn_memory m = check_status("output memory", [&](status_t* s) { return ::cldnn_get_network_output_memory(_impl, id.c_str(), s); });
        return memory(m);
    }
    std::map<primitive_id, network_output> execute(const std::vector<event>& dependencies = {}) const
    {
        std::vector<::cldnn_event> deps;
        for (auto& e : dependencies) deps.push_back(e.get());
        check_status("execute network", [&](status_t* s) { ::cldnn_execute_network(_impl, deps.data(), deps.size(), s); return 0; });
        std::map<primitive_id, network_output> result;
        for (auto& id : get_output_ids()) result.emplace(id, get_output(id));
        return result;
    }
    CLDNN_CPP_HANDLE(network, network)
};

}  // namespace cldnn
