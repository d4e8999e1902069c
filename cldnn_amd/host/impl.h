// Internal objects behind the handles of the clDNN-compatible C API (include/api/C/cldnn.h).
// Small counterpart of the reference's core runtime (src/include/{engine,memory,event,topology,
// program,network}_impl.h, refcounted_obj.h) for the one path this library serves.
#pragma once
#include <atomic>
#include <condition_variable>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/api/C/primitives.h"
#include "../../include/cldnn_hip.h"

namespace host {

struct api_error : std::runtime_error {
    cldnn_status status;
    api_error(cldnn_status s, const std::string& m) : std::runtime_error(m), status(s) {}
};
#define HOST_REQUIRE(cond, status, msg)                     \
    do {                                                    \
        if (!(cond)) throw ::host::api_error((status), (msg)); \
    } while (0)
void hip_check(cldnn_hip_status s);  // throws api_error carrying the HIP layer's message

// intrusive reference counting (reference src/include/refcounted_obj.h:33-66)
struct refcounted {
    std::atomic<int> refs{1};
    virtual ~refcounted() {}
    void retain() { refs.fetch_add(1); }
    void release()
    {
        if (refs.fetch_sub(1) == 1) delete this;
    }
};
template <class T>
struct ref {  // owning smart pointer for refcounted objects
    T* p = nullptr;
    ref() {}
    explicit ref(T* q, bool add_ref) : p(q)
    {
        if (p && add_ref) p->retain();
    }
    ref(const ref& o) : p(o.p)
    {
        if (p) p->retain();
    }
    ref& operator=(const ref& o)
    {
        if (o.p) o.p->retain();
        if (p) p->release();
        p = o.p;
        return *this;
    }
    ~ref()
    {
        if (p) p->release();
    }
    T* operator->() const { return p; }
    T* get() const { return p; }
    explicit operator bool() const { return p != nullptr; }
};

enum class prim_type { input_layout, data, reorder, activation, eltwise, convolution, fused_conv_eltwise, pooling, concatenation };

// which row of the tile-config table a convolution runs on, measured once and kept in a JSON file (tuning_cache.cpp)
struct tuning_cache {
    std::string path;
    int mode = cldnn_tuning_disabled;
    std::map<std::string, std::map<std::string, std::pair<std::string, int>>> entries;  // compute units -> signature -> (row name, row)
    bool dirty = false;
    void load(const std::string& file, int tuning_mode);
    bool find(uint32_t compute_units, const std::string& key, std::string* name, int* index) const;
    void store(uint32_t compute_units, const std::string& key, const std::string& name, int index);
    void save();
};
std::string conv_signature(const cldnn_hip_conv_desc& d);

}  // namespace host

struct cldnn_engine_impl : host::refcounted {
    cldnn_hip_engine h = nullptr;
    cldnn_hip_engine side = nullptr;  // second stream for primitives nothing waits for yet (enable_parallelisation)
    bool profiling = false;
    std::string tuning_cache_path = "cache.json";  // engine configuration; a tuning_config without a path of its own uses it
    bool memory_pool = true;  // networks share buffers between intermediate tensors whose lifetimes do not overlap
    ~cldnn_engine_impl() override;
};

struct cldnn_memory_impl : host::refcounted {
    cldnn_layout layout{};
    host::ref<cldnn_engine_impl> engine;  // empty for attached host memory
    cldnn_hip_buffer buf = nullptr;
    void* attached = nullptr;
    size_t attached_bytes = 0;
    host::ref<cldnn_memory_impl> view_of;  // a window into another memory's buffer (input of an in-place concatenation)
    size_t view_offset = 0;
    ~cldnn_memory_impl() override;
    void* device_ptr() const
    {
        if (view_of) return (char*)view_of->device_ptr() + view_offset;
        return buf ? cldnn_hip_buffer_device_ptr(buf) : nullptr;
    }
};

struct cldnn_event_impl : host::refcounted {
    host::ref<cldnn_engine_impl> engine;
    cldnn_hip_event h = nullptr;
    ~cldnn_event_impl() override;
};

namespace host {

// deep copy of a primitive descriptor
struct prim {
    prim_type type;
    std::string id;
    std::vector<std::string> inputs;
    cldnn_padding output_padding{};
    cldnn_optional_data_type out_dt{};
    // input_layout
    cldnn_layout layout{};
    // data
    ref<cldnn_memory_impl> mem;
    // reorder
    int32_t reorder_format = cldnn_format_any;
    // activation
    int32_t act_func = activation_none;
    float act_a = 0.f, act_b = 0.f;
    // pooling (shares input_offset / stride / output_size / with_output_size with the convolution fields)
    int32_t pool_mode = cldnn_pooling_max;
    bool pool_global = false;
    cldnn_tensor pool_size{};
    // concatenation: index into cldnn_tensor::sizes (0 batch, 1 feature, 2 x, 3 y)
    int32_t concat_axis = 1;
    // eltwise / fused eltw part
    std::string eltw_calib;
    float eltw_oqf = 1.f;
    int32_t eltw_mode = cldnn_eltwise_sum;
    bool eltw_with_act = false;
    float eltw_slope = 0.f;
    int32_t conv_saturate = 0;   // fused node made from a sum without activation: the convolution's int8 saturation stays
    std::vector<cldnn_tensor> eltw_stride;
    std::vector<float> eltw_coefficients;
    // convolution / fused conv part
    cldnn_tensor input_offset{}, stride{}, dilation{}, output_size{}, padding_above{}, padding_below{};
    bool with_activation = false;
    float act_slope = 0.f;
    uint32_t split = 1, groups = 1;
    bool with_output_size = false;
    std::vector<std::string> weights, bias, wqf, calib;
    float iqf = 1.f, oqf = 1.f;
    float non_conv_scale = 1.f;
    bool second_input_in_output = false;
    bool fully_connected = false;  // convolution node that stands for a fully_connected primitive
};

}  // namespace host

struct cldnn_topology_impl : host::refcounted {
    std::map<std::string, std::shared_ptr<host::prim>> prims;
    std::vector<std::string> order;
};

namespace host {

struct node {
    std::shared_ptr<prim> p;        // possibly rewritten by the graph passes
    std::string org_id;             // id in the user's topology ("" for inserted nodes)
    std::vector<node*> deps;        // data dependencies in primitive order (input, [input2], weights, bias, wqf, calib, [eltw calib])
    std::vector<node*> users;
    bool side_stream = false;       // runs on the engine's second stream, joined before its only user
    bool rw_opt = false;            // fused_conv_eltwise made to write over its second input by the read/write pass
    cldnn_layout out{};             // output layout incl. physical padding
    int32_t user_format = cldnn_format_any;  // output format before the layout pass (what the topology implies)
    bool is_output = false;
    bool first_layer = false;       // convolution that reads b_fs_yx_fsv4 and writes fs_b_yx_fsv16
    bool constant = false;          // data primitive
    // activation folded into a convolution (reference prepare_primitive_fusing.cpp:396-433)
    int32_t fused_act = activation_none;
    float fused_a = 0.f, fused_b = 0.f;
    // compiled convolution
    cldnn_hip_conv conv = nullptr;
    cldnn_hip_conv_info conv_info{};
    // convolution chain: the head holds the chain object and its members (itself first); a follower points at its
    // head and is not launched on its own.  Members are consecutive in the execution order.
    cldnn_hip_conv_chain chain = nullptr;
    std::vector<node*> chain_members;
    std::vector<int32_t> chain_keep;
    node* chain_head = nullptr;
    // in-place concatenation (reference prepare_buffer_fusing.cpp:38-140): this node writes straight into the buffer of
    // the concatenation `concat_into`, `concat_offset` bytes from its start; the concatenation itself then does nothing
    node* concat_into = nullptr;
    size_t concat_offset = 0;
    bool concat_in_place = false;   // concatenation whose inputs all write into its buffer
    // two convolutions of one input in one launch: `sibling` (on the first in execution order) is the convolution whose
    // features follow this one's in the launch; `sibling_head` (on the second) is the node that launches for both.  The
    // two results share one buffer (the second is its contiguous tail: feature slices are the outermost axis).
    node* sibling = nullptr;
    node* sibling_head = nullptr;
    cldnn_padding unpaired_padding{};  // the output padding this node had before it took the wider border of its pair
    // member of a chain whose result stays in registers: it has no buffer and nobody but the next member reads it
    bool chain_unkept() const
    {
        const node* head = chain ? this : chain_head;
        if (!head) return false;
        for (size_t k = 0; k < head->chain_members.size(); ++k)
            if (head->chain_members[k] == this) return head->chain_keep[k] == 0;
        return false;
    }
    ref<cldnn_memory_impl> eltw_calib_dev;  // device copy of eltwise calibration (stand-alone eltwise)
};

}  // namespace host

struct cldnn_program_impl : host::refcounted {
    host::ref<cldnn_engine_impl> engine;
    std::vector<std::unique_ptr<host::node>> nodes;  // execution order
    std::map<std::string, host::node*> by_id;
    bool optimize_data = false;
    host::tuning_cache tuning;       // build option tuning_config
    size_t tuned_now = 0, tuned_from_cache = 0;
    std::vector<std::string> all_org_ids;
    ~cldnn_program_impl() override;
};

// A run whose submission waits for user events that were not set when cldnn_execute_network was called.  The last of
// those events to be set submits the run from cldnn_set_event; until then the outputs carry one deferred event.
struct deferred_run {
    std::mutex m;
    std::condition_variable cv;
    int gates_left = 0;
    bool submitted = false;
    bool cancelled = false;                // the run could not be set up: the last gate reports instead of submitting
    std::string error;                     // a failure of the late submission, reported by the next call on the network
    std::vector<cldnn_event> deps;         // retained dependency list
    host::ref<cldnn_event_impl> marker;    // the deferred event the outputs carry
    cldnn_network_impl* net = nullptr;     // retained
};

struct cldnn_network_impl : host::refcounted {
    host::ref<cldnn_program_impl> program;
    std::shared_ptr<deferred_run> pending;  // a run that has not been submitted yet
    // A postponed run is submitted by whichever thread sets its last user event, while the application's thread may ask
    // for outputs, executed ids or profiling data: events, executed and stream_events are read and written under this lock.
    std::mutex run_state;
    std::map<host::node*, host::ref<cldnn_memory_impl>> mem;
    std::map<host::node*, host::ref<cldnn_event_impl>> events;
    std::map<std::string, bool> input_set;
    std::vector<std::string> executed;
    std::vector<cldnn_hip_event> stream_events;  // fork / join events between the two streams of the last run
    bool has_run = false;
    size_t allocated_bytes = 0;  // device bytes of the buffers the network allocated for its primitives' outputs
    size_t pooled_tensors = 0;   // outputs that reuse the buffer of an earlier, finished tensor
    ~cldnn_network_impl() override;
};
