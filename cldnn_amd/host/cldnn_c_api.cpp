// The clDNN-compatible C API (include/api/C/cldnn.h) on top of the HIP layer.
// Counterpart of the reference's src/cldnn.cpp (handle functions, exception -> status translation,
// thread-local last error), src/engine.cpp, src/memory.cpp, src/network.cpp:40-353 and
// src/primitive_inst.cpp:42-143 for the primitives of the convolution path.
#include <cstring>
#include <functional>

#include "impl.h"

namespace host {
int hip_dtype(size_t dt);
int hip_format(int32_t f);
cldnn_hip_tensor to_hip(const cldnn_layout& l);
size_t layout_bytes(const cldnn_layout& l);
cldnn_tensor make_tensor(int b, int f, int x, int y);
int hip_activation_code(int32_t f);
cldnn_hip_pooling_desc pooling_descriptor(const node* n);
void build_program(cldnn_program_impl* prog, cldnn_topology_impl* topo, const std::vector<std::string>& outputs);
std::string describe_node(const node* n);
std::vector<node*> launch_waits(const node* n);
std::string describe_program(const cldnn_program_impl* prog);

static thread_local std::string g_last_error;

// reference src/include/api_impl.h:63-110: exceptions become a status plus a retrievable message
template <class T, class F>
T guard(cldnn_status* status, T fallback, F&& f)
{
    try {
        if (status) *status = CLDNN_SUCCESS;
        return f();
    } catch (const api_error& e) {
        g_last_error = e.what();
        if (status) *status = e.status;
    } catch (const std::bad_alloc&) {
        g_last_error = "out of host memory";
        if (status) *status = CLDNN_OUT_OF_RESOURCES;
    } catch (const std::exception& e) {
        g_last_error = e.what();
        if (status) *status = CLDNN_ERROR;
    }
    return fallback;
}
template <class F>
void guard_void(cldnn_status* status, F&& f)
{
    guard<int>(status, 0, [&] {
        f();
        return 0;
    });
}

static size_t copy_names(const std::vector<std::string>& names, char* out, size_t size, size_t* size_ret)
{
    // names separated and terminated by '\0', plus one closing '\0' (reference src/cldnn.cpp get_*_names)
    size_t need = 1;
    for (auto& n : names) need += n.size() + 1;
    if (size_ret) *size_ret = need;
    if (out == nullptr || size < need) throw api_error(CLDNN_INVALID_ARG, "buffer too small");
    size_t i = 0;
    for (auto& n : names) {
        std::memcpy(out + i, n.c_str(), n.size() + 1);
        i += n.size() + 1;
    }
    out[i] = 0;
    return need;
}

static std::vector<std::string> ids_of(const cldnn_primitive_id_arr& a)
{
    std::vector<std::string> v;
    for (size_t i = 0; i < a.size; ++i) v.emplace_back(a.data[i] ? a.data[i] : "");
    return v;
}

static ref<cldnn_memory_impl> allocate(cldnn_engine_impl* e, const cldnn_layout& l)
{
    ref<cldnn_memory_impl> m(new cldnn_memory_impl(), false);
    m->layout = l;
    m->engine = ref<cldnn_engine_impl>(e, true);
    hip_check(cldnn_hip_buffer_alloc(e->h, layout_bytes(l), &m->buf));
    return m;
}

static bool same_layout(const cldnn_layout& a, const cldnn_layout& b)
{
    if (a.data_type != b.data_type || a.format != b.format) return false;
    for (int i = 0; i < 4; ++i)
        if (a.size.sizes[i] != b.size.sizes[i] || a.padding.lower_size.sizes[i] != b.padding.lower_size.sizes[i]
            || a.padding.upper_size.sizes[i] != b.padding.upper_size.sizes[i])
            return false;
    return true;
}

// memory of another engine / attached host memory is copied into a buffer of this engine
// (reference src/data.cpp:33-45, src/input_layout.cpp:44-63)
static ref<cldnn_memory_impl> on_engine(cldnn_engine_impl* e, cldnn_memory_impl* m)
{
    if (m->engine.get() == e && m->buf) return ref<cldnn_memory_impl>(m, true);
    ref<cldnn_memory_impl> c = allocate(e, m->layout);
    const size_t bytes = layout_bytes(m->layout);
    if (m->attached) {
        HOST_REQUIRE(m->attached_bytes >= bytes, CLDNN_INVALID_ARG, "attached memory is smaller than its layout");
        hip_check(cldnn_hip_buffer_write(c->buf, 0, m->attached, bytes));
    } else {
        std::vector<uint8_t> tmp(bytes);
        hip_check(cldnn_hip_buffer_read(m->buf, 0, tmp.data(), bytes));
        hip_check(cldnn_hip_buffer_write(c->buf, 0, tmp.data(), bytes));
    }
    return c;
}

// A run that was postponed must have been submitted before the network is touched again.  Blocks until the user
// events it waits for are set (what the reference's set_input_data / execute do by waiting for the previous run).
static void await_pending_run(cldnn_network_impl* net)
{
    std::shared_ptr<deferred_run> run = net->pending;
    if (!run) return;
    std::string error;
    {
        std::unique_lock<std::mutex> g(run->m);
        run->cv.wait(g, [&] { return run->submitted; });
        error = run->error;
    }
    net->pending.reset();
    HOST_REQUIRE(error.empty(), CLDNN_ERROR, "the postponed run of the network failed: " + error);
}

// Enqueue one run.  deferred_marker: the run was announced earlier (its outputs already carry that event) and is
// submitted now that its user events are set.
static void submit(cldnn_network_impl* net, cldnn_event* deps, size_t ndeps, cldnn_event_impl* deferred_marker)
{
    cldnn_program_impl* prog = net->program.get();
    cldnn_engine_impl* eng = prog->engine.get();
    std::lock_guard<std::mutex> state(net->run_state);
    if (ndeps) {
        std::vector<cldnn_hip_event> hs;
        for (size_t i = 0; i < ndeps; ++i) hs.push_back(deps[i]->h);
        hip_check(cldnn_hip_engine_wait_events(eng->h, hs.data(), hs.size()));
    }
    net->executed.clear();
    if (!deferred_marker) net->events.clear();
    for (cldnn_hip_event ev : net->stream_events) cldnn_hip_event_release(ev);  // the previous run's; it has been waited for
    net->stream_events.clear();
    std::map<node*, cldnn_hip_event> joins;  // completion of the primitives on the second stream
    for (auto& u : prog->nodes) {
        node* n = u.get();
        prim& p = *n->p;
        if (n->constant) continue;
        if (p.type == prim_type::input_layout) {
            // reference src/primitive_inst.cpp:45 refuses to run with an unset input
            HOST_REQUIRE(net->input_set[p.id], CLDNN_ERROR, "network input " + p.id + " has not been set");
            continue;
        }
        auto mem_of = [&](node* d) -> cldnn_memory_impl* {
            auto it = net->mem.find(d);
            HOST_REQUIRE(it != net->mem.end() && it->second, CLDNN_ERROR, "no memory for primitive " + d->p->id);
            return it->second.get();
        };
        cldnn_memory_impl* out = n->chain_unkept() ? nullptr : mem_of(n);
        // a primitive on the second stream starts when everything issued before it on the first has finished (its
        // inputs, and whatever used its output buffer before); its user waits for it
        cldnn_hip_engine where = eng->h;
        if (n->side_stream) {
            where = eng->side;
            cldnn_hip_event fork = nullptr;
            hip_check(cldnn_hip_event_record(eng->h, &fork));
            net->stream_events.push_back(fork);
            hip_check(cldnn_hip_engine_wait_events(eng->side, &fork, 1));
        }
        // the launch at the head of a chain does the work of every member: it waits for what any of them reads
        for (node* d : launch_waits(n)) {
            auto j = joins.find(d);
            if (j != joins.end()) hip_check(cldnn_hip_engine_wait_events(eng->h, &j->second, 1));
        }
        cldnn_hip_event pev = nullptr;
        if (eng->profiling) hip_check(cldnn_hip_event_record_begin(where, &pev));
        const cldnn_hip_tensor ot = to_hip(n->out);
        switch (p.type) {
        case prim_type::reorder: {
            cldnn_memory_impl* in = mem_of(n->deps[0]);
            const cldnn_hip_tensor it = to_hip(n->deps[0]->out);
            hip_check(cldnn_hip_reorder(eng->h, in->device_ptr(), &it, out->device_ptr(), &ot));
            break;
        }
        case prim_type::concatenation: {
            if (n->concat_in_place) break;  // its inputs wrote into this buffer themselves
            // reference src/gpu/concatenation_gpu.cpp:64-90: one copy per input, at its offset along the axis
            int at[4] = {0, 0, 0, 0};  // b, f, x, y
            for (size_t i = 0; i < p.inputs.size(); ++i) {
                const cldnn_hip_tensor it = to_hip(n->deps[i]->out);
                hip_check(cldnn_hip_copy_region(eng->h, mem_of(n->deps[i])->device_ptr(), &it, out->device_ptr(), &ot, at[0], at[1], at[3], at[2]));
                at[p.concat_axis] += n->deps[i]->out.size.sizes[p.concat_axis];
            }
            break;
        }
        case prim_type::pooling: {
            cldnn_memory_impl* in = mem_of(n->deps[0]);
            cldnn_hip_pooling_desc pd = pooling_descriptor(n);
            hip_check(cldnn_hip_pooling(eng->h, &pd, in->device_ptr(), out->device_ptr()));
            break;
        }
        case prim_type::activation: {
            cldnn_memory_impl* in = mem_of(n->deps[0]);
            const cldnn_hip_tensor it = to_hip(n->deps[0]->out);
            hip_check(cldnn_hip_activation(eng->h, in->device_ptr(), &it, out->device_ptr(), &ot, hip_activation_code(p.act_func),
                                           p.act_a, p.act_b));
            break;
        }
        case prim_type::eltwise: {
            // reference src/gpu/eltwise_gpu.cpp:58-145: inputs, then the calibration factors
            const size_t count = p.inputs.size();
            cldnn_hip_eltwise_desc d{};
            const void* src[CLDNN_HIP_ELTWISE_MAX_INPUTS] = {};
            d.mode = p.eltw_mode, d.n_inputs = (int32_t)count;
            for (size_t i = 0; i < count; ++i) {
                d.inputs[i] = to_hip(n->deps[i]->out);
                src[i] = mem_of(n->deps[i])->device_ptr();
                d.stride_x[i] = p.eltw_stride.empty() ? 1 : p.eltw_stride[i].sizes[2];
                d.stride_y[i] = p.eltw_stride.empty() ? 1 : p.eltw_stride[i].sizes[3];
                d.coefficients[i] = p.eltw_coefficients.empty() ? 1.0f : p.eltw_coefficients[i];
            }
            d.has_coefficients = !p.eltw_coefficients.empty();
            d.output = ot;
            const float* calib = nullptr;
            if (!p.eltw_calib.empty()) calib = (const float*)mem_of(n->deps[count])->device_ptr();
            const bool int_data = n->deps[0]->out.data_type == cldnn_i8 || n->deps[0]->out.data_type == cldnn_u8;
            d.quantized = int_data && (calib || p.eltw_oqf != 1.0f);
            d.output_quantization_factor = p.eltw_oqf;
            d.activation = CLDNN_HIP_ACT_NONE;
            if (p.eltw_with_act) d.activation = p.eltw_slope == 0.0f ? CLDNN_HIP_ACT_RELU : CLDNN_HIP_ACT_RELU_SLOPE;
            d.m = p.eltw_slope;
            hip_check(cldnn_hip_eltwise(eng->h, &d, src, calib, out->device_ptr()));
            break;
        }
        case prim_type::convolution:
        case prim_type::fused_conv_eltwise: {
            if (n->chain_head) break;  // written by the launch of its chain's head
            if (n->sibling_head) break;  // written by the launch of the convolution it is paired with
            cldnn_memory_impl* in = mem_of(n->deps[0]);
            if (n->chain) {
                void* outs[3] = {nullptr, nullptr, nullptr};
                const void* eltws[3] = {nullptr, nullptr, nullptr};
                for (size_t k = 0; k < n->chain_members.size(); ++k) {
                    node* m = n->chain_members[k];
                    if (n->chain_keep[k]) outs[k] = mem_of(m)->device_ptr();
                    if (m->p->type == prim_type::fused_conv_eltwise) eltws[k] = mem_of(m->deps[1])->device_ptr();
                }
                hip_check(cldnn_hip_conv_chain_enqueue(n->chain, in->device_ptr(), outs, eltws));
                break;
            }
            const void* eltw = nullptr;
            if (p.type == prim_type::fused_conv_eltwise && !p.second_input_in_output) eltw = mem_of(n->deps[1])->device_ptr();
            hip_check(cldnn_hip_conv_enqueue(n->conv, in->device_ptr(), out->device_ptr(), eltw));
            break;
        }
        default: break;
        }
        if (n->side_stream) {
            cldnn_hip_event join = nullptr;
            hip_check(cldnn_hip_event_record(eng->side, &join));
            net->stream_events.push_back(join);
            joins[n] = join;
        }
        if (pev) {
            hip_check(cldnn_hip_event_record_end(pev));
            ref<cldnn_event_impl> ev(new cldnn_event_impl(), false);
            ev->engine = ref<cldnn_engine_impl>(eng, true);
            ev->h = pev;
            // an output of a postponed run keeps the event its users were given when the run was announced
            if (!(deferred_marker && n->is_output)) net->events[n] = ev;
        }
        net->executed.push_back(p.id);
    }
    if (deferred_marker) {
        hip_check(cldnn_hip_event_record_deferred(deferred_marker->h));
    } else {
        // one marker for every output that has no event of its own (reference ocl_toolkit.cpp:170-178,197-230)
        ref<cldnn_event_impl> marker;
        for (auto& u : prog->nodes) {
            node* n = u.get();
            if (!n->is_output || net->events.count(n)) continue;
            if (!marker) {
                marker = ref<cldnn_event_impl>(new cldnn_event_impl(), false);
                marker->engine = ref<cldnn_engine_impl>(eng, true);
                hip_check(cldnn_hip_event_record(eng->h, &marker->h));
            }
            net->events[n] = marker;
        }
    }
    if (eng->side) hip_check(cldnn_hip_engine_flush(eng->side));
    hip_check(cldnn_hip_engine_flush(eng->h));
    net->has_run = true;
}

static void finish_deferred_run(const std::shared_ptr<deferred_run>& run);

// called by cldnn_hip_event_set (or at once, if the event got set in the meantime) for every user event a postponed
// run waits for; the last one submits the run
static void gate_opened(void* param)
{
    std::shared_ptr<deferred_run> run = *static_cast<std::shared_ptr<deferred_run>*>(param);
    delete static_cast<std::shared_ptr<deferred_run>*>(param);
    bool last = false;
    {
        std::lock_guard<std::mutex> g(run->m);
        last = --run->gates_left == 0;
    }
    if (!last) return;
    finish_deferred_run(run);
}

// Submit a postponed run (or, when it was cancelled while being set up, only report): whoever waits for its marker or
// for the network is released either way.
static void finish_deferred_run(const std::shared_ptr<deferred_run>& run)
{
    std::string error;
    bool cancelled = false;
    {
        std::lock_guard<std::mutex> g(run->m);
        cancelled = run->cancelled;
        error = run->error;
    }
    if (cancelled) {
        (void)cldnn_hip_event_record_deferred(run->marker->h);
    } else {
        try {
            submit(run->net, run->deps.data(), run->deps.size(), run->marker.get());
        } catch (const std::exception& e) {
            error = e.what();
            (void)cldnn_hip_event_record_deferred(run->marker->h);  // nobody may wait for ever
        }
    }
    for (cldnn_event d : run->deps) d->release();
    run->deps.clear();
    cldnn_network_impl* net = run->net;
    {
        std::lock_guard<std::mutex> g(run->m);
        run->error = error;
        run->submitted = true;
    }
    run->cv.notify_all();
    net->release();
}

// reference network_impl::execute (src/network.cpp:280-353) enqueues behind the dependency events and returns; an
// OpenCL user event among them may be set later, also by the calling thread.  A HIP stream cannot wait for a host
// flag, so a run behind user events that are not set yet is postponed: this call announces it (every output gets one
// deferred event), returns, and the run is submitted by the thread that sets the last of those events.
static void execute(cldnn_network_impl* net, cldnn_event* deps, size_t ndeps)
{
    for (size_t i = 0; i < ndeps; ++i) HOST_REQUIRE(deps && deps[i], CLDNN_INVALID_ARG, "null event in the dependency list");
    await_pending_run(net);
    std::vector<cldnn_event> gates;
    for (size_t i = 0; i < ndeps; ++i)
        if (cldnn_hip_event_is_user(deps[i]->h) && !cldnn_hip_event_is_set(deps[i]->h)) gates.push_back(deps[i]);
    if (gates.empty()) {
        submit(net, deps, ndeps, nullptr);
        return;
    }
    cldnn_program_impl* prog = net->program.get();
    cldnn_engine_impl* eng = prog->engine.get();
    for (auto& u : prog->nodes)  // what submit() would refuse is refused now, while the caller can still react
        if (u->p->type == prim_type::input_layout)
            HOST_REQUIRE(net->input_set[u->p->id], CLDNN_ERROR, "network input " + u->p->id + " has not been set");
    auto run = std::make_shared<deferred_run>();
    run->gates_left = (int)gates.size();
    run->net = net;
    net->retain();
    for (size_t i = 0; i < ndeps; ++i) {
        deps[i]->retain();
        run->deps.push_back(deps[i]);
    }
    run->marker = ref<cldnn_event_impl>(new cldnn_event_impl(), false);
    run->marker->engine = ref<cldnn_engine_impl>(eng, true);
    hip_check(cldnn_hip_event_create_deferred(eng->h, &run->marker->h));
    {
        std::lock_guard<std::mutex> state(net->run_state);
        net->events.clear();
        net->executed.clear();
        for (auto& u : prog->nodes) {
            node* n = u.get();
            if (n->is_output) net->events[n] = run->marker;
            if (!n->constant && n->p->type != prim_type::input_layout) net->executed.push_back(n->p->id);
        }
        net->has_run = true;
    }
    net->pending = run;
    size_t registered = 0;
    for (cldnn_event g : gates) {
        auto* param = new std::shared_ptr<deferred_run>(run);
        const cldnn_hip_status st = cldnn_hip_event_add_handler(g->h, gate_opened, param);
        if (st == CLDNN_HIP_SUCCESS) {
            ++registered;
            continue;
        }
        // The gates registered so far still count down when their events are set; the others never will.  The run is
        // cancelled: whoever reaches zero (here, or the last registered gate) releases the waiters and reports.
        delete param;
        bool finish = false;
        {
            std::lock_guard<std::mutex> lock(run->m);
            run->cancelled = true;
            run->error = "a user event of the dependency list could not be watched";
            run->gates_left -= (int)(gates.size() - registered);
            finish = run->gates_left == 0;
        }
        if (finish) finish_deferred_run(run);
        hip_check(st);
    }
}

}  // namespace host

using namespace host;

cldnn_engine_impl::~cldnn_engine_impl()
{
    if (side) cldnn_hip_engine_release(side);
    if (h) cldnn_hip_engine_release(h);
}
cldnn_memory_impl::~cldnn_memory_impl()
{
    if (buf) cldnn_hip_buffer_release(buf);
}
cldnn_event_impl::~cldnn_event_impl()
{
    if (h) cldnn_hip_event_release(h);
}
cldnn_network_impl::~cldnn_network_impl()
{
    for (cldnn_hip_event ev : stream_events) cldnn_hip_event_release(ev);
}
cldnn_program_impl::~cldnn_program_impl()
{
    for (auto& n : nodes) {
        if (n->conv) cldnn_hip_conv_release(n->conv);
        if (n->chain) cldnn_hip_conv_chain_release(n->chain);
    }
}

struct cldnn_primitive_type {
    host::prim_type t;
    const char* name;
};
static const cldnn_primitive_type g_types[] = {
    {prim_type::input_layout, "input_layout"}, {prim_type::data, "data"},       {prim_type::reorder, "reorder"},
    {prim_type::activation, "activation"},     {prim_type::eltwise, "eltwise"}, {prim_type::convolution, "convolution"},
    {prim_type::fused_conv_eltwise, "fused_conv_eltwise"}, {prim_type::pooling, "pooling"},
    // kept as a convolution node whose filter covers the input plane
    {prim_type::convolution, "fully_connected"},
    {prim_type::concatenation, "concatenation"},
};

extern "C" {

#define TYPE_ID_FN(name, idx)                                                   \
    cldnn_primitive_type_id cldnn_##name##_type_id(cldnn_status* status)       \
    {                                                                           \
        if (status) *status = CLDNN_SUCCESS;                                    \
        return &g_types[idx];                                                   \
    }
TYPE_ID_FN(input_layout, 0)
TYPE_ID_FN(data, 1)
TYPE_ID_FN(reorder, 2)
TYPE_ID_FN(activation, 3)
TYPE_ID_FN(eltwise, 4)
TYPE_ID_FN(convolution, 5)
TYPE_ID_FN(fused_conv_eltwise, 6)
TYPE_ID_FN(pooling, 7)
TYPE_ID_FN(fully_connected, 8)
TYPE_ID_FN(concatenation, 9)

const char* cldnn_get_last_error_message() { return g_last_error.c_str(); }

cldnn_version cldnn_get_version(cldnn_status* status)
{
    if (status) *status = CLDNN_SUCCESS;
    return cldnn_version{1, 4, 25, 0};
}

// ---------------------------------------------------------------------------------------------- topology
cldnn_topology cldnn_create_topology(cldnn_status* status)
{
    return guard<cldnn_topology>(status, nullptr, [] { return new cldnn_topology_impl(); });
}

void cldnn_add_primitive(cldnn_topology topology, const struct cldnn_primitive_desc* dto, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(topology, CLDNN_INVALID_ARG, "Topology should not be null.");
        HOST_REQUIRE(dto && dto->id && dto->type, CLDNN_INVALID_ARG, "Invalid primitive descriptor.");
        auto p = std::make_shared<prim>();
        p->type = dto->type->t;
        p->id = dto->id;
        HOST_REQUIRE(!topology->prims.count(p->id), CLDNN_INVALID_ARG, "Topology already contains primitive with id: " + p->id);
        p->inputs = ids_of(dto->input);
        p->output_padding = dto->output_padding;
        p->out_dt = dto->output_data_type;
        if (dto->type == &g_types[8]) {
            // fully_connected -> convolution node with the filter of the weights' own size (checked against the input when the
            // program is built), stride 1, no padding (reference src/fully_connected.cpp:58-80, src/gpu/fully_connected_gpu.cpp)
            auto* d = reinterpret_cast<const cldnn_fully_connected_desc*>(dto);
            auto one = [](const char* s) { return s && *s ? std::vector<std::string>{s} : std::vector<std::string>{}; };
            HOST_REQUIRE(!p->out_dt.enabled, CLDNN_INVALID_ARG, "output data type forcing is not supported for fully_connected");
            p->fully_connected = true;
            p->stride = make_tensor(1, 1, 1, 1), p->dilation = make_tensor(1, 1, 1, 1), p->input_offset = make_tensor(0, 0, 0, 0);
            p->padding_above = make_tensor(0, 0, 0, 0), p->padding_below = make_tensor(0, 0, 0, 0);
            p->with_activation = d->with_activation != 0, p->act_slope = d->activation_negative_slope;
            p->split = 1, p->groups = 1;
            p->weights = one(d->weights), p->bias = one(d->bias);
            p->wqf = one(d->weights_quantization_factors), p->calib = one(d->output_calibration_factors);
            p->iqf = d->input_quantization_factor, p->oqf = d->output_quantization_factor;
            HOST_REQUIRE(p->weights.size() == 1, CLDNN_INVALID_ARG, "fully_connected needs weights");
            topology->prims[p->id] = p;
            topology->order.push_back(p->id);
            return;
        }
        switch (p->type) {
        case prim_type::input_layout: p->layout = reinterpret_cast<const cldnn_input_layout_desc*>(dto)->layout; break;
        case prim_type::data: {
            cldnn_memory m = reinterpret_cast<const cldnn_data_desc*>(dto)->mem;
            HOST_REQUIRE(m, CLDNN_INVALID_ARG, "data primitive without memory");
            p->mem = ref<cldnn_memory_impl>(m, true);
            break;
        }
        case prim_type::reorder: {
            auto* d = reinterpret_cast<const cldnn_reorder_desc*>(dto);
            HOST_REQUIRE((!d->mean_subtract || !*d->mean_subtract) && d->subtract_per_feature.size == 0, CLDNN_INVALID_ARG,
                         "reorder with mean subtraction is not supported by this library");
            p->reorder_format = d->output_format;
            break;
        }
        case prim_type::concatenation: {
            auto* d = reinterpret_cast<const cldnn_concatenation_desc*>(dto);
            HOST_REQUIRE(d->axis == cldnn_concatenation_along_b || d->axis == cldnn_concatenation_along_f || d->axis == cldnn_concatenation_along_x
                             || d->axis == cldnn_concatenation_along_y,
                         CLDNN_INVALID_ARG, "concatenation axis must be b, f, x or y (no five-dimensional tensors in this library)");
            p->concat_axis = (int32_t)d->axis;
            break;
        }
        case prim_type::pooling: {
            auto* d = reinterpret_cast<const cldnn_pooling_desc*>(dto);
            HOST_REQUIRE(!d->argmax || !*d->argmax, CLDNN_INVALID_ARG, "pooling with an argmax output is not supported by this library");
            HOST_REQUIRE(d->mode == cldnn_pooling_max || d->mode == cldnn_pooling_average || d->mode == cldnn_pooling_average_no_padding,
                         CLDNN_INVALID_ARG, "pooling mode not supported by this library (max, average, average_no_padding)");
            p->pool_mode = d->mode, p->pool_global = d->global_pooling != 0;
            p->input_offset = d->input_offset, p->stride = d->stride, p->pool_size = d->size;
            p->with_output_size = d->with_output_size != 0, p->output_size = d->output_size;
            break;
        }
        case prim_type::activation: {
            auto* d = reinterpret_cast<const cldnn_activation_desc*>(dto);
            HOST_REQUIRE(!d->additional_params_input || !*d->additional_params_input, CLDNN_INVALID_ARG,
                         "activation with a parameter input is not supported by this library");
            p->act_func = d->activation_func, p->act_a = d->additional_params.a, p->act_b = d->additional_params.b;
            break;
        }
        case prim_type::eltwise: {
            auto* d = reinterpret_cast<const cldnn_eltwise_desc*>(dto);
            p->eltw_calib = d->output_calibration_factors ? d->output_calibration_factors : "";
            p->eltw_oqf = d->output_quantization_factor;
            p->eltw_mode = d->mode;
            p->eltw_with_act = d->with_activation != 0;
            p->eltw_slope = d->activation_negative_slope;
            for (size_t i = 0; i < d->stride.size; ++i) p->eltw_stride.push_back(d->stride.data[i]);
            // reference api/CPP/eltwise.hpp:230-252
            HOST_REQUIRE(d->mode >= cldnn_eltwise_sum && d->mode <= cldnn_eltwise_mod, CLDNN_INVALID_ARG,
                         "eltwise: the comparison and logic modes are not supported by this library");
            for (size_t i = 0; i < d->coefficients.size; ++i) p->eltw_coefficients.push_back(d->coefficients.data[i]);
            HOST_REQUIRE(d->mode == cldnn_eltwise_sum || p->eltw_coefficients.empty(), CLDNN_INVALID_ARG,
                         "Only eltwise sum operation supports blob-wise coefficients");
            HOST_REQUIRE(p->eltw_coefficients.empty() || p->eltw_coefficients.size() == p->inputs.size(), CLDNN_INVALID_ARG,
                         "Invalid eltwise sum coefficients count (should be equal to 0 or input.size)");
            break;
        }
        case prim_type::convolution: {
            auto* d = reinterpret_cast<const cldnn_convolution_desc*>(dto);
            p->input_offset = d->input_offset, p->stride = d->stride, p->dilation = d->dilation;
            p->with_activation = d->with_activation != 0, p->act_slope = d->activation_negative_slope;
            p->split = d->split, p->groups = d->groups ? d->groups : 1;
            p->with_output_size = d->with_output_size != 0, p->output_size = d->output_size;
            p->weights = ids_of(d->weights), p->bias = ids_of(d->bias);
            p->wqf = ids_of(d->weights_quantization_factors), p->calib = ids_of(d->output_calibration_factors);
            p->iqf = d->input_quantization_factor, p->oqf = d->output_quantization_factor;
            p->padding_above = d->padding_above, p->padding_below = d->padding_below;
            // reference src/convolution.cpp:174-200
            HOST_REQUIRE(p->weights.size() == p->split, CLDNN_INVALID_ARG, "Weights number does not match the split");
            HOST_REQUIRE(p->bias.empty() || p->bias.size() == p->weights.size(), CLDNN_INVALID_ARG, "Bias number does not match the weights number");
            break;
        }
        case prim_type::fused_conv_eltwise: {
            auto* d = reinterpret_cast<const cldnn_fused_conv_eltwise_desc*>(dto);
            p->input_offset = d->conv.input_offset, p->stride = d->conv.stride, p->dilation = d->conv.dilation;
            p->with_activation = d->conv.with_activation != 0, p->act_slope = d->conv.activation_negative_slope;
            p->split = d->conv.split;
            p->with_output_size = d->conv.with_output_size != 0, p->output_size = d->conv.output_size;
            p->weights = ids_of(d->conv.weights), p->bias = ids_of(d->conv.bias);
            p->wqf = ids_of(d->conv.weights_quantization_factors), p->calib = ids_of(d->conv.output_calibration_factors);
            p->iqf = d->conv.input_quantization_factor, p->oqf = d->conv.output_quantization_factor;
            p->eltw_calib = d->eltw.output_calibration_factors ? d->eltw.output_calibration_factors : "";
            p->eltw_oqf = 1.0f;  // the reference leaves this field uninitialised; it is defined as 1 here
            p->eltw_mode = d->eltw.mode;
            p->eltw_with_act = d->eltw.with_activation != 0, p->eltw_slope = d->eltw.activation_negative_slope;
            for (size_t i = 0; i < d->eltw.stride.size; ++i) p->eltw_stride.push_back(d->eltw.stride.data[i]);
            p->non_conv_scale = d->non_conv_scale;
            p->second_input_in_output = d->second_input_in_output != 0;
            p->padding_above = make_tensor(0, 0, 0, 0), p->padding_below = make_tensor(0, 0, 0, 0);
            HOST_REQUIRE(p->weights.size() == 1 && p->split == 1, CLDNN_INVALID_ARG, "fused_conv_eltwise: split must be 1");
            break;
        }
        }
        topology->prims[p->id] = p;
        topology->order.push_back(p->id);
    });
}

void cldnn_change_input_layout(cldnn_topology topology, cldnn_primitive_id id, cldnn_layout new_layout, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(topology && id, CLDNN_INVALID_ARG, "Topology should not be null.");
        HOST_REQUIRE(new_layout.format >= cldnn_format_any && new_layout.format < cldnn_format_format_num, CLDNN_INVALID_ARG, "Unknown format of layout.");
        auto it = topology->prims.find(id);
        HOST_REQUIRE(it != topology->prims.end() && it->second->type == prim_type::input_layout, CLDNN_INVALID_ARG,
                     std::string("Primitive ") + id + " is not input layout.");
        it->second->layout = new_layout;
    });
}

void cldnn_get_primitive_ids(cldnn_topology topology, char* ids, size_t size, size_t* size_ret, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(topology, CLDNN_INVALID_ARG, "Topology should not be null.");
        copy_names(topology->order, ids, size, size_ret);
    });
}

#define RETAIN_RELEASE(what)                                                                  \
    void cldnn_retain_##what(cldnn_##what h, cldnn_status* status)                            \
    {                                                                                         \
        guard_void(status, [&] {                                                              \
            HOST_REQUIRE(h, CLDNN_INVALID_ARG, #what " should not be null.");                 \
            h->retain();                                                                      \
        });                                                                                   \
    }                                                                                         \
    void cldnn_release_##what(cldnn_##what h, cldnn_status* status)                           \
    {                                                                                         \
        guard_void(status, [&] {                                                              \
            HOST_REQUIRE(h, CLDNN_INVALID_ARG, #what " should not be null.");                 \
            h->release();                                                                     \
        });                                                                                   \
    }
RETAIN_RELEASE(topology)
RETAIN_RELEASE(engine)
RETAIN_RELEASE(event)
RETAIN_RELEASE(program)
RETAIN_RELEASE(network)
RETAIN_RELEASE(memory)

// ---------------------------------------------------------------------------------------------- engine
uint32_t cldnn_get_engine_count(int32_t type, cldnn_status* status)
{
    return guard<uint32_t>(status, 0, [&]() -> uint32_t {
        HOST_REQUIRE(type == cldnn_engine_ocl, CLDNN_DEVICE_ERROR, "Invalid engine type.");
        return cldnn_hip_device_count();
    });
}

void cldnn_release_pending_memory(cldnn_engine engine, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(engine, CLDNN_INVALID_ARG, "Engine should not be null.");
        hip_check(cldnn_hip_engine_finish(engine->h));
    });
}

cldnn_engine cldnn_create_engine(int32_t type, uint32_t engine_num, const cldnn_engine_configuration* cfg, cldnn_status* status)
{
    return guard<cldnn_engine>(status, nullptr, [&]() -> cldnn_engine {
        HOST_REQUIRE(type == cldnn_engine_ocl, CLDNN_DEVICE_ERROR, "Invalid engine type.");
        if (cfg) {
            HOST_REQUIRE(cfg->context == nullptr, CLDNN_INVALID_ARG, "a user-supplied device context is not supported");
            HOST_REQUIRE(cfg->priority_mode == cldnn_priority_disabled, CLDNN_INVALID_ARG,
                         "queue priorities are not supported: the engine's stream runs at the default priority");
        }
        ref<cldnn_engine_impl> e(new cldnn_engine_impl(), false);
        e->profiling = cfg && cfg->enable_profiling;
        const bool parallel = cfg && cfg->enable_parallelisation;
        if (cfg && cfg->tuning_cache_path && cfg->tuning_cache_path[0]) e->tuning_cache_path = cfg->tuning_cache_path;
        e->memory_pool = !cfg || cfg->enable_memory_pool;
        hip_check(cldnn_hip_engine_create(engine_num, e->profiling ? 1 : 0, &e->h));
        if (parallel) hip_check(cldnn_hip_engine_create(engine_num, e->profiling ? 1 : 0, &e->side));
        e->retain();
        return e.get();
    });
}

cldnn_engine_info cldnn_get_engine_info(cldnn_engine engine, cldnn_status* status)
{
    return guard<cldnn_engine_info>(status, cldnn_engine_info{}, [&] {
        HOST_REQUIRE(engine, CLDNN_INVALID_ARG, "Engine should not be null.");
        cldnn_hip_engine_info hi{};
        hip_check(cldnn_hip_engine_get_info(engine->h, &hi));
        cldnn_engine_info i{};
        i.cores_count = hi.cores_count, i.core_frequency = hi.core_frequency;
        i.max_work_group_size = hi.max_work_group_size, i.max_local_mem_size = hi.max_local_mem_size;
        i.max_global_mem_size = hi.max_global_mem_size, i.max_alloc_mem_size = hi.max_alloc_mem_size;
        i.supports_imad = 1, i.supports_immad = 1;
        return i;
    });
}

int32_t cldnn_get_engine_type(cldnn_engine engine, cldnn_status* status)
{
    return guard<int32_t>(status, 0, [&] {
        HOST_REQUIRE(engine, CLDNN_INVALID_ARG, "Engine should not be null.");
        return (int32_t)cldnn_engine_ocl;
    });
}

int64_t cldnn_get_temp_used_device_memory_size(cldnn_engine engine, cldnn_status* status)
{
    return guard<int64_t>(status, 0, [&] {
        HOST_REQUIRE(engine, CLDNN_INVALID_ARG, "Engine should not be null.");
        return cldnn_hip_engine_used_memory(engine->h);
    });
}

int64_t cldnn_get_max_used_device_memory_size(cldnn_engine engine, cldnn_status* status)
{
    return guard<int64_t>(status, 0, [&] {
        HOST_REQUIRE(engine, CLDNN_INVALID_ARG, "Engine should not be null.");
        return cldnn_hip_engine_max_used_memory(engine->h);
    });
}

// ---------------------------------------------------------------------------------------------- events
cldnn_event cldnn_create_user_event(cldnn_engine engine, cldnn_status* status)
{
    return guard<cldnn_event>(status, nullptr, [&]() -> cldnn_event {
        HOST_REQUIRE(engine, CLDNN_INVALID_ARG, "Engine should not be null.");
        ref<cldnn_event_impl> ev(new cldnn_event_impl(), false);
        ev->engine = ref<cldnn_engine_impl>(engine, true);
        hip_check(cldnn_hip_event_create_user(engine->h, 0, &ev->h));
        ev->retain();
        return ev.get();
    });
}

int32_t cldnn_is_user_event(cldnn_event event, cldnn_status* status)
{
    return guard<int32_t>(status, 0, [&] {
        HOST_REQUIRE(event, CLDNN_INVALID_ARG, "Event should not be null.");
        return cldnn_hip_event_is_user(event->h);
    });
}

void cldnn_wait_for_event(cldnn_event event, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(event, CLDNN_INVALID_ARG, "Event should not be null.");
        hip_check(cldnn_hip_event_wait(event->h));
    });
}

void cldnn_set_event(cldnn_event event, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(event, CLDNN_INVALID_ARG, "Event should not be null.");
        hip_check(cldnn_hip_event_set(event->h));
    });
}

void cldnn_add_event_handler(cldnn_event event, cldnn_event_handler handler, void* param, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(event && handler, CLDNN_INVALID_ARG, "Event and handler should not be null.");
        hip_check(cldnn_hip_event_add_handler(event->h, handler, param));
    });
}

void cldnn_get_event_profiling_info(cldnn_event event, cldnn_profiling_interval* profiling, size_t size, size_t* size_ret, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(event, CLDNN_INVALID_ARG, "Event should not be null.");
        HOST_REQUIRE(profiling || size == 0, CLDNN_INVALID_ARG, "Profiling should not be null.");
        // the three intervals of the reference (src/gpu/ocl_base_event.cpp:68-96)
        if (size_ret) *size_ret = 3;
        HOST_REQUIRE(size >= 3, CLDNN_INVALID_ARG, "buffer too small");
        uint64_t ns = 0;
        hip_check(cldnn_hip_event_elapsed_ns(event->h, &ns));
        profiling[0] = {"submission", 0};
        profiling[1] = {"starting", 0};
        profiling[2] = {"executing", ns};
    });
}

// ---------------------------------------------------------------------------------------------- program / network
static cldnn_program build(cldnn_engine engine, cldnn_topology topology, cldnn_build_option* options, size_t n)
{
    HOST_REQUIRE(topology, CLDNN_INVALID_ARG, "Topology should not be null.");
    ref<cldnn_program_impl> prog(new cldnn_program_impl(), false);
    if (engine) prog->engine = ref<cldnn_engine_impl>(engine, true);
    std::vector<std::string> outputs;
    for (size_t i = 0; i < n; ++i) {
        switch (options[i].type) {
        case cldnn_build_option_optimize_data: prog->optimize_data = true; break;
        case cldnn_build_option_outputs:
            if (options[i].data) outputs = ids_of(*reinterpret_cast<const cldnn_primitive_id_arr*>(options[i].data));
            break;
        case cldnn_build_option_tuning_config:
            if (options[i].data) {
                auto* t = reinterpret_cast<const cldnn_tuning_config*>(options[i].data);
                HOST_REQUIRE(t->mode >= cldnn_tuning_disabled && t->mode <= cldnn_tuning_tune_and_cache, CLDNN_INVALID_ARG, "unknown tuning mode");
                if (t->mode != cldnn_tuning_disabled) {
                    // reference src/program.cpp:305-309
                    HOST_REQUIRE(t->mode != cldnn_tuning_tune_and_cache || !engine || engine->profiling, CLDNN_INVALID_ARG,
                                 "Engine must be created with profiling enabled in tune_and_cache mode!");
                    std::string path = t->cache_file_path ? t->cache_file_path : "";
                    if (path.empty()) path = engine ? engine->tuning_cache_path : "cache.json";
                    prog->tuning.load(path, t->mode);  // planning without an engine still reads (and so validates) the file
                }
            }
            break;
        default: break;  // fusing, debug, graph_dumps_dir, learning_config: accepted, no effect here
        }
    }
    build_program(prog.get(), topology, outputs);
    prog->retain();
    return prog.get();
}

cldnn_program cldnn_build_program(cldnn_engine engine, cldnn_topology topology, cldnn_build_option* options, size_t options_num, cldnn_status* status)
{
    return guard<cldnn_program>(status, nullptr, [&] {
        HOST_REQUIRE(engine, CLDNN_INVALID_ARG, "Engine should not be null.");
        return build(engine, topology, options, options_num);
    });
}

void cldnn_plan_topology(cldnn_topology topology, cldnn_build_option* options, size_t options_num, char* json, size_t size, size_t* size_ret,
                         cldnn_status* status)
{
    guard_void(status, [&] {
        cldnn_program p = build(nullptr, topology, options, options_num);
        const std::string s = describe_program(p);
        p->release();
        if (size_ret) *size_ret = s.size() + 1;
        HOST_REQUIRE(json && size >= s.size() + 1, CLDNN_INVALID_ARG, "buffer too small");
        std::memcpy(json, s.c_str(), s.size() + 1);
    });
}

cldnn_network cldnn_allocate_network(cldnn_program program, cldnn_status* status)
{
    return guard<cldnn_network>(status, nullptr, [&]() -> cldnn_network {
        HOST_REQUIRE(program, CLDNN_INVALID_ARG, "Program should not be null.");
        ref<cldnn_network_impl> net(new cldnn_network_impl(), false);
        net->program = ref<cldnn_program_impl>(program, true);
        cldnn_engine_impl* e = program->engine.get();
        // Memory pool (reference src/memory_pool.cpp, engine option enable_memory_pool): an intermediate tensor takes
        // over the buffer of an earlier one of exactly the same layout once that one's last consumer has been passed in
        // execution order -- everything runs in order on one stream.  Same layout only: producers write the logical
        // elements and never the zero border or the feature padding, so those stay as the allocation left them.
        // Outputs, inputs and constants keep buffers of their own.
        std::map<node*, size_t> index, last_use;
        bool aliasing = false;
        for (size_t i = 0; i < program->nodes.size(); ++i) {
            node* n = program->nodes[i].get();
            index[n] = i;
            // asked for by the application: anything may alias, the pool stays out of it.  Set by the read/write
            // pass: the pool follows the buffer through the chain (below)
            if (n->p->type == prim_type::fused_conv_eltwise && n->p->second_input_in_output && !n->rw_opt) aliasing = true;
        }
        for (auto& u : program->nodes)
            for (node* d : u->deps) last_use[d] = std::max(last_use[d], index[u.get()]);
        // a primitive on the second stream may still read its inputs while the first stream moves on: they stay
        // reserved until the primitive that waits for it
        for (auto& u : program->nodes)
            if (u->side_stream)
                for (node* d : u->deps) last_use[d] = std::max(last_use[d], index[u->users.at(0)]);
        // a convolution chain reads and writes everything its members touch in the ONE launch at its head: whatever a
        // member reads stays reserved until the last member, so that no member's output can take that buffer over
        for (auto& u : program->nodes) {
            if (u->chain_members.empty()) continue;
            const size_t tail = index[u->chain_members.back()];
            for (node* m : u->chain_members)
                for (node* d : m->deps) last_use[d] = std::max(last_use[d], tail);
        }
        const bool pool = e->memory_pool && !aliasing;
        std::vector<std::pair<size_t, ref<cldnn_memory_impl>>> in_flight;  // (index of the last consumer, buffer)
        std::vector<ref<cldnn_memory_impl>> idle;
        for (size_t i = 0; i < program->nodes.size(); ++i) {
            node* n = program->nodes[i].get();
            if (n->constant) {
                net->mem[n] = on_engine(e, n->p->mem.get());
                continue;
            }
            if (n->p->type == prim_type::input_layout) {
                net->input_set[n->p->id] = false;
                continue;
            }
            if (n->p->type == prim_type::fused_conv_eltwise && n->p->second_input_in_output) {
                net->mem[n] = net->mem[n->deps[1]];
                // the buffer now holds this tensor: it stays reserved until this tensor's last reader
                for (auto& f : in_flight)
                    if (f.second.get() == net->mem[n].get() && last_use.count(n)) f.first = std::max(f.first, last_use[n]);
                continue;
            }
            if (n->chain_unkept()) continue;  // never written: the next member of the chain takes it in registers
            if (n->sibling_head) continue;  // a window into the pair's buffer, made when the pair's first node came up
            if (n->concat_in_place || n->concat_into) {
                // an in-place concatenation owns one buffer of its own (outside the pool); its inputs, which come earlier
                // in the order, are windows into it
                node* c = n->concat_in_place ? n : n->concat_into;
                if (!net->mem.count(c)) {
                    net->mem[c] = allocate(e, c->out);
                    net->allocated_bytes += layout_bytes(c->out);
                }
                if (n->concat_into) {
                    ref<cldnn_memory_impl> w(new cldnn_memory_impl(), false);
                    w->layout = n->out;
                    w->engine = ref<cldnn_engine_impl>(e, true);
                    w->view_of = net->mem[c];
                    w->view_offset = n->concat_offset;
                    net->mem[n] = w;
                }
                continue;
            }
            // buffers whose tensors nobody reads at or after this primitive become idle
            for (auto it = in_flight.begin(); it != in_flight.end();) {
                if (it->first < i) {
                    idle.push_back(it->second);
                    it = in_flight.erase(it);
                } else {
                    ++it;
                }
            }
            cldnn_layout want = n->out;
            if (n->sibling) want.size.sizes[1] += n->sibling->out.size.sizes[1];
            ref<cldnn_memory_impl> m;
            if (pool && !n->is_output) {
                for (auto it = idle.begin(); it != idle.end(); ++it)
                    if (same_layout((*it)->layout, want)) {
                        m = *it;
                        idle.erase(it);
                        net->pooled_tensors++;
                        break;
                    }
            }
            if (!m) {
                m = allocate(e, want);
                net->allocated_bytes += layout_bytes(want);
            }
            if (n->sibling) {
                // the pair's buffer is one tensor as far as the pool goes; the two nodes see windows
                node* b = n->sibling;
                size_t until = last_use.count(n) ? last_use[n] : i;
                if (last_use.count(b)) until = std::max(until, last_use[b]);
                if (pool) in_flight.emplace_back(until, m);
                auto window = [&](const cldnn_layout& l, size_t offset) {
                    ref<cldnn_memory_impl> w(new cldnn_memory_impl(), false);
                    w->layout = l;
                    w->engine = ref<cldnn_engine_impl>(e, true);
                    w->view_of = m;
                    w->view_offset = offset;
                    return w;
                };
                net->mem[n] = window(n->out, 0);
                net->mem[b] = window(b->out, layout_bytes(n->out));
                continue;
            }
            net->mem[n] = m;
            if (pool && !n->is_output && last_use.count(n)) in_flight.emplace_back(last_use[n], m);
        }
        net->retain();
        return net.get();
    });
}

cldnn_network cldnn_build_network(cldnn_engine engine, cldnn_topology topology, cldnn_build_option* options, size_t options_num, cldnn_status* status)
{
    return guard<cldnn_network>(status, nullptr, [&]() -> cldnn_network {
        HOST_REQUIRE(engine, CLDNN_INVALID_ARG, "Engine should not be null.");
        cldnn_program p = build(engine, topology, options, options_num);
        cldnn_status st = CLDNN_SUCCESS;
        cldnn_network n = cldnn_allocate_network(p, &st);
        p->release();
        if (st != CLDNN_SUCCESS) throw api_error(st, g_last_error);
        return n;
    });
}

void cldnn_set_network_input(cldnn_network network, cldnn_primitive_id id, cldnn_memory mem, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(network, CLDNN_INVALID_ARG, "Network should not be null.");
        HOST_REQUIRE(id && mem, CLDNN_INVALID_ARG, "Id and memory should not be null.");
        cldnn_program_impl* prog = network->program.get();
        auto it = prog->by_id.find(id);
        HOST_REQUIRE(it != prog->by_id.end() && it->second->p->type == prim_type::input_layout, CLDNN_INVALID_ARG,
                     std::string("primitive ") + id + " is not an input");
        // the previous run must be over before its input is replaced (reference network.cpp:112-113)
        await_pending_run(network);
        hip_check(cldnn_hip_engine_finish(prog->engine->h));
        HOST_REQUIRE(same_layout(mem->layout, it->second->out), CLDNN_INVALID_ARG, "set_network_input: memory layout differs from the input's layout");
        network->mem[it->second] = on_engine(prog->engine.get(), mem);
        network->input_set[id] = true;
    });
}

void cldnn_get_primitive_info(cldnn_network network, cldnn_primitive_id id, char* info, size_t size, size_t* size_ret, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(network && id, CLDNN_INVALID_ARG, "Network should not be null.");
        auto it = network->program->by_id.find(id);
        HOST_REQUIRE(it != network->program->by_id.end(), CLDNN_INVALID_ARG, std::string("unknown primitive ") + id);
        const std::string s = describe_node(it->second);
        if (size_ret) *size_ret = s.size() + 1;
        HOST_REQUIRE(info && size >= s.size() + 1, CLDNN_INVALID_ARG, "buffer too small");
        std::memcpy(info, s.c_str(), s.size() + 1);
    });
}

cldnn_engine cldnn_get_network_engine(cldnn_network network, cldnn_status* status)
{
    return guard<cldnn_engine>(status, nullptr, [&] {
        HOST_REQUIRE(network, CLDNN_INVALID_ARG, "Network should not be null.");
        network->program->engine->retain();
        return network->program->engine.get();
    });
}

cldnn_program cldnn_get_network_program(cldnn_network network, cldnn_status* status)
{
    return guard<cldnn_program>(status, nullptr, [&] {
        HOST_REQUIRE(network, CLDNN_INVALID_ARG, "Network should not be null.");
        network->program->retain();
        return network->program.get();
    });
}

static std::vector<std::string> names_if(cldnn_network net, const std::function<bool(node*)>& pred)
{
    std::vector<std::string> v;
    for (auto& u : net->program->nodes)
        if (pred(u.get())) v.push_back(u->p->id);
    return v;
}

void cldnn_get_network_output_names(cldnn_network network, char* names, size_t size, size_t* size_ret, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(network, CLDNN_INVALID_ARG, "Network should not be null.");
        copy_names(names_if(network, [](node* n) { return n->is_output; }), names, size, size_ret);
    });
}

void cldnn_get_network_executed_primitive_names(cldnn_network network, char* names, size_t size, size_t* size_ret, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(network, CLDNN_INVALID_ARG, "Network should not be null.");
        std::lock_guard<std::mutex> state(network->run_state);
        copy_names(network->executed, names, size, size_ret);
    });
}

void cldnn_get_network_all_primitive_names(cldnn_network network, char* names, size_t size, size_t* size_ret, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(network, CLDNN_INVALID_ARG, "Network should not be null.");
        copy_names(names_if(network, [](node*) { return true; }), names, size, size_ret);
    });
}

void cldnn_get_network_all_primitive_org_names(cldnn_network network, char* names, size_t size, size_t* size_ret, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(network, CLDNN_INVALID_ARG, "Network should not be null.");
        copy_names(network->program->all_org_ids, names, size, size_ret);
    });
}

void cldnn_execute_network(cldnn_network network, cldnn_event* dependencies, size_t deps_num, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(network, CLDNN_INVALID_ARG, "Network should not be null.");
        execute(network, dependencies, deps_num);
    });
}

static node* output_node(cldnn_network network, const char* name)
{
    HOST_REQUIRE(network && name && *name, CLDNN_INVALID_ARG, "ID of primitive should not be null or empty.");
    auto it = network->program->by_id.find(name);
    HOST_REQUIRE(it != network->program->by_id.end() && it->second->is_output, CLDNN_INVALID_ARG,
                 std::string("primitive ") + name + " is not an output of the network");
    HOST_REQUIRE(network->has_run, CLDNN_ERROR, "the network has not been executed");
    return it->second;
}

cldnn_network_output cldnn_get_network_output(cldnn_network network, const char* name, cldnn_status* status)
{
    return guard<cldnn_network_output>(status, cldnn_network_output{nullptr, nullptr}, [&] {
        node* n = output_node(network, name);
        std::lock_guard<std::mutex> state(network->run_state);
        cldnn_network_output o{network->events.at(n).get(), network->mem.at(n).get()};
        o.event->retain();
        o.memory->retain();
        return o;
    });
}

cldnn_memory cldnn_get_network_output_memory(cldnn_network network, const char* name, cldnn_status* status)
{
    return guard<cldnn_memory>(status, nullptr, [&] {
        node* n = output_node(network, name);
        cldnn_memory m = network->mem.at(n).get();
        m->retain();
        return m;
    });
}

cldnn_event cldnn_get_network_output_event(cldnn_network network, const char* name, cldnn_status* status)
{
    return guard<cldnn_event>(status, nullptr, [&] {
        node* n = output_node(network, name);
        std::lock_guard<std::mutex> state(network->run_state);
        cldnn_event e = network->events.at(n).get();
        e->retain();
        return e;
    });
}

// ---------------------------------------------------------------------------------------------- memory
cldnn_memory cldnn_allocate_memory(cldnn_engine engine, cldnn_layout layout, cldnn_status* status)
{
    return guard<cldnn_memory>(status, nullptr, [&]() -> cldnn_memory {
        HOST_REQUIRE(engine, CLDNN_INVALID_ARG, "Engine should not be null.");
        HOST_REQUIRE(layout.format >= cldnn_format_any && layout.format < cldnn_format_format_num, CLDNN_INVALID_ARG, "Unknown format of layout.");
        ref<cldnn_memory_impl> m = allocate(engine, layout);
        m->retain();
        return m.get();
    });
}

cldnn_memory cldnn_attach_memory(cldnn_layout layout, void* pointer, size_t size, cldnn_status* status)
{
    return guard<cldnn_memory>(status, nullptr, [&]() -> cldnn_memory {
        HOST_REQUIRE(pointer, CLDNN_INVALID_ARG, "pointer should not be null");
        HOST_REQUIRE(size >= layout_bytes(layout), CLDNN_INVALID_ARG, "buffer size does not match layout size");
        ref<cldnn_memory_impl> m(new cldnn_memory_impl(), false);
        m->layout = layout;
        m->attached = pointer;
        m->attached_bytes = size;
        m->retain();
        return m.get();
    });
}

int32_t cldnn_is_the_same_buffer(cldnn_memory mem1, cldnn_memory mem2, cldnn_status* status)
{
    return guard<int32_t>(status, 0, [&]() -> int32_t {
        HOST_REQUIRE(mem1 && mem2, CLDNN_INVALID_ARG, "Memory should not be null.");
        if (mem1 == mem2) return 1;
        if (mem1->buf && mem2->buf) return cldnn_hip_buffer_device_ptr(mem1->buf) == cldnn_hip_buffer_device_ptr(mem2->buf);
        if (mem1->attached && mem2->attached) return mem1->attached == mem2->attached;
        return 0;
    });
}

void* cldnn_lock_memory(cldnn_memory memory, cldnn_status* status)
{
    return guard<void*>(status, nullptr, [&]() -> void* {
        HOST_REQUIRE(memory, CLDNN_INVALID_ARG, "Memory should not be null.");
        if (memory->attached) return memory->attached;
        void* p = cldnn_hip_buffer_lock(memory->buf);
        if (!p) throw api_error(CLDNN_DEVICE_ERROR, cldnn_hip_last_error());
        return p;
    });
}

void cldnn_unlock_memory(cldnn_memory memory, cldnn_status* status)
{
    guard_void(status, [&] {
        HOST_REQUIRE(memory, CLDNN_INVALID_ARG, "Memory should not be null.");
        if (!memory->attached) hip_check(cldnn_hip_buffer_unlock(memory->buf));
    });
}

cldnn_layout cldnn_get_memory_layout(cldnn_memory memory, cldnn_status* status)
{
    return guard<cldnn_layout>(status, cldnn_layout{}, [&] {
        HOST_REQUIRE(memory, CLDNN_INVALID_ARG, "Memory should not be null.");
        return memory->layout;
    });
}

cldnn_engine cldnn_get_memory_engine(cldnn_memory memory, cldnn_status* status)
{
    return guard<cldnn_engine>(status, nullptr, [&]() -> cldnn_engine {
        HOST_REQUIRE(memory, CLDNN_INVALID_ARG, "Memory should not be null.");
        if (!memory->engine) return nullptr;
        memory->engine->retain();
        return memory->engine.get();
    });
}

}  // extern "C"
