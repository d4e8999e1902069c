// Program build: topology -> ordered graph, the three graph passes the convolution path uses
// (activation fusing, conv+eltwise fusing, layout selection with reorder insertion and border
// preparation), output-layout calculation and compilation of the convolution objects.
//
// Reference counterparts: src/program.cpp:312-451 (pipeline), src/convolution.cpp:32-130 and
// src/fused_conv_eltwise.cpp:32-122 (output layout + validation), src/include/sliding_window_utils.h:90-129,
// src/graph_optimizer/prepare_primitive_fusing.cpp:181-337,396-433, src/layout_optimizer.cpp:187-291,
// src/graph_optimizer/{reorder_inputs,prepare_padding,handle_input_padding,compile_graph}.cpp,
// src/gpu/convolution_gpu.cpp:71-162, src/gpu/fused_conv_eltwise_gpu.cpp:70-200.
#include <algorithm>
#include <cstring>
#include <functional>
#include <set>

#include "impl.h"

namespace host {

void hip_check(cldnn_hip_status s)
{
    if (s != CLDNN_HIP_SUCCESS) throw api_error((cldnn_status)s, cldnn_hip_last_error());
}

// ------------------------------------------------------------------------------------------ layouts
int hip_dtype(size_t dt)
{
    switch (dt) {
    case cldnn_i8: return CLDNN_HIP_S8;
    case cldnn_u8: return CLDNN_HIP_U8;
    case cldnn_i32: return CLDNN_HIP_I32;
    case cldnn_f32: return CLDNN_HIP_F32;
    default: throw api_error(CLDNN_UNSUPPORTED_FORMAT, "data type not supported by this library (i8, u8, i32, f32 only)");
    }
}

int hip_format(int32_t f)
{
    switch (f) {
    case cldnn_format_bfyx: return CLDNN_HIP_FMT_BFYX;
    case cldnn_format_yxfb: return CLDNN_HIP_FMT_YXFB;
    case cldnn_format_byxf: return CLDNN_HIP_FMT_BYXF;
    case cldnn_format_fs_b_yx_fsv16: return CLDNN_HIP_FMT_FS_B_YX_FSV16;
    case cldnn_format_b_fs_yx_fsv4: return CLDNN_HIP_FMT_B_FS_YX_FSV4;
    default: throw api_error(CLDNN_UNSUPPORTED_FORMAT, "memory format not supported by this library");
    }
}

cldnn_hip_tensor to_hip(const cldnn_layout& l)
{
    cldnn_hip_tensor t{};
    t.dtype = hip_dtype(l.data_type);
    t.format = hip_format(l.format);
    t.b = l.size.sizes[0], t.f = l.size.sizes[1], t.x = l.size.sizes[2], t.y = l.size.sizes[3];
    const int32_t* lo = l.padding.lower_size.sizes;
    const int32_t* hi = l.padding.upper_size.sizes;
    t.pad_lo_b = lo[0], t.pad_lo_f = lo[1], t.pad_lo_x = lo[2], t.pad_lo_y = lo[3];
    t.pad_hi_b = hi[0], t.pad_hi_f = hi[1], t.pad_hi_x = hi[2], t.pad_hi_y = hi[3];
    return t;
}

size_t layout_bytes(const cldnn_layout& l)
{
    cldnn_hip_tensor t = to_hip(l);
    size_t b = cldnn_hip_tensor_bytes(&t);
    HOST_REQUIRE(b > 0, CLDNN_INVALID_ARG, std::string("bad layout: ") + cldnn_hip_last_error());
    return b;
}

cldnn_tensor make_tensor(int b, int f, int x, int y)
{
    cldnn_tensor t{};
    t.batch_num = 1, t.feature_num = 1, t.spatial_num = 3, t.local_num = 2;
    for (int i = 0; i < CLDNN_TENSOR_DIM_MAX; ++i) t.sizes[i] = 1;
    t.sizes[0] = b, t.sizes[1] = f, t.sizes[2] = x, t.sizes[3] = y;
    return t;
}

static cldnn_padding no_padding()
{
    cldnn_padding p{};
    p.lower_size = make_tensor(0, 0, 0, 0);
    p.upper_size = make_tensor(0, 0, 0, 0);
    for (int i = 4; i < CLDNN_TENSOR_DIM_MAX; ++i) p.lower_size.sizes[i] = p.upper_size.sizes[i] = 0;
    return p;
}

static bool is_int8(size_t dt) { return dt == cldnn_i8 || dt == cldnn_u8; }

// ------------------------------------------------------------------------------------------ constants
// host copy of a data primitive's memory, element count checked
static std::vector<uint8_t> read_constant(node* n, size_t expect_elems, const char* what)
{
    HOST_REQUIRE(n && n->constant && n->p->mem, CLDNN_INVALID_ARG, std::string(what) + " must be a data primitive");
    cldnn_memory_impl* m = n->p->mem.get();
    const cldnn_layout& l = m->layout;
    size_t elems = (size_t)l.size.sizes[0] * l.size.sizes[1] * l.size.sizes[2] * l.size.sizes[3];
    HOST_REQUIRE(elems == expect_elems, CLDNN_DIMENSION_MISMATCH,
                 std::string(what) + ": " + std::to_string(elems) + " elements, expected " + std::to_string(expect_elems));
    cldnn_hip_tensor t = to_hip(l);
    HOST_REQUIRE(t.pad_lo_x == 0 && t.pad_lo_y == 0 && t.pad_hi_x == 0 && t.pad_hi_y == 0 && t.pad_lo_f == 0 && t.pad_hi_f == 0,
                 CLDNN_UNSUPPORTED_FORMAT, std::string(what) + ": padded constants are not supported");
    size_t bytes = layout_bytes(l);
    std::vector<uint8_t> out(bytes);
    if (m->attached) {
        std::memcpy(out.data(), m->attached, bytes);
    } else {
        hip_check(cldnn_hip_buffer_read(m->buf, 0, out.data(), bytes));
    }
    return out;
}

// ------------------------------------------------------------------------------------------ output layouts
static int spatial(const cldnn_tensor& t, int i) { return t.sizes[2 + i]; }

struct conv_geom {
    int B, IFM, IH, IW, OFM, FY, FX, sy, sx, dy, dx, py, px, OH, OW, groups;
    int ey, ex;  // zero padding on the high side minus the padding on the low side (asymmetric padding_above / below)
    int vy, vx;  // positive input offset: the input is the view that leaves this many elements out on both sides (IH / IW are the view's)
};

// output extent with `lo` zeros in front of and `hi` behind the input (reference sliding_window_utils.h:113-126)
static int window_extent(int in, int lo, int hi, int filt, int dil, int stride)
{
    const int wnd = (filt - 1) * dil + 1, span = in + lo + hi;
    return wnd > span ? 1 : (span - wnd) / stride + 1;
}

static conv_geom conv_geometry(const prim& p, const cldnn_layout& in, const cldnn_layout& w)
{
    conv_geom g{};
    g.B = in.size.sizes[0], g.IFM = in.size.sizes[1], g.IW = in.size.sizes[2], g.IH = in.size.sizes[3];
    g.groups = p.groups ? (int)p.groups : 1;
    // split: one weights / bias / ... primitive per part, each [OFM/split][IFM/split][y][x]; part i reads input features
    // [i*IFM/split, ...) and writes output features [i*OFM/split, ...) (reference fused_conv_eltwise_gpu_ref.cl:111,
    // 134-136,194) -- the same arithmetic as `groups = split` on the concatenated constants
    const int split = p.split ? (int)p.split : 1;
    HOST_REQUIRE(split == 1 || g.groups == 1, CLDNN_INVALID_ARG, "convolution: split and groups exclude each other");
    if (split > 1) g.groups = split;
    HOST_REQUIRE(w.format == cldnn_format_bfyx, CLDNN_UNSUPPORTED_FORMAT, "convolution weights must be given in bfyx (o, i, y, x)");
    g.OFM = w.size.sizes[0] * split;
    g.FX = w.size.sizes[2], g.FY = w.size.sizes[3];
    HOST_REQUIRE(w.size.sizes[1] * g.groups == g.IFM, CLDNN_DIMENSION_MISMATCH,
                 "weights input feature count (x groups) differs from the input's feature count");
    HOST_REQUIRE(g.OFM % g.groups == 0, CLDNN_DIMENSION_MISMATCH, "output features do not divide into groups");
    if (p.fully_connected)
        HOST_REQUIRE(g.FX == g.IW && g.FY == g.IH, CLDNN_DIMENSION_MISMATCH,
                     "fully_connected: the weights' spatial size differs from the input's");
    g.sx = spatial(p.stride, 0), g.sy = spatial(p.stride, 1);
    g.dx = spatial(p.dilation, 0), g.dy = spatial(p.dilation, 1);
    // reference src/convolution.cpp:54-61
    HOST_REQUIRE(g.sx > 0 && g.sy > 0, CLDNN_INVALID_ARG, "stride spatial X/Y must be positive");
    HOST_REQUIRE(g.dx > 0 && g.dy > 0, CLDNN_INVALID_ARG, "dilation spatial X/Y must be positive");
    HOST_REQUIRE(p.input_offset.sizes[0] == 0 && p.input_offset.sizes[1] == 0, CLDNN_INVALID_ARG,
                 "input offset in batch / feature is not supported");
    int ox = spatial(p.input_offset, 0), oy = spatial(p.input_offset, 1);
    // a positive offset moves the origin of the input into the data: the convolution runs on the view that leaves
    // `offset` elements out on both sides (reference src/gpu/convolution_gpu.cpp:94-98 with the size rule of
    // sliding_window_utils.h:113-126, input - 2 * offset)
    g.vx = std::max(ox, 0), g.vy = std::max(oy, 0);
    HOST_REQUIRE(2 * g.vx < g.IW && 2 * g.vy < g.IH, CLDNN_INVALID_ARG, "input offset is greater than the input data range");
    g.IW -= 2 * g.vx, g.IH -= 2 * g.vy;
    ox = std::min(ox, 0), oy = std::min(oy, 0);
    // padding_above / padding_below: zeros in front of / behind the input.  The reference folds the symmetric case
    // into the offset and puts a zero border primitive in front of the convolution otherwise
    // (handle_input_padding.cpp:27-92); here both are padding of the convolution itself.
    int pax = spatial(p.padding_above, 0), pay = spatial(p.padding_above, 1);
    int pbx = spatial(p.padding_below, 0), pby = spatial(p.padding_below, 1);
    HOST_REQUIRE(p.padding_above.sizes[0] == 0 && p.padding_above.sizes[1] == 0 && p.padding_below.sizes[0] == 0
                     && p.padding_below.sizes[1] == 0, CLDNN_INVALID_ARG, "padding above / below in batch or feature is not supported");
    HOST_REQUIRE(pax >= 0 && pay >= 0 && pbx >= 0 && pby >= 0, CLDNN_INVALID_ARG, "padding above / below cannot be negative");
    HOST_REQUIRE((g.vx == 0 || (pax == 0 && pbx == 0)) && (g.vy == 0 || (pay == 0 && pby == 0)), CLDNN_INVALID_ARG,
                 "a positive input offset together with padding above / below on the same axis is not supported");
    g.px = -ox + pax, g.py = -oy + pay;
    g.ex = pbx - pax, g.ey = pby - pay;
    const int ow = window_extent(g.IW, g.px, g.px + g.ex, g.FX, g.dx, g.sx);
    const int oh = window_extent(g.IH, g.py, g.py + g.ey, g.FY, g.dy, g.sy);
    if (p.with_output_size) {
        g.OW = spatial(p.output_size, 0), g.OH = spatial(p.output_size, 1);
        HOST_REQUIRE(g.OW > 0 && g.OH > 0, CLDNN_INVALID_ARG, "user-defined output size must be positive");
        HOST_REQUIRE(g.OW == ow && g.OH == oh, CLDNN_INVALID_ARG, "user-defined output size differs from the computed one");
    } else {
        g.OW = ow, g.OH = oh;
    }
    return g;
}

struct pool_geom {
    int ky, kx, sy, sx, py, px, OH, OW, divider;
};

static pool_geom pooling_geometry(const prim& p, const cldnn_layout& in)
{
    pool_geom g{};
    const int IW = in.size.sizes[2], IH = in.size.sizes[3];
    g.kx = p.pool_global ? IW : spatial(p.pool_size, 0), g.ky = p.pool_global ? IH : spatial(p.pool_size, 1);
    g.sx = spatial(p.stride, 0), g.sy = spatial(p.stride, 1);
    const int ox = spatial(p.input_offset, 0), oy = spatial(p.input_offset, 1);
    HOST_REQUIRE(g.sx > 0 && g.sy > 0, CLDNN_INVALID_ARG, "pooling: stride spatial X/Y must be positive");
    HOST_REQUIRE(g.kx > 0 && g.ky > 0, CLDNN_INVALID_ARG, "pooling: window size spatial X/Y must be positive");
    HOST_REQUIRE(2 * ox <= IW && 2 * oy <= IH, CLDNN_INVALID_ARG, "pooling: input offset is greater than the input data range");
    HOST_REQUIRE(-ox <= g.kx && -oy <= g.ky, CLDNN_INVALID_ARG, "pooling: first window is outside of the image, reduce the input offset");
    HOST_REQUIRE(p.input_offset.sizes[0] == 0 && p.input_offset.sizes[1] == 0, CLDNN_INVALID_ARG,
                 "pooling: input offset in batch / feature is not supported");
    HOST_REQUIRE(ox <= 0 && oy <= 0, CLDNN_INVALID_ARG, "pooling: positive input offsets are not supported");
    g.px = -ox, g.py = -oy;
    if (p.with_output_size) {
        g.OW = spatial(p.output_size, 0), g.OH = spatial(p.output_size, 1);
        HOST_REQUIRE(g.OW > 0 && g.OH > 0, CLDNN_INVALID_ARG, "pooling: user-defined output size must be positive");
    } else {
        g.OW = cldnn_hip_pooling_out_extent(IW, g.px, g.kx, g.sx);
        g.OH = cldnn_hip_pooling_out_extent(IH, g.py, g.ky, g.sy);
    }
    // divisor of an average (reference src/gpu/pooling_gpu.cpp:36-52,100-108)
    const bool overhang = (g.OW - 1) * g.sx + g.kx > 2 * g.px + IW || (g.OH - 1) * g.sy + g.ky > 2 * g.py + IH;
    g.divider = p.pool_mode == cldnn_pooling_average_no_padding ? CLDNN_HIP_POOL_DIV_VALID
                : (p.pool_mode == cldnn_pooling_average && overhang ? CLDNN_HIP_POOL_DIV_PADDED : CLDNN_HIP_POOL_DIV_FIXED);
    return g;
}

static node* dep_named(node* n, const std::string& id)
{
    for (node* d : n->deps)
        if (d->p->id == id) return d;
    throw api_error(CLDNN_ERROR, "internal: dependency " + id + " of " + n->p->id + " not found");
}

static void calc_layout(node* n)
{
    prim& p = *n->p;
    cldnn_padding pad = p.output_padding;
    switch (p.type) {
    case prim_type::input_layout: n->out = p.layout; return;
    case prim_type::data: n->out = p.mem->layout; return;
    case prim_type::reorder: {
        n->out = n->deps[0]->out;
        n->out.format = p.reorder_format;
        if (p.out_dt.enabled) n->out.data_type = p.out_dt.data_type;
        break;
    }
    case prim_type::activation: {
        n->out = n->deps[0]->out;
        if (p.out_dt.enabled) n->out.data_type = p.out_dt.data_type;
        break;
    }
    case prim_type::pooling: {
        // reference src/pooling.cpp:30-117
        const cldnn_layout& in = n->deps[0]->out;
        HOST_REQUIRE(!p.out_dt.enabled, CLDNN_INVALID_ARG, "output data type forcing is not supported for pooling");
        const pool_geom g = pooling_geometry(p, in);
        n->out = in;
        n->out.size = make_tensor(in.size.sizes[0], in.size.sizes[1], g.OW, g.OH);
        break;
    }
    case prim_type::concatenation: {
        // reference src/concatenation.cpp:31-54 (layout) and :85-120 (every other axis must agree, one format)
        HOST_REQUIRE(!p.out_dt.enabled, CLDNN_INVALID_ARG, "output data type forcing is not supported for concatenation");
        HOST_REQUIRE(p.concat_axis >= 0 && p.concat_axis <= 3, CLDNN_INVALID_ARG, "concatenation axis must be b, f, x or y");
        const cldnn_layout& first = n->deps[0]->out;
        n->out = first;
        n->out.size.sizes[p.concat_axis] = 0;
        for (size_t k = 0; k < p.inputs.size(); ++k) {
            const cldnn_layout& in = n->deps[k]->out;
            for (int i = 0; i < 4; ++i)
                HOST_REQUIRE(i == p.concat_axis || in.size.sizes[i] == first.size.sizes[i], CLDNN_DIMENSION_MISMATCH,
                             "concatenation: every input must have the same size along the other axes");
            HOST_REQUIRE(in.data_type == first.data_type, CLDNN_INVALID_ARG, "concatenation: the inputs differ in data type");
            n->out.size.sizes[p.concat_axis] += in.size.sizes[p.concat_axis];
        }
        break;
    }
    case prim_type::eltwise: {
        const size_t count = p.inputs.size();
        HOST_REQUIRE(count >= 2 && n->deps.size() >= count, CLDNN_INVALID_ARG, "eltwise needs two inputs");
        HOST_REQUIRE(count <= CLDNN_HIP_ELTWISE_MAX_INPUTS, CLDNN_INVALID_ARG, "eltwise: at most 4 inputs are supported by this library");
        const cldnn_layout& a = n->deps[0]->out;
        // reference src/eltwise.cpp:38-46
        if (is_int8(a.data_type))
            HOST_REQUIRE(p.eltw_mode != cldnn_eltwise_pow, CLDNN_INVALID_ARG, "Requested eltwise mode is not supported for integer types.");
        n->out = a;
        if (!p.eltw_stride.empty()) {
            // strided inputs: the first input's size divided by its stride (reference src/eltwise.cpp:59-66)
            HOST_REQUIRE(p.eltw_stride.size() == count, CLDNN_INVALID_ARG, "eltwise needs one stride per input");
            for (int i = 2; i < 4; ++i) {
                for (size_t k = 0; k < count; ++k)
                    HOST_REQUIRE(p.eltw_stride[k].sizes[i] > 0, CLDNN_INVALID_ARG, "eltwise stride must be positive");
                n->out.size.sizes[i] = a.size.sizes[i] / p.eltw_stride[0].sizes[i];
                for (size_t k = 1; k < count; ++k)
                    HOST_REQUIRE(n->out.size.sizes[i] == n->deps[k]->out.size.sizes[i] / p.eltw_stride[k].sizes[i],
                                 CLDNN_DIMENSION_MISMATCH, "eltwise inputs differ in size after striding");
            }
        } else {
            // broadcast: every axis takes the largest size among the inputs (reference src/eltwise.cpp:68-72)
            for (int i = 0; i < 4; ++i)
                for (size_t k = 1; k < count; ++k) n->out.size.sizes[i] = std::max(n->out.size.sizes[i], n->deps[k]->out.size.sizes[i]);
            for (int i = 0; i < 4; ++i)
                for (size_t k = 0; k < count; ++k) {
                    const int s = n->deps[k]->out.size.sizes[i];
                    HOST_REQUIRE(s == n->out.size.sizes[i] || s == 1, CLDNN_DIMENSION_MISMATCH,
                                 "eltwise inputs differ in size and cannot be broadcast");
                }
        }
        if (p.out_dt.enabled) n->out.data_type = p.out_dt.data_type;
        break;
    }
    case prim_type::convolution:
    case prim_type::fused_conv_eltwise: {
        const cldnn_layout& in = n->deps[0]->out;
        node* w = dep_named(n, p.weights.at(0));
        conv_geom g = conv_geometry(p, in, w->out);
        n->out = in;  // format follows the input (reference src/convolution.cpp:129)
        if (n->first_layer) n->out.format = cldnn_format_fs_b_yx_fsv16;  // b_fs_yx_fsv4 in, blocked out
        n->out.size = make_tensor(g.B, g.OFM, g.OW, g.OH);
        if (p.out_dt.enabled) n->out.data_type = p.out_dt.data_type;
        if (p.fully_connected && in.format != cldnn_format_fs_b_yx_fsv16) {
            // reference src/fully_connected.cpp:58-80: batch-innermost output for yxfb inputs and for bfyx inputs with batch > 1
            const bool batch_last = in.format == cldnn_format_yxfb || (in.format == cldnn_format_bfyx && g.B > 1);
            n->out.format = batch_last ? cldnn_format_yxfb : cldnn_format_bfyx;
        }
        break;
    }
    }
    n->out.padding = pad;  // explicit output padding of the primitive; the border pass may widen it
}

// ------------------------------------------------------------------------------------------ graph helpers
static node* add_node(cldnn_program_impl* prog, std::shared_ptr<prim> p, const std::string& org)
{
    auto n = std::unique_ptr<node>(new node());
    n->p = std::move(p);
    n->org_id = org;
    n->constant = n->p->type == prim_type::data;
    node* raw = n.get();
    HOST_REQUIRE(!prog->by_id.count(raw->p->id), CLDNN_INVALID_ARG, "duplicate primitive id: " + raw->p->id);
    prog->by_id[raw->p->id] = raw;
    prog->nodes.push_back(std::move(n));
    return raw;
}

static void replace_dep(node* user, node* from, node* to)
{
    for (auto& d : user->deps)
        if (d == from) d = to;
    for (auto& s : user->p->inputs)
        if (s == from->p->id) s = to->p->id;
    from->users.erase(std::remove(from->users.begin(), from->users.end(), user), from->users.end());
    to->users.push_back(user);
}

static void remove_node(cldnn_program_impl* prog, node* n)
{
    for (node* d : n->deps) d->users.erase(std::remove(d->users.begin(), d->users.end(), n), d->users.end());
    prog->by_id.erase(n->p->id);
    prog->nodes.erase(std::remove_if(prog->nodes.begin(), prog->nodes.end(), [n](const std::unique_ptr<node>& u) { return u.get() == n; }),
                      prog->nodes.end());
}

static void sort_nodes(cldnn_program_impl* prog)
{
    std::vector<std::unique_ptr<node>> sorted;
    std::set<node*> done;
    std::map<node*, std::unique_ptr<node>> owned;
    std::vector<node*> order;
    for (auto& u : prog->nodes) order.push_back(u.get());
    for (auto& u : prog->nodes) owned[u.get()] = std::move(u);
    std::function<void(node*, int)> visit = [&](node* n, int depth) {
        if (done.count(n)) return;
        HOST_REQUIRE(depth < 100000, CLDNN_INVALID_ARG, "topology contains a cycle");
        done.insert(n);
        for (node* d : n->deps) visit(d, depth + 1);
        sorted.push_back(std::move(owned[n]));
    };
    for (node* n : order) visit(n, 0);
    prog->nodes = std::move(sorted);
}

static size_t position(cldnn_program_impl* prog, node* n)
{
    for (size_t i = 0; i < prog->nodes.size(); ++i)
        if (prog->nodes[i].get() == n) return i;
    return (size_t)-1;
}

static std::shared_ptr<prim> make_reorder(const std::string& id, const std::string& input, int32_t format)
{
    auto r = std::make_shared<prim>();
    r->type = prim_type::reorder;
    r->id = id;
    r->inputs = {input};
    r->output_padding = no_padding();
    r->reorder_format = format;
    return r;
}

// ------------------------------------------------------------------------------------------ passes
// activation -> fused into the producing convolution (reference prepare_primitive_fusing.cpp:396-433)
static void fuse_activations(cldnn_program_impl* prog)
{
    std::vector<node*> acts;
    for (auto& u : prog->nodes)
        if (u->p->type == prim_type::activation) acts.push_back(u.get());
    for (node* a : acts) {
        node* in = a->deps[0];
        if (a->is_output || in->is_output || a->deps.size() != 1) continue;
        if (in->users.size() != 1 || in->fused_act != activation_none) continue;
        if (in->p->type != prim_type::convolution) continue;
        const int f = a->p->act_func;
        if (!(f == activation_relu || f == activation_relu_negative_slope || f == activation_clamp || f == activation_none)) continue;
        in->fused_act = f, in->fused_a = a->p->act_a, in->fused_b = a->p->act_b;
        in->p->output_padding = a->p->output_padding;
        for (node* u : std::vector<node*>(a->users)) replace_dep(u, a, in);
        remove_node(prog, a);
    }
}

static bool filter_is_1x1(node* conv)
{
    node* w = dep_named(conv, conv->p->weights.at(0));
    return w->out.size.sizes[2] == 1 && w->out.size.sizes[3] == 1;
}

// An eltwise whose every user is a 1x1 convolution with one and the same stride > 1 computes only the elements those
// convolutions read: the stride moves into the eltwise and the convolutions become stride 1
// (reference src/graph_optimizer/eltwise_shrinking.cpp:25-132).
static void eltwise_shrinking(cldnn_program_impl* prog)
{
    for (auto& u : prog->nodes) {
        node* e = u.get();
        if (e->p->type != prim_type::eltwise || !e->p->eltw_stride.empty() || e->users.empty() || e->is_output) continue;
        if (!is_int8(e->out.data_type) && e->out.data_type != cldnn_f32) continue;
        int sx = 0, sy = 0;
        bool can_shrink = true;
        for (node* c : e->users) {
            if (c->p->type != prim_type::convolution || c->p->fully_connected || c->p->weights.size() != 1 || c->deps[0] != e
                || std::count(c->deps.begin(), c->deps.end(), e) != 1 || !filter_is_1x1(c)) {
                can_shrink = false;
                break;
            }
            const int cx = spatial(c->p->stride, 0), cy = spatial(c->p->stride, 1);
            if (cx <= 1 && cy <= 1) {
                can_shrink = false;
                break;
            }
            if (sx == 0) sx = cx, sy = cy;
            // a 1x1 window at offset 0: the convolution reads exactly the elements (y * sy, x * sx)
            if (cx != sx || cy != sy || spatial(c->p->input_offset, 0) != 0 || spatial(c->p->input_offset, 1) != 0
                || spatial(c->p->padding_above, 0) != 0 || spatial(c->p->padding_above, 1) != 0
                || spatial(c->p->padding_below, 0) != 0 || spatial(c->p->padding_below, 1) != 0) {
                can_shrink = false;
                break;
            }
        }
        if (!can_shrink) continue;
        // every convolution keeps the output size it had: the shrunk eltwise must have exactly that size
        for (node* c : e->users)
            if (c->out.size.sizes[2] != e->out.size.sizes[2] / sx || c->out.size.sizes[3] != e->out.size.sizes[3] / sy) can_shrink = false;
        if (!can_shrink) continue;
        e->p = std::make_shared<prim>(*e->p);
        cldnn_tensor st = make_tensor(1, 1, sx, sy);
        e->p->eltw_stride.assign(e->p->inputs.size(), st);
        calc_layout(e);
        for (node* c : e->users) {
            c->p = std::make_shared<prim>(*c->p);
            c->p->stride.sizes[2] = 1, c->p->stride.sizes[3] = 1;
            c->p->with_output_size = false;
            calc_layout(c);
        }
    }
}

// The stride of a strided eltwise input moves up into the convolutions that produce it, so that they no longer compute
// elements nobody reads: through 1x1 convolutions (which pass it on to their own producer) into the first convolution
// whose filter is wide enough to take it as its own stride (reference src/graph_optimizer/eltwise_remove_stride.cpp:27-105).
static bool conv_stride_extend(node* c, cldnn_tensor& st)
{
    if (c->users.size() > 1 || c->is_output || c->p->type != prim_type::convolution || c->p->fully_connected || c->p->weights.size() != 1)
        return false;
    if (filter_is_1x1(c)) {
        // only a pointwise convolution of stride 1 without padding commutes with the sub-sampling
        if (spatial(c->p->stride, 0) != 1 || spatial(c->p->stride, 1) != 1 || spatial(c->p->input_offset, 0) != 0
            || spatial(c->p->input_offset, 1) != 0)
            return false;
        node* d = c->deps[0];
        if (!conv_stride_extend(d, st)) return false;
        c->p = std::make_shared<prim>(*c->p);
        c->p->with_output_size = false;
        calc_layout(c);
        return true;
    }
    node* w = dep_named(c, c->p->weights.at(0));
    const int fx = w->out.size.sizes[2], fy = w->out.size.sizes[3];
    const int cx = spatial(c->p->stride, 0), cy = spatial(c->p->stride, 1), ex = st.sizes[2], ey = st.sizes[3];
    // reference :54-55; the sub-sampled outputs (y * ey, x * ex) of a stride-(cy, cx) convolution are the outputs of a
    // convolution of stride (cy * ey, cx * ex) -- the reference adds, which is the same for the stride-1 convolutions
    // it meets, and a product is what the geometry asks for otherwise
    if (fx - (cx + (ex - 1)) < 0 || fy - (cy + (ey - 1)) < 0) return false;
    const cldnn_layout before = c->out;
    auto p = std::make_shared<prim>(*c->p);
    p->stride.sizes[2] = cx * ex, p->stride.sizes[3] = cy * ey;
    p->with_output_size = false;
    std::shared_ptr<prim> old = c->p;
    c->p = p;
    calc_layout(c);
    if (c->out.size.sizes[2] != before.size.sizes[2] / ex || c->out.size.sizes[3] != before.size.sizes[3] / ey) {
        c->p = old;  // the strided convolution would not produce exactly the sub-sampled tensor
        calc_layout(c);
        return false;
    }
    st.sizes[2] = 1, st.sizes[3] = 1;
    return true;
}

static void eltwise_remove_stride(cldnn_program_impl* prog)
{
    for (auto& u : prog->nodes) {
        node* e = u.get();
        if (e->p->type != prim_type::eltwise || e->p->eltw_stride.empty()) continue;
        for (size_t i = 0; i < e->p->inputs.size(); ++i) {
            cldnn_tensor& st = e->p->eltw_stride[i];
            if (st.sizes[2] == 1 && st.sizes[3] == 1) continue;
            if (std::count(e->deps.begin(), e->deps.end(), e->deps[i]) != 1) continue;
            conv_stride_extend(e->deps[i], st);
        }
        calc_layout(e);
    }
}

static bool wants_blocked(node* n);

// convolution (1x1, stride 1) + eltwise sum with relu -> fused_conv_eltwise (reference :181-337).
// A sum WITHOUT activation stays a primitive of its own in the reference (a residual sum of MobileNet-v2).  Its
// arithmetic differs from the fused primitive's in one point: it adds to the convolution's int8 output, that is to the
// saturated value.  With that saturation kept inside the fused kernel (conv_saturate) the results are the same, so a
// quantized s8 sum of that kind is fused here as well: one launch and one tensor round trip less per block.
static void fuse_conv_eltwise(cldnn_program_impl* prog)
{
    std::vector<node*> convs;
    for (auto& u : prog->nodes)
        if (u->p->type == prim_type::convolution && !u->p->fully_connected) convs.push_back(u.get());
    for (node* c : convs) {
        if (c->users.size() != 1 || c->is_output) continue;
        node* e = c->users[0];
        if (e->p->type != prim_type::eltwise || e->is_output || e->p->inputs.size() != 2) continue;
        if (e->p->eltw_mode != cldnn_eltwise_sum) continue;
        const bool keep_saturation = !e->p->eltw_with_act;
        if (keep_saturation) {
            // the stand-alone quantized sum: round((a + b) * factor[f]), saturated to the signed range
            // (reference generic_eltwise_ref.cl:318-330); s8 everywhere, no coefficients, quantized convolution
            bool ok = !e->p->eltw_calib.empty() && e->p->eltw_coefficients.empty() && !c->p->wqf.empty();
            for (node* t : {c, e, e->deps[0], e->deps[1]}) ok = ok && t->out.data_type == cldnn_i8;
            if (!ok) continue;
        }
        // Which convolutions the reference fuses (prepare_primitive_fusing.cpp:197-205): int8 in fs_bs_yx_bsv4_fsv32,
        // int8 / uint8 in b_fs_yx_fsv4, f32 in bfyx.  The blocked layout of this library stands where the reference has
        // fs_bs_yx_bsv4_fsv32, so the first case reads: an int8 convolution that the layout rule is going to run in
        // fs_b_yx_fsv16.  Any other int8 convolution in a plain layout (grouped ones, unquantized ones) stays unfused,
        // as in the reference: fused, the sum would see the unsaturated accumulator instead of the int8 tensor.
        const cldnn_layout& cl = c->out;
        const bool ok_type = (is_int8(cl.data_type) && (cl.format == cldnn_format_b_fs_yx_fsv4 || cl.format == cldnn_format_fs_b_yx_fsv16
                                                        || wants_blocked(c)))
                             || (cl.format == cldnn_format_bfyx && cl.data_type == cldnn_f32);
        if (!ok_type) continue;
        node* w = dep_named(c, c->p->weights.at(0));
        if (w->out.size.sizes[2] != 1 || w->out.size.sizes[3] != 1) continue;
        if (spatial(c->p->stride, 0) != 1 || spatial(c->p->stride, 1) != 1) continue;
        if (c->fused_act != activation_none) continue;
        // the convolution must be the later-executed input of the eltwise
        node* in0 = e->deps[0];
        node* in1 = e->deps[1];
        const int fused_idx = position(prog, in0) < position(prog, in1) ? 1 : 0;
        if (e->deps[fused_idx] != c) continue;
        node* other = e->deps[1 - fused_idx];

        auto f = std::make_shared<prim>(*c->p);
        f->type = prim_type::fused_conv_eltwise;
        f->id = c->p->id + "_fused_" + e->p->id;
        f->inputs = {c->p->inputs[0], other->p->id};
        f->eltw_calib = e->p->eltw_calib;
        f->eltw_oqf = e->p->eltw_oqf;
        f->eltw_mode = e->p->eltw_mode;
        f->eltw_with_act = e->p->eltw_with_act;
        f->eltw_slope = e->p->eltw_slope;
        f->conv_saturate = keep_saturation ? 1 : 0;
        f->non_conv_scale = 1.0f;
        f->output_padding = e->p->output_padding;
        f->out_dt.data_type = (cldnn_data_type)e->out.data_type;  // the fused primitive produces what the eltwise produced
        f->out_dt.enabled = 1;
        if (e->p->eltw_stride.size() == 2) {
            f->stride.sizes[2] *= e->p->eltw_stride[fused_idx].sizes[2];
            f->stride.sizes[3] *= e->p->eltw_stride[fused_idx].sizes[3];
            f->eltw_stride = {e->p->eltw_stride[1 - fused_idx]};
        } else {
            f->eltw_stride.clear();
        }
        node* nf = add_node(prog, f, e->org_id);
        nf->user_format = e->user_format;
        {
            // the fused node executes where the eltwise did: a later block must still find its own closing convolution
            // to be the later-executed input of its sum
            auto self = std::move(prog->nodes.back());
            prog->nodes.pop_back();
            prog->nodes.insert(prog->nodes.begin() + position(prog, e), std::move(self));
        }
        // dependencies: input, input2, weights, bias, wqf, calib, eltw calib
        nf->deps.push_back(c->deps[0]);
        nf->deps.push_back(other);
        for (size_t i = 1; i < c->deps.size(); ++i) nf->deps.push_back(c->deps[i]);
        for (size_t i = 2; i < e->deps.size(); ++i) nf->deps.push_back(e->deps[i]);
        for (node* d : nf->deps) d->users.push_back(nf);
        for (node* u : std::vector<node*>(e->users)) replace_dep(u, e, nf);
        remove_node(prog, e);
        remove_node(prog, c);
        calc_layout(nf);  // a later sum asks for the type of this one
    }
}

static bool quantized(const prim& p)
{
    if (p.type == prim_type::fused_conv_eltwise) return !p.wqf.empty();
    return !p.wqf.empty() || !p.calib.empty() || p.oqf != 1.0f;
}

// does this convolution run on the int8 matrix-core / depthwise kernels if its tensors are blocked?
static bool wants_blocked(node* n)
{
    const prim& p = *n->p;
    if (p.type != prim_type::convolution && p.type != prim_type::fused_conv_eltwise) return false;
    const cldnn_layout& in = n->deps[0]->out;
    node* w = dep_named(n, p.weights.at(0));
    if (!is_int8(in.data_type) || w->out.data_type != cldnn_i8) return false;
    const bool int_mode = quantized(p) || (p.type == prim_type::fused_conv_eltwise);
    if (!int_mode) return false;
    const int groups = p.groups ? (int)p.groups : 1;
    const bool depthwise = groups > 1 && groups == in.size.sizes[1] && groups == w->out.size.sizes[0];
    if (groups == 1 || depthwise) return true;
    // other group counts run on the matrix-core kernels with a block-diagonal weight matrix, up to 64 MiB of it
    if (p.weights.size() != 1) return false;
    const size_t dense = (size_t)w->out.size.sizes[0] * (size_t)in.size.sizes[1] * (size_t)w->out.size.sizes[2] * (size_t)w->out.size.sizes[3];
    return dense <= ((size_t)64 << 20);
}

// The layout rule that stands where the reference has byxf_af32 / fs_bs_yx_bsv4_fsv32 (which its own
// layout_optimizer never selects, src/layout_optimizer.cpp:245-250): quantized int8 convolutions run in
// fs_b_yx_fsv16; reorders are inserted where a tensor enters or leaves that format.
static void select_layouts(cldnn_program_impl* prog)
{
    std::map<std::pair<node*, int32_t>, node*> blocked_copy;  // (producer, format) -> its reorder into that format
    int counter = 0;
    auto blocked_version = [&](node* src, node* before, int32_t fmt = cldnn_format_fs_b_yx_fsv16) -> node* {
        if (src->out.format == fmt) return src;
        auto it = blocked_copy.find({src, fmt});
        if (it != blocked_copy.end()) return it->second;
        auto r = make_reorder(src->p->id + (fmt == cldnn_format_b_fs_yx_fsv4 ? "_to_fsv4_" : "_to_fsv16_") + std::to_string(counter++),
                              src->p->id, fmt);
        node* rn = add_node(prog, r, "");
        rn->deps = {src};
        src->users.push_back(rn);
        calc_layout(rn);
        // keep execution order: place the reorder right before its first consumer
        auto self = std::move(prog->nodes.back());
        prog->nodes.pop_back();
        prog->nodes.insert(prog->nodes.begin() + position(prog, before), std::move(self));
        blocked_copy[{src, fmt}] = rn;
        return rn;
    };
    for (size_t i = 0; i < prog->nodes.size(); ++i) {
        node* n = prog->nodes[i].get();
        if (n->constant) continue;
        for (node* d : n->deps)
            if (!d->constant && d->out.format == cldnn_format_any) calc_layout(d);
        if (wants_blocked(n)) {
            const int32_t user_format = n->user_format;
            // a first layer (at most 4 input features, no horizontal dilation) reads b_fs_yx_fsv4
            {
                node* wn = dep_named(n, n->p->weights.at(0));
                const int fx = wn->out.size.sizes[2], fy = wn->out.size.sizes[3];
                n->first_layer = n->p->type == prim_type::convolution && n->p->groups <= 1 && n->deps[0]->out.size.sizes[1] <= 4
                                 && spatial(n->p->dilation, 0) == 1 && n->deps[0]->out.format != cldnn_format_fs_b_yx_fsv16
                                 && (fy * ((fx + 3) / 4) + 3) / 4 <= 8;  // what the first-layer kernel holds in registers
            }
            node* a = blocked_version(n->deps[0], n, n->first_layer ? cldnn_format_b_fs_yx_fsv4 : cldnn_format_fs_b_yx_fsv16);
            if (a != n->deps[0]) replace_dep(n, n->deps[0], a);
            if (n->p->type == prim_type::fused_conv_eltwise && !n->p->second_input_in_output) {
                node* b = blocked_version(n->deps[1], n);
                if (b != n->deps[1]) replace_dep(n, n->deps[1], b);
            }
            calc_layout(n);
            i = position(prog, n);
            if (n->is_output && user_format != cldnn_format_fs_b_yx_fsv16) {
                // the user sees the result under the same id in the format the topology implies
                const std::string id = n->p->id;
                prog->by_id.erase(id);
                n->p = std::make_shared<prim>(*n->p);
                n->p->id = id + "_fsv16";
                prog->by_id[n->p->id] = n;
                auto r = make_reorder(id, n->p->id, user_format);
                node* rn = add_node(prog, r, n->org_id);
                rn->deps = {n};
                for (node* u : n->users)  // other consumers keep reading the blocked tensor
                    for (auto& s : u->p->inputs)
                        if (s == id) s = n->p->id;
                n->users.push_back(rn);
                rn->is_output = true;
                n->is_output = false;
                auto self = std::move(prog->nodes.back());
                prog->nodes.pop_back();
                prog->nodes.insert(prog->nodes.begin() + i + 1, std::move(self));
                calc_layout(rn);
            }
        } else {
            calc_layout(n);
            if (n->is_output && n->out.format == cldnn_format_fs_b_yx_fsv16 && n->p->type != prim_type::reorder) {
                // an elementwise node that inherited the blocked format from its producer
                const bool user_blocked = n->user_format == cldnn_format_fs_b_yx_fsv16;
                if (!user_blocked) {
                    const std::string id = n->p->id;
                    prog->by_id.erase(id);
                    n->p = std::make_shared<prim>(*n->p);
                    n->p->id = id + "_fsv16";
                    prog->by_id[n->p->id] = n;
                    auto r = make_reorder(id, n->p->id, n->user_format);
                    node* rn = add_node(prog, r, n->org_id);
                    rn->deps = {n};
                    n->users.push_back(rn);
                    rn->is_output = true;
                    n->is_output = false;
                    auto self = std::move(prog->nodes.back());
                    prog->nodes.pop_back();
                    prog->nodes.insert(prog->nodes.begin() + i + 1, std::move(self));
                    calc_layout(rn);
                }
            }
        }
    }
}

// Give the input of every padded blocked convolution a physical zero border, so the kernels address taps
// with constant offsets (reference prepare_padding.cpp does the same for its optimised kernels).
static void prepare_borders(cldnn_program_impl* prog)
{
    for (auto& u : prog->nodes) {
        node* n = u.get();
        if (!wants_blocked(n)) continue;
        if (n->deps[0]->out.format != cldnn_format_fs_b_yx_fsv16 && !(n->first_layer && n->deps[0]->out.format == cldnn_format_b_fs_yx_fsv4))
            continue;
        node* w = dep_named(n, n->p->weights.at(0));
        conv_geom g = conv_geometry(*n->p, n->deps[0]->out, w->out);
        if (g.px == 0 && g.py == 0 && g.FX == 1 && g.FY == 1) continue;
        node* src = n->deps[0];
        if (src->p->type == prim_type::input_layout || src->p->type == prim_type::data) continue;  // user memory: checked kernel
        const int hi_x = std::max(0, (g.OW - 1) * g.sx - g.px + (g.FX - 1) * g.dx - (g.IW - 1));
        const int hi_y = std::max(0, (g.OH - 1) * g.sy - g.py + (g.FY - 1) * g.dy - (g.IH - 1));
        cldnn_padding& pad = src->out.padding;
        pad.lower_size.sizes[2] = std::max(pad.lower_size.sizes[2], g.px);
        pad.lower_size.sizes[3] = std::max(pad.lower_size.sizes[3], g.py);
        pad.upper_size.sizes[2] = std::max(pad.upper_size.sizes[2], hi_x);
        pad.upper_size.sizes[3] = std::max(pad.upper_size.sizes[3], hi_y);
    }
}

// ------------------------------------------------------------------------------------------ compile
// prepare_buffer_fusing (reference src/graph_optimizer/prepare_buffer_fusing.cpp:38-140): the inputs of a concatenation
// write straight into the concatenation's buffer and the concatenation itself does nothing.  The reference expresses an
// input's place as output padding along the concatenation axis, which its kernels honour on every axis; the kernels
// here take borders in y and x only, so the pass applies where an input's place is one CONTIGUOUS piece of the buffer
// with the input's own layout: the concatenation axis is the outermost axis of the memory order that has more than one
// element -- feature slices in fs_b_yx_fsv16 (every input but the last a multiple of 16 features), the batch in bfyx, the
// features in bfyx at batch 1 -- and all tensors carry the same border.  As in the reference an input must not be an
// output or user memory, and (stricter) belongs to one in-place concatenation only and is no concatenation itself.
static void prepare_buffer_fusing(cldnn_program_impl* prog)
{
    for (auto& u : prog->nodes) {
        node* c = u.get();
        if (c->p->type != prim_type::concatenation) continue;
        const int axis = c->p->concat_axis;
        const cldnn_layout& out = c->out;
        const int B = out.size.sizes[0];
        bool outermost = false;
        if (out.format == cldnn_format_fs_b_yx_fsv16) outermost = axis == 1;
        else if (out.format == cldnn_format_bfyx) outermost = axis == 0 || (axis == 1 && B == 1);
        if (!outermost) continue;
        const size_t count = c->p->inputs.size();
        // one border for the whole group: the widest any member needs
        cldnn_padding pad = out.padding;
        bool ok = true;
        for (size_t k = 0; k < count && ok; ++k) {
            node* in = c->deps[k];
            ok = !in->constant && !in->is_output && in->p->type != prim_type::input_layout && in->p->type != prim_type::concatenation
                 && !in->concat_into && in->out.format == out.format && !in->side_stream
                 && !(in->p->type == prim_type::fused_conv_eltwise && in->p->second_input_in_output);
            for (size_t j = 0; j < k && ok; ++j) ok = c->deps[j] != in;  // the same tensor twice needs two copies
            if (ok && out.format == cldnn_format_fs_b_yx_fsv16 && k + 1 < count) ok = in->out.size.sizes[1] % 16 == 0;
            for (int i = 0; i < 4 && ok; ++i) {
                pad.lower_size.sizes[i] = std::max(pad.lower_size.sizes[i], in->out.padding.lower_size.sizes[i]);
                pad.upper_size.sizes[i] = std::max(pad.upper_size.sizes[i], in->out.padding.upper_size.sizes[i]);
            }
        }
        if (!ok) continue;
        c->out.padding = pad;
        size_t offset = 0;
        for (size_t k = 0; k < count; ++k) {
            node* in = c->deps[k];
            in->out.padding = pad;
            in->concat_into = c;
            in->concat_offset = offset;
            offset += layout_bytes(in->out);
        }
        c->concat_in_place = true;
    }
}

static int hip_act(int32_t f)
{
    switch (f) {
    case activation_none: return CLDNN_HIP_ACT_NONE;
    case activation_relu: return CLDNN_HIP_ACT_RELU;
    case activation_relu_negative_slope: return CLDNN_HIP_ACT_RELU_SLOPE;
    case activation_clamp: return CLDNN_HIP_ACT_CLAMP;
    default: throw api_error(CLDNN_INVALID_ARG, "activation function not supported by this library (none, relu, relu_negative_slope, clamp)");
    }
}
int hip_activation_code(int32_t f) { return hip_act(f); }

// pooling node -> descriptor of the C-ABI call (reference src/gpu/pooling_gpu.cpp:78-130)
cldnn_hip_pooling_desc pooling_descriptor(const node* n)
{
    const prim& p = *n->p;
    const pool_geom g = pooling_geometry(p, n->deps[0]->out);
    cldnn_hip_pooling_desc d{};
    d.input = to_hip(n->deps[0]->out), d.output = to_hip(n->out);
    d.mode = p.pool_mode == cldnn_pooling_max ? CLDNN_HIP_POOL_MAX : CLDNN_HIP_POOL_AVERAGE;
    d.divider = g.divider;
    d.size_y = g.ky, d.size_x = g.kx, d.stride_y = g.sy, d.stride_x = g.sx, d.pad_y = g.py, d.pad_x = g.px;
    return d;
}

// convolution / fused_conv_eltwise -> one cldnn_hip_conv object (reference convolution_gpu.cpp:71-162)
// descriptor and host copies of the constants of one convolution node
struct conv_build {
    cldnn_hip_conv_desc d{};
    std::vector<uint8_t> wv, bv, qv, cv, ev;
    const void* weights() const { return wv.data(); }
    const void* bias() const { return bv.empty() ? nullptr : bv.data(); }
    const float* wqf() const { return qv.empty() ? nullptr : (const float*)qv.data(); }
    const float* calib() const { return cv.empty() ? nullptr : (const float*)cv.data(); }
    const float* eltw_calib() const { return ev.empty() ? nullptr : (const float*)ev.data(); }
};

static void prepare_conv(cldnn_program_impl* prog, node* n, conv_build& cb)
{
    (void)prog;
    cldnn_hip_conv_desc& d = cb.d;
    std::vector<uint8_t>&wv = cb.wv, &bv = cb.bv, &qv = cb.qv, &cv = cb.cv, &ev = cb.ev;
    prim& p = *n->p;
    const bool fused = p.type == prim_type::fused_conv_eltwise;
    node* in = n->deps[0];
    node* w = dep_named(n, p.weights.at(0));
    conv_geom g = conv_geometry(p, in->out, w->out);
    const int ifm_g = g.IFM / g.groups;

    d.input = to_hip(in->out);
    // a positive input offset: the same buffer, seen as the smaller tensor with what is left out counted as border
    d.input.y = g.IH, d.input.x = g.IW;
    d.input.pad_lo_y += g.vy, d.input.pad_hi_y += g.vy, d.input.pad_lo_x += g.vx, d.input.pad_hi_x += g.vx;
    d.output = to_hip(n->out);
    d.weights_dtype = hip_dtype(w->out.data_type);
    HOST_REQUIRE(d.weights_dtype == CLDNN_HIP_S8 || d.weights_dtype == CLDNN_HIP_F32, CLDNN_INVALID_ARG, "weights must be i8 or f32");
    d.ofm = g.OFM, d.ifm = g.IFM, d.fy = g.FY, d.fx = g.FX;
    d.stride_y = g.sy, d.stride_x = g.sx, d.dilation_y = g.dy, d.dilation_x = g.dx;
    d.pad_y = g.py, d.pad_x = g.px, d.groups = g.groups;
    d.pad_end_delta_y = g.ey, d.pad_end_delta_x = g.ex;
    d.fully_connected = p.fully_connected ? 1 : 0;
    d.input_quantization_factor = p.iqf;
    d.output_quantization_factor = p.oqf;
    d.bias_dtype = CLDNN_HIP_NO_TYPE;

    // constants: one primitive per part of a split convolution, concatenated along the output features
    const size_t parts = p.weights.size();
    const size_t wcount = (size_t)g.OFM * ifm_g * g.FY * g.FX;
    auto gather = [&](const std::vector<std::string>& ids, size_t total, const char* what, size_t* dt) {
        HOST_REQUIRE(ids.size() == parts, CLDNN_INVALID_ARG, std::string(what) + ": one primitive per part of the split is needed");
        std::vector<uint8_t> all;
        for (const std::string& id : ids) {
            node* c = dep_named(n, id);
            if (dt) {
                HOST_REQUIRE(all.empty() || *dt == c->out.data_type, CLDNN_INVALID_ARG, std::string(what) + ": parts differ in data type");
                *dt = c->out.data_type;
            }
            std::vector<uint8_t> part = read_constant(c, total / parts, what);
            all.insert(all.end(), part.begin(), part.end());
        }
        return all;
    };
    size_t wdt = w->out.data_type, bdt = cldnn_f32, fdt = cldnn_f32;
    wv = gather(p.weights, wcount, "weights", &wdt);
    for (const std::string& id : p.weights) {
        const cldnn_layout& wl = dep_named(n, id)->out;
        HOST_REQUIRE(wl.format == cldnn_format_bfyx && wl.size.sizes[0] == w->out.size.sizes[0] && wl.size.sizes[1] == w->out.size.sizes[1]
                         && wl.size.sizes[2] == w->out.size.sizes[2] && wl.size.sizes[3] == w->out.size.sizes[3],
                     CLDNN_DIMENSION_MISMATCH, "the weights of a split convolution must agree in size and format");
    }
    if (!p.bias.empty()) {
        bv = gather(p.bias, g.OFM, "bias", &bdt);
        d.bias_dtype = hip_dtype(bdt);
        HOST_REQUIRE(d.bias_dtype == CLDNN_HIP_I32 || d.bias_dtype == CLDNN_HIP_F32, CLDNN_INVALID_ARG, "bias must be i32 or f32");
    }
    if (!p.wqf.empty()) {
        qv = gather(p.wqf, g.OFM, "weights_quantization_factors", &fdt);
        HOST_REQUIRE(fdt == cldnn_f32, CLDNN_INVALID_ARG, "weights_quantization_factors must be f32");
        d.has_wqf = 1;
    }
    if (!p.calib.empty()) {
        // the API requires quantization factors whenever calibration factors are given (reference api/CPP/convolution.hpp:462-463)
        HOST_REQUIRE(!p.wqf.empty() || fused, CLDNN_INVALID_ARG, "output_calibration_factors need weights_quantization_factors");
        fdt = cldnn_f32;
        cv = gather(p.calib, g.OFM, "output_calibration_factors", &fdt);
        HOST_REQUIRE(fdt == cldnn_f32, CLDNN_INVALID_ARG, "output_calibration_factors must be f32");
        d.has_calib = 1;
    }
    // with_activation overrides whatever activation was folded in (reference convolution_gpu.cpp:100-101)
    if (p.with_activation) {
        d.activation = p.act_slope == 0.0f ? CLDNN_HIP_ACT_RELU : CLDNN_HIP_ACT_RELU_SLOPE;
        d.activation_m = p.act_slope;
    } else {
        d.activation = hip_act(n->fused_act);
        d.activation_m = n->fused_a, d.activation_n = n->fused_b;
    }
    if (fused) {
        HOST_REQUIRE(p.eltw_mode == cldnn_eltwise_sum, CLDNN_INVALID_ARG, "fused_conv_eltwise supports the sum mode only");
        d.fused = 1;
        d.non_conv_scale = p.non_conv_scale;
        d.second_input_in_output = p.second_input_in_output ? 1 : 0;
        d.conv_saturate = p.conv_saturate;
        if (!p.second_input_in_output) d.eltw = to_hip(n->deps[1]->out);
        if (p.eltw_with_act) {
            d.eltw_activation = p.eltw_slope == 0.0f ? CLDNN_HIP_ACT_RELU : CLDNN_HIP_ACT_RELU_SLOPE;
            d.eltw_activation_m = p.eltw_slope;
        }
        d.eltw_stride_x = d.eltw_stride_y = 1;
        if (!p.eltw_stride.empty()) d.eltw_stride_x = p.eltw_stride[0].sizes[2], d.eltw_stride_y = p.eltw_stride[0].sizes[3];
        if (!p.eltw_calib.empty()) {
            node* c = dep_named(n, p.eltw_calib);
            ev = read_constant(c, g.OFM, "eltwise output_calibration_factors");
            d.has_eltw_calib = 1;
        }
    }
    d.impl = CLDNN_HIP_IMPL_AUTO;
}

// Build option tuning_config: which row of the tile table runs this convolution.  Reference
// src/gpu/convolution_gpu.cpp:147-154, kernel_selector/core/kernel_selector.cpp GetAutoTuneBestKernel: take the cached choice;
// in tune_and_cache mode measure what the cache does not hold and add it.  Applies to every convolution object the
// program creates, a pair of convolutions in one launch included; a chain has no rows to choose from and is kept.
static void apply_tuning(cldnn_program_impl* prog, cldnn_hip_conv_desc& d, const void* weights, const void* bias, const float* wqf,
                         const float* calib, const float* eltw_calib)
{
    if (prog->tuning.mode == cldnn_tuning_disabled) return;
    cldnn_hip_engine_info info{};
    hip_check(cldnn_hip_engine_get_info(prog->engine->h, &info));
    const std::string key = conv_signature(d);
    std::string name;
    int row = -1;
    if (prog->tuning.find(info.cores_count, key, &name, &row)) {
        if (row >= 0 && row < cldnn_hip_tile_config_count() && name == cldnn_hip_tile_config_name(row)) d.tile_override = row + 1;
        ++prog->tuned_from_cache;
    } else if (prog->tuning.mode == cldnn_tuning_tune_and_cache) {
        float best_us = 0.0f;
        hip_check(cldnn_hip_conv_tune(prog->engine->h, &d, weights, bias, wqf, calib, eltw_calib, 20, &row, &best_us, nullptr, nullptr));
        prog->tuning.store(info.cores_count, key, row >= 0 ? cldnn_hip_tile_config_name(row) : "table", row);
        if (row >= 0) d.tile_override = row + 1;
        ++prog->tuned_now;
    }
}

static void compile_conv(cldnn_program_impl* prog, node* n)
{
    conv_build cb;
    prepare_conv(prog, n, cb);
    cldnn_hip_conv_desc& d = cb.d;
    const void* bias_ptr = cb.bias();
    const float* wqf_ptr = cb.wqf();
    const float* calib_ptr = cb.calib();
    const void* eltw_calib = cb.eltw_calib();
    std::vector<uint8_t>& wv = cb.wv;
    apply_tuning(prog, d, wv.data(), bias_ptr, wqf_ptr, calib_ptr, (const float*)eltw_calib);
    hip_check(cldnn_hip_conv_create(n->side_stream ? prog->engine->side : prog->engine->h, &d, wv.data(), bias_ptr, wqf_ptr, calib_ptr,
                                    (const float*)eltw_calib, &n->conv));
    hip_check(cldnn_hip_conv_get_info(n->conv, &n->conv_info));
}

// ------------------------------------------------------------------------------------------ sibling convolutions
// Two quantized convolutions that read the same tensor with the same filter size, stride, padding and dilation (a
// residual block's shortcut projection and its opening 1x1; the 1x1 branches of an inception module) run as ONE launch
// over the concatenated output features (cldnn_hip_conv_desc.sibling_split).  The reference launches every node
// (src/gpu/primitive_gpu_base.h:117-168); the results per feature are the same.  In fs_b_yx_fsv16 the second result is the
// contiguous tail of the pair's buffer, so both nodes keep output tensors of their own for their readers.  The pair
// takes the wider of the two borders.  Whether the kernels have a short epilogue for the pair is decided when it is
// compiled (compile_siblings); a pair they refuse is taken apart again.
static bool sibling_candidate(const node* n)
{
    const prim& p = *n->p;
    if (p.type != prim_type::convolution || p.fully_connected || p.split != 1 || p.groups != 1) return false;
    if (n->is_output || n->side_stream || n->first_layer || n->concat_into || n->concat_in_place || n->sibling || n->sibling_head) return false;
    if (n->chain_head || !n->chain_members.empty()) return false;
    if (p.wqf.empty() || p.calib.empty() || p.iqf != 1.0f) return false;
    for (const node* u : n->users)  // a sum written over this tensor needs it in a buffer of its own
        if (u->p->type == prim_type::fused_conv_eltwise && u->p->second_input_in_output && u->deps.size() > 1 && u->deps[1] == n) return false;
    const auto int8 = [](int32_t t) { return t == cldnn_i8 || t == cldnn_u8; };
    return n->out.format == cldnn_format_fs_b_yx_fsv16 && n->deps[0]->out.format == cldnn_format_fs_b_yx_fsv16 && int8(n->out.data_type)
           && int8(n->deps[0]->out.data_type);
}

static void pair_siblings(cldnn_program_impl* prog)
{
    for (size_t i = 0; i < prog->nodes.size(); ++i) {
        node* a = prog->nodes[i].get();
        if (!sibling_candidate(a) || a->out.size.sizes[1] % 16 != 0) continue;
        const conv_geom ga = conv_geometry(*a->p, a->deps[0]->out, dep_named(a, a->p->weights.at(0))->out);
        for (node* b : a->deps[0]->users) {
            if (b == a || !sibling_candidate(b) || b->deps[0] != a->deps[0] || position(prog, b) < i) continue;
            if (b->out.data_type != a->out.data_type || b->p->bias.empty() != a->p->bias.empty()) continue;
            const conv_geom gb = conv_geometry(*b->p, b->deps[0]->out, dep_named(b, b->p->weights.at(0))->out);
            if (gb.FY != ga.FY || gb.FX != ga.FX || gb.sy != ga.sy || gb.sx != ga.sx || gb.py != ga.py || gb.px != ga.px || gb.dy != ga.dy
                || gb.dx != ga.dx || gb.ey != ga.ey || gb.ex != ga.ex || gb.vy != ga.vy || gb.vx != ga.vx || gb.OH != ga.OH || gb.OW != ga.OW)
                continue;
            a->unpaired_padding = a->out.padding, b->unpaired_padding = b->out.padding;
            for (int k = 0; k < 4; ++k) {
                int32_t& la = a->out.padding.lower_size.sizes[k], &lb = b->out.padding.lower_size.sizes[k];
                int32_t& ua = a->out.padding.upper_size.sizes[k], &ub = b->out.padding.upper_size.sizes[k];
                la = lb = std::max(la, lb), ua = ub = std::max(ua, ub);
            }
            a->sibling = b, b->sibling_head = a;
            break;
        }
    }
}

// One convolution object for a pair.  false: the kernels have no short form for this pair (the pair is taken apart).
static bool compile_siblings(cldnn_program_impl* prog, node* a);

static bool compile_siblings(cldnn_program_impl* prog, node* a)
{
    node* b = a->sibling;
    conv_build ca, cb;
    prepare_conv(prog, a, ca);
    prepare_conv(prog, b, cb);
    cldnn_hip_conv_desc d = ca.d;
    const bool alike = ca.d.bias_dtype == cb.d.bias_dtype && ca.d.weights_dtype == cb.d.weights_dtype && cb.d.has_wqf && cb.d.has_calib
                       && ca.d.has_wqf && ca.d.has_calib;
    if (alike) {
        d.sibling_split = ca.d.ofm;
        d.sibling_activation = cb.d.activation, d.sibling_activation_m = cb.d.activation_m, d.sibling_activation_n = cb.d.activation_n;
        d.ofm = ca.d.ofm + cb.d.ofm;
        d.output.f = d.ofm;
        auto join = [](std::vector<uint8_t>& x, const std::vector<uint8_t>& y) { x.insert(x.end(), y.begin(), y.end()); };
        join(ca.wv, cb.wv), join(ca.bv, cb.bv), join(ca.qv, cb.qv), join(ca.cv, cb.cv);
        cldnn_hip_conv c = nullptr;
        apply_tuning(prog, d, ca.weights(), ca.bias(), ca.wqf(), ca.calib(), nullptr);
        const cldnn_hip_status st = cldnn_hip_conv_create(prog->engine->h, &d, ca.weights(), ca.bias(), ca.wqf(), ca.calib(), nullptr, &c);
        if (st == CLDNN_HIP_SUCCESS) {
            cldnn_hip_conv_info info{};
            hip_check(cldnn_hip_conv_get_info(c, &info));
            if (!std::strstr(info.kernel_name, "generic")) {
                a->conv = c, a->conv_info = info;
                return true;
            }
            cldnn_hip_conv_release(c);  // element by element two launches are faster
        } else if (st != CLDNN_HIP_UNSUPPORTED_FORMAT && st != CLDNN_HIP_UNSUPPORTED_SIZE) {
            hip_check(st);
        }
    }
    // taken apart: each side gets its own border back (nothing has been compiled against the wider one yet: the nodes
    // that read these tensors come later in the order)
    a->out.padding = a->unpaired_padding, b->out.padding = b->unpaired_padding;
    a->sibling = nullptr, b->sibling_head = nullptr;
    return false;
}

// ------------------------------------------------------------------------------------------ convolution chains
// A convolution and the one or two 1x1 / stride-1 / unpadded convolutions that read its result run as ONE launch
// (cldnn_hip_conv_chain): the tail of a ResNet bottleneck (3x3 -> 1x1 + sum -> the next block's 1x1) or of a MobileNet
// block (depthwise 3x3 -> 1x1 -> the next block's 1x1).  The reference launches every node
// (src/gpu/primitive_gpu_base.h:117-168); results are the same bits.  A follower moves up in the execution order to
// sit right behind its predecessor, which is allowed when everything else it reads (the residual operand) is produced
// before the head; results that other nodes read, or that are outputs, are written (keep), the rest never leaves
// the registers.  Whether the kernels can run the group as a chain is decided by cldnn_hip_conv_chain_create (feature
// counts, weights that fit into LDS ...); what it refuses runs node by node.
static bool chain_follower(cldnn_program_impl* prog, node* prev, node* c, size_t head_pos)
{
    const prim& p = *c->p;
    if (p.type != prim_type::convolution && p.type != prim_type::fused_conv_eltwise) return false;
    if (p.fully_connected || p.second_input_in_output || c->side_stream || c->first_layer || c->deps[0] != prev) return false;
    if (c->sibling || c->sibling_head) return false;
    node* w = dep_named(c, p.weights.at(0));
    const conv_geom g = conv_geometry(p, prev->out, w->out);
    if (g.FY != 1 || g.FX != 1 || g.sy != 1 || g.sx != 1 || g.py != 0 || g.px != 0 || g.groups != 1) return false;
    for (size_t i = 1; i < c->deps.size(); ++i)  // the residual operand has to exist when the head starts
        if (!c->deps[i]->constant && position(prog, c->deps[i]) >= head_pos) return false;
    return true;
}

static void group_chains(cldnn_program_impl* prog)
{
    for (size_t i = 0; i < prog->nodes.size(); ++i) {
        node* head = prog->nodes[i].get();
        const prim& hp = *head->p;
        if (head->chain_head || (hp.type != prim_type::convolution && hp.type != prim_type::fused_conv_eltwise)) continue;
        if (head->sibling || head->sibling_head) continue;  // launched as a pair
        if (hp.fully_connected || hp.second_input_in_output || head->side_stream || head->first_layer) continue;
        if (head->out.format != cldnn_format_fs_b_yx_fsv16 || head->deps[0]->out.format != cldnn_format_fs_b_yx_fsv16) continue;
        std::vector<node*> members{head};
        while (members.size() < 3) {
            node* prev = members.back();
            node* next = nullptr;
            for (node* u : prev->users)
                if (!u->chain_head && chain_follower(prog, prev, u, i)) {
                    next = u;
                    break;
                }
            if (!next) break;
            members.push_back(next);
        }
        if (members.size() < 2) continue;
        // followers move up behind the head
        for (size_t k = 1; k < members.size(); ++k) {
            const size_t from = position(prog, members[k]);
            std::unique_ptr<node> moved = std::move(prog->nodes[from]);
            prog->nodes.erase(prog->nodes.begin() + from);
            prog->nodes.insert(prog->nodes.begin() + i + k, std::move(moved));
            members[k]->chain_head = head;
        }
        head->chain_members = members;
        for (size_t k = 0; k < members.size(); ++k) {
            bool keep = members[k]->is_output || k + 1 == members.size();
            for (node* u : members[k]->users) keep = keep || k + 1 >= members.size() || u != members[k + 1];
            head->chain_keep.push_back(keep ? 1 : 0);
        }
    }
}

// Create the chain of a head node; members the kernels refuse as a chain are compiled one by one (a group of three is
// tried as its first two members as well).
static void compile_chain(cldnn_program_impl* prog, node* head)
{
    std::vector<node*> members = head->chain_members;
    std::vector<conv_build> cb(members.size());
    for (size_t k = 0; k < members.size(); ++k) prepare_conv(prog, members[k], cb[k]);
    for (size_t count = members.size(); count >= 2 && !head->chain; --count) {
        std::vector<cldnn_hip_conv_desc> descs;
        std::vector<const void*> w, b;
        std::vector<const float*> q, c, e;
        std::vector<int32_t> keep(head->chain_keep.begin(), head->chain_keep.begin() + count);
        keep[count - 1] = 1;
        for (size_t k = 0; k < count; ++k) {
            descs.push_back(cb[k].d);
            w.push_back(cb[k].weights()), b.push_back(cb[k].bias()), q.push_back(cb[k].wqf()), c.push_back(cb[k].calib());
            e.push_back(cb[k].eltw_calib());
        }
        const cldnn_hip_status st = cldnn_hip_conv_chain_create(prog->engine->h, (int32_t)count, descs.data(), w.data(), b.data(), q.data(),
                                                                c.data(), e.data(), keep.data(), &head->chain);
        if (st == CLDNN_HIP_SUCCESS) {
            head->chain_keep = keep;
            for (size_t k = count; k < members.size(); ++k) members[k]->chain_head = nullptr;
            members.resize(count);
            head->chain_members = members;
            hip_check(cldnn_hip_conv_chain_get_info(head->chain, &head->conv_info));
            for (size_t k = 1; k < count; ++k) {
                members[k]->conv_info = cldnn_hip_conv_info{};
                std::snprintf(members[k]->conv_info.kernel_name, sizeof(members[k]->conv_info.kernel_name), "in the chain of %s",
                              head->p->id.substr(0, 40).c_str());
            }
            return;
        }
        if (st != CLDNN_HIP_UNSUPPORTED_FORMAT) hip_check(st);
    }
    for (node* m : members) m->chain_head = nullptr;
    head->chain_members.clear();
    head->chain_keep.clear();
}

// enable_parallelisation (reference api/C/cldnn.h:152, "parallel execution of primitives which don't depend on each
// other"): a convolution whose only user comes at least two primitives later in execution order -- the projection
// shortcut of a residual block -- runs on the engine's second stream while the primitives in between run on the
// first; the user waits for it.
static void assign_streams(cldnn_program_impl* prog)
{
    for (size_t i = 0; i < prog->nodes.size(); ++i) {
        node* x = prog->nodes[i].get();
        if (x->constant || x->is_output || x->users.size() != 1) continue;
        if (x->p->type != prim_type::convolution || x->p->fully_connected) continue;
        bool plain_deps = true;
        for (node* d : x->deps) plain_deps = plain_deps && !d->side_stream;
        if (!plain_deps) continue;
        node* user = x->users[0];
        if (user->p->type == prim_type::fused_conv_eltwise && user->p->second_input_in_output && !user->rw_opt) continue;
        size_t between = 0;  // primitives that execute between the two
        const size_t pu = position(prog, user);
        for (size_t k = i + 1; k < pu; ++k)
            if (!prog->nodes[k]->constant && prog->nodes[k]->p->type != prim_type::input_layout) ++between;
        if (pu == (size_t)-1 || pu <= i || between == 0) continue;
        x->side_stream = true;
    }
}

// prepare_conv_eltw_read_write_opt (reference prepare_primitive_fusing.cpp:468-534): a fused_conv_eltwise whose
// output layout equals its second input's writes over that input (second_input_in_output): every thread reads the
// residual values it is about to replace, so the sum needs no buffer of its own.  The reference shares the buffer
// whatever else reads the second input; here every other reader has to come earlier in the execution order, and
// tensors the application sees (inputs, constants, outputs) are left alone.  Results do not depend on it.
static bool layouts_equal(const cldnn_layout& a, const cldnn_layout& b)
{
    if (a.data_type != b.data_type || a.format != b.format) return false;
    for (int i = 0; i < 4; ++i)
        if (a.size.sizes[i] != b.size.sizes[i] || a.padding.lower_size.sizes[i] != b.padding.lower_size.sizes[i]
            || a.padding.upper_size.sizes[i] != b.padding.upper_size.sizes[i])
            return false;
    return true;
}

static void conv_eltw_read_write_opt(cldnn_program_impl* prog)
{
    for (size_t i = 0; i < prog->nodes.size(); ++i) {
        node* n = prog->nodes[i].get();
        if (n->p->type != prim_type::fused_conv_eltwise || n->p->second_input_in_output || n->is_output || n->concat_into) continue;
        node* r = n->deps[1];
        if (r->constant || r->is_output || r->p->type == prim_type::input_layout || r->concat_into || r->concat_in_place) continue;
        if (!layouts_equal(r->out, n->out)) continue;
        bool last_reader = true;
        for (node* u : r->users) last_reader = last_reader && (u == n || position(prog, u) < i);
        if (!last_reader) continue;
        n->p = std::make_shared<prim>(*n->p);
        n->p->second_input_in_output = true;
        n->rw_opt = true;
    }
}

// ------------------------------------------------------------------------------------------ build
void build_program(cldnn_program_impl* prog, cldnn_topology_impl* topo, const std::vector<std::string>& outputs)
{
    // nodes + dependencies
    for (const std::string& id : topo->order) add_node(prog, std::make_shared<prim>(*topo->prims.at(id)), id);
    prog->all_org_ids = topo->order;
    auto link = [&](node* n, const std::string& id) {
        auto it = prog->by_id.find(id);
        HOST_REQUIRE(it != prog->by_id.end(), CLDNN_INVALID_ARG, "primitive " + n->p->id + " refers to unknown primitive " + id);
        n->deps.push_back(it->second);
        it->second->users.push_back(n);
    };
    for (auto& u : prog->nodes) {
        node* n = u.get();
        prim& p = *n->p;
        for (auto& s : p.inputs) link(n, s);
        for (auto* v : {&p.weights, &p.bias, &p.wqf, &p.calib})
            for (auto& s : *v) link(n, s);
        if (!p.eltw_calib.empty()) link(n, p.eltw_calib);
        const size_t need = (p.type == prim_type::input_layout || p.type == prim_type::data) ? 0
                            : (p.type == prim_type::eltwise || p.type == prim_type::fused_conv_eltwise) ? 2 : 1;
        HOST_REQUIRE(p.inputs.size() >= need, CLDNN_INVALID_ARG, "primitive " + p.id + " has too few inputs");
    }
    // outputs: the build option's list, else every primitive nobody consumes (reference program.cpp mark_outputs)
    if (!outputs.empty()) {
        for (auto& id : outputs) {
            auto it = prog->by_id.find(id);
            HOST_REQUIRE(it != prog->by_id.end(), CLDNN_INVALID_ARG, "unknown output primitive " + id);
            it->second->is_output = true;
        }
    } else {
        for (auto& u : prog->nodes)
            if (u->users.empty() && !u->constant) u->is_output = true;
    }
    sort_nodes(prog);
    for (auto& u : prog->nodes) u->out.format = cldnn_format_any;
    for (auto& u : prog->nodes) calc_layout(u.get());  // layouts in the user's formats (also validates)
    for (auto& u : prog->nodes) u->user_format = u->out.format;

    if (prog->optimize_data) {
        fuse_activations(prog);
        eltwise_shrinking(prog);
        eltwise_remove_stride(prog);
        fuse_conv_eltwise(prog);
        sort_nodes(prog);
        for (auto& u : prog->nodes) u->out.format = cldnn_format_any;
        for (auto& u : prog->nodes)
            if (u->constant || u->p->type == prim_type::input_layout) calc_layout(u.get());
        select_layouts(prog);
    }
    for (auto& u : prog->nodes) calc_layout(u.get());
    prepare_borders(prog);
    if (prog->optimize_data) prepare_buffer_fusing(prog);
    // with the memory pool on, buffers are recycled anyway and the in-place form measures 1.7 % slower on ResNet-50
    // (same kernels; reads and writes of one launch then share their cache lines), so the pass serves engines without a pool
    if (prog->optimize_data && prog->engine && !prog->engine->memory_pool) conv_eltw_read_write_opt(prog);
    if (!prog->engine) return;  // planning only: the graph is inspected, nothing is compiled
    if (prog->engine->side) assign_streams(prog);
    // pairs and chains come with the graph optimisations; a tuning cache composes with them (it picks the rows of the
    // launches that have rows: single convolutions and pairs)
    if (prog->optimize_data) {
        pair_siblings(prog);
        for (auto& u : prog->nodes)
            if (u->sibling) compile_siblings(prog, u.get());
        group_chains(prog);
    }
    for (auto& u : prog->nodes) {
        node* n = u.get();
        if (!n->chain_members.empty()) compile_chain(prog, n);
    }
    for (auto& u : prog->nodes) {
        node* n = u.get();
        const bool conv = n->p->type == prim_type::convolution || n->p->type == prim_type::fused_conv_eltwise;
        if (conv && !n->conv && !n->chain && !n->chain_head && !n->sibling_head) compile_conv(prog, n);
    }
    prog->tuning.save();
}

// ------------------------------------------------------------------------------------------ inspection
static std::string four(const int32_t* s)
{
    return "[" + std::to_string(s[0]) + "," + std::to_string(s[1]) + "," + std::to_string(s[2]) + "," + std::to_string(s[3]) + "]";
}

// one node as JSON; sizes and paddings are [b, f, x, y] like cldnn_tensor::sizes
// Primitives on the second stream whose completion the launch of n has to wait for: what n reads and, for the head of
// a chain, what ANY member reads (its one kernel does the work of all of them, e.g. a follower's residual operand that
// a shortcut convolution on the second stream produces).
std::vector<node*> launch_waits(const node* n)
{
    std::vector<node*> w;
    auto add = [&](const node* m) {
        for (node* d : m->deps)
            if (d->side_stream && std::find(w.begin(), w.end(), d) == w.end()) w.push_back(d);
    };
    add(n);
    for (const node* m : n->chain_members) add(m);
    if (n->sibling) add(n->sibling);
    return w;
}

std::string describe_node(const node* n)
{
    static const char* tn[] = {"input_layout", "data", "reorder", "activation", "eltwise", "convolution", "fused_conv_eltwise", "pooling",
                               "concatenation"};
    const prim& p = *n->p;
    std::string s = "{\"id\":\"" + p.id + "\",\"type\":\"" + tn[(int)p.type] + "\",\"org_id\":\"" + n->org_id + "\",\"deps\":[";
    for (size_t i = 0; i < n->deps.size(); ++i) s += std::string(i ? "," : "") + "\"" + n->deps[i]->p->id + "\"";
    s += "],\"is_output\":" + std::string(n->is_output ? "true" : "false");
    s += ",\"format\":" + std::to_string(n->out.format) + ",\"data_type\":" + std::to_string(n->out.data_type);
    s += ",\"size\":" + four(n->out.size.sizes) + ",\"pad_lower\":" + four(n->out.padding.lower_size.sizes) + ",\"pad_upper\":"
         + four(n->out.padding.upper_size.sizes);
    if (p.type == prim_type::convolution || p.type == prim_type::fused_conv_eltwise) {
        if (p.fully_connected) s += ",\"fully_connected\":true";
        s += ",\"stride\":" + four(p.stride.sizes) + ",\"fused_activation\":" + std::to_string(n->fused_act);
        s += ",\"fused_activation_params\":[" + std::to_string(n->fused_a) + "," + std::to_string(n->fused_b) + "]";
    }
    if (p.type == prim_type::fused_conv_eltwise) {
        s += ",\"eltw_stride\":" + (p.eltw_stride.empty() ? std::string("null") : four(p.eltw_stride[0].sizes));
        s += ",\"eltw_slope\":" + std::to_string(p.eltw_slope) + ",\"eltw_calib\":\"" + p.eltw_calib + "\"";
        if (p.second_input_in_output) s += ",\"second_input_in_output\":true";
        if (p.conv_saturate) s += ",\"conv_saturate\":" + std::to_string(p.conv_saturate);
    }
    if (p.type == prim_type::eltwise) {
        s += ",\"mode\":" + std::to_string(p.eltw_mode) + ",\"strides\":[";
        for (size_t i = 0; i < p.eltw_stride.size(); ++i) s += (i ? "," : "") + four(p.eltw_stride[i].sizes);
        s += "]";
    }
    if (p.type == prim_type::concatenation) s += ",\"axis\":" + std::to_string(p.concat_axis) + ",\"in_place\":" + (n->concat_in_place ? "true" : "false");
    if (n->concat_into) s += ",\"concat_into\":\"" + n->concat_into->p->id + "\",\"concat_offset\":" + std::to_string(n->concat_offset);
    if (n->side_stream) s += ",\"stream\":1";
    if (!n->chain_head && !n->sibling_head) {
        const std::vector<node*> waits = launch_waits(n);
        if (!waits.empty()) {
            s += ",\"waits_for\":[";
            for (size_t i = 0; i < waits.size(); ++i) s += (i ? ",\"" : "\"") + waits[i]->p->id + "\"";
            s += "]";
        }
    }
    if (n->sibling) s += ",\"launches_also\":\"" + n->sibling->p->id + "\"";
    if (n->sibling_head) s += ",\"launched_by\":\"" + n->sibling_head->p->id + "\"";
    if (n->conv || n->chain || n->chain_head)
        s += std::string(",\"kernel\":\"") + n->conv_info.kernel_name + "\",\"grid\":" + std::to_string(n->conv_info.grid)
             + ",\"ops\":" + std::to_string(n->conv_info.ops) + ",\"bytes\":" + std::to_string(n->conv_info.bytes);
    return s + "}";
}

std::string describe_program(const cldnn_program_impl* prog)
{
    std::string s = "[";
    for (size_t i = 0; i < prog->nodes.size(); ++i) s += (i ? "," : "") + describe_node(prog->nodes[i].get());
    return s + "]";
}

}  // namespace host
