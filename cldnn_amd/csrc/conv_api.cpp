// Convolution objects of the C-ABI: validation, arithmetic-mode selection, kernel-family and
// tile choice (the gfx950 tile-config table stands where the reference has kernel_selector and
// its tuning cache), weight pre-packing, launch.
#include <algorithm>
#include <chrono>
#include <cstring>
#include <vector>

#include "conv_chain.h"
#include "kernels.h"
#include "runtime.h"

using namespace chip;

struct cldnn_hip_conv_s {
    cldnn_hip_engine engine = nullptr;
    cldnn_hip_conv_desc desc{};
    ConvProblem p{};
    Epilogue epi{};       // device pointers inside
    int impl = CLDNN_HIP_IMPL_REF;
    bool fast = false;
    FastEpi fe{};
    MfmaPlan mplan{};
    DwPlan dplan{};
    // device allocations
    void* w_raw = nullptr;    // dense weights (reference kernel)
    void* w_packed = nullptr; // MFMA / depthwise operand stream
    void* w_masked = nullptr; // depthwise 3x3 kernel: one weight byte per dword
    void* ktab = nullptr;
    void* gather = nullptr;   // scratch of the small-batch kernel (activations in fragment order)
    void* acc_init = nullptr;      // int32: offset correction + int32 bias
    void* acc_init_raw = nullptr;  // int32: offset correction only (accumulator probe)
    void* bias = nullptr;
    void* wqf = nullptr;
    void* calib = nullptr;
    void* ecal = nullptr;
    cldnn_hip_conv_info info{};
    std::vector<void*> owned;
};

struct cldnn_hip_conv_chain_s {
    cldnn_hip_engine engine = nullptr;
    int count = 0;
    cldnn_hip_conv stage[3] = {nullptr, nullptr, nullptr};
    int keep[3] = {0, 0, 0};
    ChainStageIn in[3]{};
    ChainPlan plan{};
    void* packed = nullptr;
    cldnn_hip_conv_info info{};
};

namespace {

bool is_int8(int dt) { return dt == CLDNN_HIP_S8 || dt == CLDNN_HIP_U8; }

int out_extent(int in, int pad, int filt, int dil, int stride, int pad_end_delta = 0)
{
    // reference src/include/sliding_window_utils.h:113-126; a window larger than the padded input gives 1
    const int wnd = (filt - 1) * dil + 1;
    const int span = in + 2 * pad + pad_end_delta;
    if (wnd > span) return 1;
    return (span - wnd) / stride + 1;
}

void* upload(cldnn_hip_conv c, const void* host, size_t bytes, size_t padded_bytes = 0)
{
    if (padded_bytes < bytes) padded_bytes = bytes;
    void* d = nullptr;
    hipError_t r = hipMalloc(&d, padded_bytes + 64);
    if (r != hipSuccess) {
        (void)hipGetLastError();
        throw error(CLDNN_HIP_OUT_OF_RESOURCES, std::string("hipMalloc: ") + hipGetErrorString(r));
    }
    c->owned.push_back(d);
    CHIP_CHECK(hipMemsetAsync(d, 0, padded_bytes + 64, c->engine->stream));
    if (host && bytes) CHIP_CHECK(hipMemcpyAsync(d, host, bytes, hipMemcpyHostToDevice, c->engine->stream));
    CHIP_CHECK(hipStreamSynchronize(c->engine->stream));
    return d;
}

void build(cldnn_hip_conv c, const void* weights, const void* bias, const float* wqf, const float* calib,
           const float* eltw_calib)
{
    const cldnn_hip_conv_desc& d = c->desc;
    ConvProblem& p = c->p;
    CHIP_REQUIRE(weights, CLDNN_HIP_INVALID_ARG, "convolution without weights");
    CHIP_REQUIRE(d.groups >= 1 && d.ifm % d.groups == 0 && d.ofm % d.groups == 0, CLDNN_HIP_INVALID_ARG,
                 "feature counts must divide into groups");
    CHIP_REQUIRE(d.fy > 0 && d.fx > 0 && d.stride_y > 0 && d.stride_x > 0 && d.dilation_y > 0 && d.dilation_x > 0,
                 CLDNN_HIP_INVALID_ARG, "filter size, stride and dilation must be positive");
    CHIP_REQUIRE(d.pad_y >= 0 && d.pad_x >= 0 && d.pad_y + d.pad_end_delta_y >= 0 && d.pad_x + d.pad_end_delta_x >= 0,
                 CLDNN_HIP_INVALID_ARG, "negative padding");
    CHIP_REQUIRE(d.input.f == d.ifm, CLDNN_HIP_DIMENSION_MISMATCH, "input feature count differs from weights");
    CHIP_REQUIRE(d.output.f == d.ofm && d.output.b == d.input.b, CLDNN_HIP_DIMENSION_MISMATCH,
                 "output batch/feature count mismatch");
    CHIP_REQUIRE((d.has_wqf != 0) == (wqf != nullptr), CLDNN_HIP_INVALID_ARG, "has_wqf does not match the wqf pointer");
    CHIP_REQUIRE((d.has_calib != 0) == (calib != nullptr), CLDNN_HIP_INVALID_ARG, "has_calib does not match the calib pointer");
    CHIP_REQUIRE((d.has_eltw_calib != 0) == (eltw_calib != nullptr), CLDNN_HIP_INVALID_ARG,
                 "has_eltw_calib does not match the eltw_calib pointer");
    CHIP_REQUIRE((d.bias_dtype != CLDNN_HIP_NO_TYPE) == (bias != nullptr), CLDNN_HIP_INVALID_ARG,
                 "bias_dtype does not match the bias pointer");
    if (bias) CHIP_REQUIRE(d.bias_dtype == CLDNN_HIP_I32 || d.bias_dtype == CLDNN_HIP_F32, CLDNN_HIP_INVALID_ARG, "bias must be i32 or f32");

    p.B = d.input.b, p.IFM = d.ifm, p.IH = d.input.y, p.IW = d.input.x, p.OFM = d.ofm;
    p.FY = d.fy, p.FX = d.fx, p.sy = d.stride_y, p.sx = d.stride_x, p.dy = d.dilation_y, p.dx = d.dilation_x;
    p.py = d.pad_y, p.px = d.pad_x, p.groups = d.groups;
    p.OH = out_extent(p.IH, p.py, p.FY, p.dy, p.sy, d.pad_end_delta_y);
    p.OW = out_extent(p.IW, p.px, p.FX, p.dx, p.sx, d.pad_end_delta_x);
    CHIP_REQUIRE(d.output.y == p.OH && d.output.x == p.OW, CLDNN_HIP_DIMENSION_MISMATCH,
                 "output spatial size differs from the computed one");
    p.in_dt = d.input.dtype, p.w_dt = d.weights_dtype, p.out_dt = d.output.dtype;
    p.eltw_dt = d.fused ? d.eltw.dtype : CLDNN_HIP_NO_TYPE;
    p.in_t = d.input, p.out_t = d.output;
    p.in_p = make_pitch(d.input), p.out_p = make_pitch(d.output);
    p.esy = d.fused ? (d.eltw_stride_y > 0 ? d.eltw_stride_y : 1) : 1;
    p.esx = d.fused ? (d.eltw_stride_x > 0 ? d.eltw_stride_x : 1) : 1;
    if (d.fused) {
        if (d.second_input_in_output) {
            p.eltw_t = d.output;
            p.eltw_dt = d.output.dtype;
        } else {
            p.eltw_t = d.eltw;
        }
        p.eltw_p = make_pitch(p.eltw_t);
        CHIP_REQUIRE(p.eltw_t.f == p.OFM && p.eltw_t.b == p.B && p.eltw_t.y >= (p.OH - 1) * p.esy + 1
                         && p.eltw_t.x >= (p.OW - 1) * p.esx + 1,
                     CLDNN_HIP_DIMENSION_MISMATCH, "second input of fused_conv_eltwise does not cover the output");
    }

    // ---- data-type legality (reference convolution_kernel_ref.cpp:124-166, fused ..._kernel_ref.cpp:21-47)
    const bool in8 = is_int8(p.in_dt);
    CHIP_REQUIRE(in8 || p.in_dt == CLDNN_HIP_F32, CLDNN_HIP_INVALID_ARG, "input must be s8, u8 or f32");
    CHIP_REQUIRE(is_int8(p.out_dt) || p.out_dt == CLDNN_HIP_F32, CLDNN_HIP_INVALID_ARG, "output must be s8, u8 or f32");
    if (in8) CHIP_REQUIRE(p.w_dt == CLDNN_HIP_S8, CLDNN_HIP_INVALID_ARG, "int8 activations need s8 weights");
    else CHIP_REQUIRE(p.w_dt == CLDNN_HIP_F32, CLDNN_HIP_INVALID_ARG, "f32 activations need f32 weights");

    // ---- arithmetic mode (reference fused_conv_eltwise_gpu_ref.cl:18-48 and the flags the host emits)
    Epilogue& e = c->epi;
    if (d.fused) {
        if (d.has_wqf) e.mode = MODE_Q;
        else if (in8 || is_int8(p.out_dt) || is_int8(p.eltw_dt)) e.mode = MODE_FINT;
        else e.mode = MODE_NAT;
    } else {
        e.mode = (d.has_wqf || d.has_calib || d.output_quantization_factor != 1.0f) ? MODE_Q : MODE_NAT;
    }
    if (e.mode == MODE_NAT && in8)
        CHIP_REQUIRE(p.in_dt == CLDNN_HIP_S8 && p.out_dt == CLDNN_HIP_S8, CLDNN_HIP_INVALID_ARG,
                     "u8 data and precision changes need weights_quantization_factors");
    const bool calib_on = d.fused ? (d.has_wqf && d.has_calib) : (d.has_calib != 0);
    e.bias_dt = d.bias_dtype;
    e.bias_after = (!d.fused && d.has_wqf && bias && d.bias_dtype == CLDNN_HIP_F32) ? 1 : 0;
    e.oqf_on = d.fused ? 1 : (d.output_quantization_factor != 1.0f);
    e.iqf = d.input_quantization_factor, e.oqf = d.output_quantization_factor;
    e.act = d.activation, e.act_m = d.activation_m, e.act_n = d.activation_n;
    e.fused = d.fused ? 1 : 0;
    e.ncs = d.non_conv_scale, e.ncs_on = d.fused && d.non_conv_scale != 1.0f;
    e.eltw_act = d.eltw_activation, e.eltw_m = d.eltw_activation_m, e.eltw_n = d.eltw_activation_n;
    e.out_dt = p.out_dt, e.eltw_dt = p.eltw_dt, e.in_dt = p.in_dt;
    e.round_even = d.round_to_even;
    e.fc = (d.fully_connected && d.has_wqf && !d.fused) ? 1 : 0;
    CHIP_REQUIRE(d.conv_saturate >= 0 && d.conv_saturate <= 2 && (!d.conv_saturate || (d.fused && d.has_wqf)), CLDNN_HIP_INVALID_ARG,
                 "conv_saturate is 0, 1 (s8) or 2 (u8) and goes with the quantized fused form");
    e.conv_sat = d.conv_saturate;
    if (d.sibling_split) {
        CHIP_REQUIRE(d.sibling_split > 0 && d.sibling_split < d.ofm && d.sibling_split % 16 == 0, CLDNN_HIP_INVALID_ARG,
                     "sibling_split is a multiple of 16 inside (0, ofm)");
        CHIP_REQUIRE(d.groups == 1 && d.has_wqf && !d.fused && !d.fully_connected, CLDNN_HIP_UNSUPPORTED_FORMAT,
                     "two convolutions in one launch: one group, the quantized form, no fused second input");
        // one convolution as far as the arithmetic goes when both sides take the same activation
        const bool same = d.sibling_activation == d.activation
                          && (d.activation == CLDNN_HIP_ACT_NONE || d.activation == CLDNN_HIP_ACT_RELU
                              || (d.sibling_activation_m == d.activation_m && d.sibling_activation_n == d.activation_n));
        if (!same) e.split_f = d.sibling_split, e.act2 = d.sibling_activation, e.act2_m = d.sibling_activation_m, e.act2_n = d.sibling_activation_n;
    }
    if (e.fc) {
        CHIP_REQUIRE(p.OH == 1 && p.OW == 1 && p.FY == p.IH && p.FX == p.IW && p.py == 0 && p.px == 0, CLDNN_HIP_INVALID_ARG,
                     "fully_connected: the filter must cover the whole input plane");
        CHIP_REQUIRE(p.out_dt == CLDNN_HIP_S8, CLDNN_HIP_INVALID_ARG, "quantized fully_connected writes s8");
    }

    // ---- kernel family
    const bool blocked = d.input.format == CLDNN_HIP_FMT_FS_B_YX_FSV16 && d.output.format == CLDNN_HIP_FMT_FS_B_YX_FSV16
                         && (!d.fused || p.eltw_t.format == CLDNN_HIP_FMT_FS_B_YX_FSV16);
    const bool int_path = in8 && p.w_dt == CLDNN_HIP_S8 && e.mode != MODE_NAT;
    const bool depthwise = d.groups > 1 && d.groups == d.ifm && d.groups == d.ofm;
    // first layers: at most 4 input features in b_fs_yx_fsv4 (4 horizontal taps x 4 features = one 16-byte fragment)
    const bool stem = d.input.format == CLDNN_HIP_FMT_B_FS_YX_FSV4 && d.output.format == CLDNN_HIP_FMT_FS_B_YX_FSV16
                      && (!d.fused || p.eltw_t.format == CLDNN_HIP_FMT_FS_B_YX_FSV16) && d.ifm <= 4 && d.groups == 1
                      && d.dilation_x == 1 && conv_border_covers(p) && (p.FY * ((p.FX + 3) / 4) + 3) / 4 <= 8;
    // Grouped (not depthwise) convolutions run on the same matrix-core kernels as one dense convolution whose weight
    // matrix is block-diagonal: feature f only has weights for the input features of its own group, the rest are zero.
    // That is the arithmetic of the reference's per-group launches (fused_conv_eltwise_gpu_ref.cl:108-112,134-136) in one
    // launch; the zero blocks cost matrix-core time that these layers do not miss (they are bound by launch and memory),
    // and dense weights of more than 64 MiB stay on the one-thread-per-output kernel.
    const bool grouped = d.groups > 1 && !depthwise;
    const bool grouped_dense = grouped && blocked && (size_t)d.ofm * d.ifm * d.fy * d.fx <= ((size_t)64 << 20);
    int impl = d.impl;
    if (impl == CLDNN_HIP_IMPL_AUTO) {
        if ((blocked || stem) && int_path && (d.groups == 1 || grouped_dense)) impl = CLDNN_HIP_IMPL_MFMA;
        else if (blocked && int_path && depthwise) impl = CLDNN_HIP_IMPL_DEPTHWISE;
        else impl = CLDNN_HIP_IMPL_REF;
    }
    if (impl == CLDNN_HIP_IMPL_MFMA)
        CHIP_REQUIRE((blocked || stem) && int_path && (d.groups == 1 || grouped_dense), CLDNN_HIP_UNSUPPORTED_FORMAT,
                     "the MFMA kernel needs int8 data in fs_b_yx_fsv16 (first layers: bordered b_fs_yx_fsv4 input), "
                     "quantisation, and groups == 1 or a block-diagonal weight matrix of at most 64 MiB");
    if (impl == CLDNN_HIP_IMPL_DEPTHWISE)
        CHIP_REQUIRE(blocked && int_path && depthwise, CLDNN_HIP_UNSUPPORTED_FORMAT,
                     "the depthwise kernel needs int8 data in fs_b_yx_fsv16, quantisation and groups == features");
    c->impl = impl;

    const int ifm_g = p.IFM / p.groups;
    const size_t wcount = (size_t)p.OFM * ifm_g * p.FY * p.FX;
    c->engine->make_current();

    // per-feature vectors, zero padded so that vector loads of a partly filled tile stay in bounds
    const size_t ofm_pad = ((size_t)p.OFM + 255) / 256 * 256;
    if (wqf) c->wqf = upload(c, wqf, p.OFM * 4, ofm_pad * 4);
    if (calib && calib_on) c->calib = upload(c, calib, p.OFM * 4, ofm_pad * 4);
    if (eltw_calib) c->ecal = upload(c, eltw_calib, p.OFM * 4, ofm_pad * 4);
    e.wqf = (const float*)c->wqf, e.calib = (const float*)c->calib, e.eltw_calib = (const float*)c->ecal;

    cldnn_hip_conv_info& inf = c->info;
    inf.impl = impl;
    inf.tile_index = -1;
    inf.ops = 2ll * p.B * p.OH * p.OW * p.OFM * ifm_g * p.FY * p.FX;
    inf.bytes = (int64_t)p.B * p.IH * p.IW * p.IFM * (int64_t)dtype_size(p.in_dt)
                + (int64_t)p.B * p.OH * p.OW * p.OFM * (int64_t)dtype_size(p.out_dt)
                + (int64_t)wcount * (int64_t)dtype_size(p.w_dt)
                + 4ll * p.OFM * ((bias ? 1 : 0) + (wqf ? 1 : 0) + (calib ? 1 : 0) + (eltw_calib ? 1 : 0))
                + (d.fused ? (int64_t)p.B * p.OH * p.OW * p.OFM * (int64_t)dtype_size(p.eltw_dt) : 0);

    if (impl == CLDNN_HIP_IMPL_REF) {
        c->w_raw = upload(c, weights, wcount * dtype_size(p.w_dt));
        if (bias) c->bias = upload(c, bias, p.OFM * 4, ofm_pad * 4);
        e.bias = c->bias;
        inf.block = 256;
        inf.grid = (int)(((int64_t)p.B * p.OFM * p.OH * p.OW + 255) / 256);
        std::snprintf(inf.kernel_name, sizeof(inf.kernel_name), "conv_ref_kernel");
        return;
    }

    // ---- accumulator start values: 128*sum(w) for u8 on the signed matrix cores, plus an int32 bias
    const int8_t* w8 = (const int8_t*)weights;
    std::vector<int32_t> init(ofm_pad, 0), init_raw(ofm_pad, 0);
    // can the short epilogue reproduce the long one?  (an int32 bias is folded into the start values, a float one is not)
    {
        Epilogue probe = e;
        probe.bias = bias && (d.bias_dtype == CLDNN_HIP_F32 || e.fc) ? (const void*)weights : nullptr;
        c->fast = mfma_fast_epilogue(p, probe, calib_on ? calib : nullptr, eltw_calib, wqf, &c->fe);
    }
    if (impl == CLDNN_HIP_IMPL_DEPTHWISE && e.fc) c->fast = false;  // the depthwise kernels have no short fully_connected form
    const bool dw_fast = impl == CLDNN_HIP_IMPL_DEPTHWISE && dw_fast_applies(p, c->fast);
    const bool xor_u8 = (impl == CLDNN_HIP_IMPL_MFMA || dw_fast) && p.in_dt == CLDNN_HIP_U8;
    for (int f = 0; f < p.OFM; ++f) {
        int64_t s = 0;
        if (xor_u8)
            for (size_t i = 0; i < (size_t)ifm_g * p.FY * p.FX; ++i) s += w8[(size_t)f * ifm_g * p.FY * p.FX + i];
        uint32_t v = (uint32_t)(int32_t)(128 * s);
        init_raw[f] = impl == CLDNN_HIP_IMPL_MFMA ? (int32_t)v : 0;  // the accumulator probe of the depthwise path never flips signs
        // (the fully_connected form adds its bias as a float after the dequantisation, whatever its type)
        if (bias && d.bias_dtype == CLDNN_HIP_I32 && !e.bias_after && !e.fc) v += (uint32_t)((const int32_t*)bias)[f];
        init[f] = (int32_t)v;
    }
    c->acc_init = upload(c, init.data(), ofm_pad * 4);
    c->acc_init_raw = upload(c, init_raw.data(), ofm_pad * 4);
    if (bias && (d.bias_dtype == CLDNN_HIP_F32 || e.fc)) {
        c->bias = upload(c, bias, p.OFM * 4, ofm_pad * 4);
        e.bias = c->bias;
    } else {
        e.bias = nullptr;  // folded into acc_init
        e.bias_dt = CLDNN_HIP_NO_TYPE;
    }

    std::vector<int8_t> dense;
    if (impl == CLDNN_HIP_IMPL_MFMA && grouped) {
        // [ofm][ifm / groups][fy][fx] -> block-diagonal [ofm][ifm][fy][fx]
        const size_t taps = (size_t)p.FY * p.FX, ofm_g = (size_t)p.OFM / p.groups;
        dense.assign((size_t)p.OFM * p.IFM * taps, 0);
        for (int f = 0; f < p.OFM; ++f) {
            const size_t g = (size_t)f / ofm_g;
            std::memcpy(&dense[((size_t)f * p.IFM + g * ifm_g) * taps], w8 + (size_t)f * ifm_g * taps, (size_t)ifm_g * taps);
        }
        w8 = dense.data();
        p.groups = 1;  // from here on the problem is the dense one (the algorithmic work above counts the real weights)
    }
    if (impl == CLDNN_HIP_IMPL_MFMA) {
        int tile = d.tile_override > 0 ? d.tile_override - 1 : mfma_choose(p, c->engine->props.multiProcessorCount);
        CHIP_REQUIRE(tile >= 0 && tile < tile_config_count(), CLDNN_HIP_INVALID_ARG, "tile_override out of range");
        c->mplan = mfma_plan(p, tile, c->engine->props.multiProcessorCount);
        std::vector<int8_t> packed(c->mplan.packed_bytes);
        std::vector<int32_t> ktab(c->mplan.ktab_bytes / sizeof(int32_t));
        mfma_pack_weights(p, c->mplan, w8, packed.data(), ktab.data());
        c->w_packed = upload(c, packed.data(), packed.size());
        c->ktab = upload(c, ktab.data(), ktab.size() * 4);
        if (const size_t g = mfma_gather_bytes(p, c->mplan)) c->gather = upload(c, nullptr, 0, g);
        const TileConfig& tc = tile_config(tile);
        inf.tile_index = tile, inf.tile_pixels = tc.tile_pixels, inf.tile_ofm = tc.tile_ofm;
        inf.grid = c->mplan.grid, inf.block = c->mplan.gemv ? 64 * c->mplan.gemv_waves : c->mplan.block, inf.lds_bytes = c->mplan.lds_bytes;
        std::snprintf(inf.kernel_name, sizeof(inf.kernel_name), "conv_%s<%s,%s,%s>", c->mplan.gemv ? "gemv" : c->mplan.halo ? "halo" : c->mplan.stream ? "stream" : (c->mplan.bdir ? "bdir" : (c->mplan.wsl ? "wsl" : "mfma")),
                      tc.name, c->mplan.checked ? "checked" : "border", c->fast && !c->mplan.gemv ? "fast" : "generic");
    } else {
        c->dplan = dw_plan(p);
        std::vector<int8_t> packed(c->dplan.packed_bytes);
        dw_pack_weights(p, w8, packed.data());
        c->w_packed = upload(c, packed.data(), packed.size());
        if (dw_fast) {
            std::vector<int32_t> masked(c->dplan.mask_bytes / 4);
            dw_mask_weights(p, w8, masked.data());
            c->w_masked = upload(c, masked.data(), c->dplan.mask_bytes);
        }
        inf.grid = c->dplan.grid * ((p.OFM + 15) / 16), inf.block = c->dplan.block, inf.lds_bytes = dw_fast ? 0 : p.FY * p.FX * 16;
        std::snprintf(inf.kernel_name, sizeof(inf.kernel_name), "%s<%s>", dw_fast ? "conv_dw3x3_kernel" : "conv_dw_kernel",
                      p.in_dt == CLDNN_HIP_U8 ? "u8" : "s8");
    }
}

}  // namespace

extern "C" {

int32_t cldnn_hip_conv_out_extent(int32_t in, int32_t pad, int32_t filt, int32_t dil, int32_t stride)
{
    return out_extent(in, pad, filt, dil, stride);
}

int32_t cldnn_hip_tile_config_count(void) { return tile_config_count(); }
const char* cldnn_hip_tile_config_name(int32_t i)
{
    return (i >= 0 && i < tile_config_count()) ? tile_config(i).name : nullptr;
}

cldnn_hip_status cldnn_hip_conv_create(cldnn_hip_engine e, const cldnn_hip_conv_desc* desc, const void* weights,
                                       const void* bias, const float* wqf, const float* calib,
                                       const float* eltw_calib, cldnn_hip_conv* out)
{
    return guarded([&] {
        CHIP_REQUIRE(e && desc && out, CLDNN_HIP_INVALID_ARG, "null argument");
        *out = nullptr;
        auto* c = new cldnn_hip_conv_s();
        c->engine = e;
        c->desc = *desc;
        e->refs.fetch_add(1);
        try {
            build(c, weights, bias, wqf, calib, eltw_calib);
        } catch (...) {
            cldnn_hip_conv_release(c);
            throw;
        }
        *out = c;
    });
}

cldnn_hip_status cldnn_hip_conv_release(cldnn_hip_conv c)
{
    return guarded([&] {
        CHIP_REQUIRE(c, CLDNN_HIP_INVALID_ARG, "null convolution");
        cldnn_hip_engine e = c->engine;
        (void)hipSetDevice(e->device);
        (void)hipStreamSynchronize(e->stream);
        for (void* d : c->owned) (void)hipFree(d);
        delete c;
        cldnn_hip_engine_release(e);
    });
}

static void run(cldnn_hip_conv c, const void* in, void* out, const void* eltw, int32_t* raw, bool static_scratch = false)
{
    CHIP_REQUIRE(c && in && (out || raw), CLDNN_HIP_INVALID_ARG, "null argument");
    const ConvProblem& p = c->p;
    if (c->desc.fused && !raw) {
        if (c->desc.second_input_in_output) eltw = out;
        CHIP_REQUIRE(eltw, CLDNN_HIP_INVALID_ARG, "fused convolution without its second input");
    }
    c->engine->make_current();
    hipStream_t s = c->engine->stream;
    switch (c->impl) {
    case CLDNN_HIP_IMPL_REF:
        launch_conv_ref(s, p, c->epi, in, c->w_raw, eltw, out, raw);
        break;
    case CLDNN_HIP_IMPL_MFMA: {
        MfmaBuffers wb{(const int8_t*)c->w_packed, (const int32_t*)c->ktab, c->gather};
        if (static_scratch) {
            // the gather scratch comes from the array inside the code object instead of the object's own allocation
            const size_t need = mfma_gather_bytes(p, c->mplan);
            CHIP_REQUIRE(need <= mfma_static_scratch_bytes(), CLDNN_HIP_UNSUPPORTED_SIZE,
                         "this convolution gathers " + std::to_string(need) + " bytes of activations, the static scratch holds "
                             + std::to_string(mfma_static_scratch_bytes()));
            if (need) wb.gather = c->engine->static_scratch;
        }
        if (raw)
            launch_conv_mfma(s, p, c->mplan, wb, (const int32_t*)c->acc_init_raw, c->epi, nullptr, in, nullptr, nullptr, raw);
        else
            launch_conv_mfma(s, p, c->mplan, wb, (const int32_t*)c->acc_init, c->epi, c->fast ? &c->fe : nullptr, in, eltw,
                             out, nullptr);
        break;
    }
    case CLDNN_HIP_IMPL_DEPTHWISE:
        launch_conv_dw(s, p, c->dplan, (const int8_t*)c->w_packed, (const int32_t*)c->w_masked,
                       (const int32_t*)(raw ? c->acc_init_raw : c->acc_init), c->epi, c->fast ? &c->fe : nullptr, in, eltw, out,
                       raw);
        break;
    default: throw error(CLDNN_HIP_ERROR, "convolution without an implementation");
    }
}

cldnn_hip_status cldnn_hip_conv_enqueue(cldnn_hip_conv c, const void* input_dev, void* output_dev, const void* eltw_dev)
{
    return guarded([&] { run(c, input_dev, output_dev, eltw_dev, nullptr); });
}

cldnn_hip_status cldnn_hip_conv_enqueue_static_scratch(cldnn_hip_conv c, const void* input_dev, void* output_dev,
                                                       const void* eltw_dev)
{
    return guarded([&] { run(c, input_dev, output_dev, eltw_dev, nullptr, true); });
}

cldnn_hip_status cldnn_hip_conv_chain_create(cldnn_hip_engine e, int32_t count, const cldnn_hip_conv_desc* descs,
                                             const void* const* weights, const void* const* bias, const float* const* wqf,
                                             const float* const* calib, const float* const* eltw_calib,
                                             const int32_t* keep_output, cldnn_hip_conv_chain* out)
{
    return guarded([&] {
        CHIP_REQUIRE(e && descs && weights && out, CLDNN_HIP_INVALID_ARG, "null argument");
        CHIP_REQUIRE(count >= 2 && count <= 3, CLDNN_HIP_INVALID_ARG, "a chain has two or three convolutions");
        *out = nullptr;
        auto* ch = new cldnn_hip_conv_chain_s();
        ch->engine = e;
        ch->count = count;
        e->refs.fetch_add(1);
        try {
            for (int k = 0; k < count; ++k) {
                // every stage is an ordinary convolution object: validation, arithmetic mode, per-feature vectors and the
                // accumulator start values come from there
                cldnn_hip_conv c = nullptr;
                const cldnn_hip_status st = cldnn_hip_conv_create(e, &descs[k], weights[k], bias ? bias[k] : nullptr, wqf ? wqf[k] : nullptr,
                                                                  calib ? calib[k] : nullptr, eltw_calib ? eltw_calib[k] : nullptr, &c);
                if (st != CLDNN_HIP_SUCCESS) throw error(st, std::string("stage ") + std::to_string(k) + ": " + cldnn_hip_last_error());
                ch->stage[k] = c;
                const bool dw_head = k == 0 && c->impl == CLDNN_HIP_IMPL_DEPTHWISE && c->w_masked;
                CHIP_REQUIRE(c->impl == CLDNN_HIP_IMPL_MFMA || dw_head, CLDNN_HIP_UNSUPPORTED_FORMAT,
                             "stage " + std::to_string(k) + " of a chain must be a dense int8 convolution in fs_b_yx_fsv16 (the first "
                             "stage may be a depthwise 3x3)");
                CHIP_REQUIRE(!descs[k].second_input_in_output, CLDNN_HIP_UNSUPPORTED_FORMAT, "a chained stage cannot read its residual from its own output");
                CHIP_REQUIRE(!descs[k].sibling_split, CLDNN_HIP_UNSUPPORTED_FORMAT, "a chained stage cannot be two convolutions in one");
                CHIP_REQUIRE(descs[k].groups == 1 || dw_head, CLDNN_HIP_UNSUPPORTED_FORMAT, "a chained stage cannot be a grouped convolution");
                ch->keep[k] = keep_output ? (keep_output[k] != 0) : 1;
                ch->in[k] = ChainStageIn{&c->p, &c->epi, &c->fe, c->fast, (const int32_t*)c->acc_init,
                                         dw_head ? (const int32_t*)c->w_masked : nullptr};
            }
            CHIP_REQUIRE(ch->keep[count - 1], CLDNN_HIP_INVALID_ARG, "the last stage of a chain always writes its output");
            const int cus = e->props.multiProcessorCount;
            const std::string why = chain_plan(ch->in, count, cus, &ch->plan);
            if (!why.empty()) throw error(CLDNN_HIP_UNSUPPORTED_FORMAT, "these convolutions cannot run as one chain: " + why);
            std::vector<int8_t> packed(chain_packed_bytes(ch->plan));
            const int8_t* w8[3] = {nullptr, nullptr, nullptr};
            for (int k = 0; k < count; ++k) w8[k] = (const int8_t*)weights[k];
            // the accumulator start values exist on the device only (the stage objects folded offset correction and bias)
            e->make_current();
            std::vector<std::vector<int32_t>> init(count);
            ChainVectors vec[3]{};
            for (int k = 0; k < count; ++k) {
                init[k].resize(descs[k].ofm);
                CHIP_CHECK(hipMemcpy(init[k].data(), ch->stage[k]->acc_init, (size_t)descs[k].ofm * 4, hipMemcpyDeviceToHost));
                const bool calib_on = ch->stage[k]->epi.calib != nullptr;
                vec[k] = ChainVectors{init[k].data(), calib_on && calib ? calib[k] : nullptr, eltw_calib ? eltw_calib[k] : nullptr,
                                      wqf ? wqf[k] : nullptr};
            }
            chain_pack_weights(ch->in, ch->plan, cus, w8, vec, packed.data());
            // The chain launches none of its stage objects (they never leave this file): their own operand streams (packed weights, tap table, gather
            // scratch) would only hold every chained layer's weights on the device a second time.
            for (int k = 0; k < count; ++k) {
                cldnn_hip_conv c = ch->stage[k];
                for (void** buf : {&c->w_packed, &c->ktab, &c->gather}) {
                    if (!*buf) continue;
                    c->owned.erase(std::remove(c->owned.begin(), c->owned.end(), *buf), c->owned.end());
                    CHIP_CHECK(hipFree(*buf));
                    *buf = nullptr;
                }
            }
            CHIP_CHECK(hipMalloc(&ch->packed, packed.size()));
            CHIP_CHECK(hipMemcpyAsync(ch->packed, packed.data(), packed.size(), hipMemcpyHostToDevice, e->stream));
            CHIP_CHECK(hipStreamSynchronize(e->stream));
            cldnn_hip_conv_info& inf = ch->info;
            inf.impl = CLDNN_HIP_IMPL_MFMA, inf.tile_index = -1, inf.tile_pixels = 64 * (ch->plan.dw ? 4 : ch->plan.nt), inf.tile_ofm = 64;
            inf.grid = ch->plan.grid, inf.block = 256, inf.lds_bytes = ch->plan.lds_bytes;
            std::snprintf(inf.kernel_name, sizeof(inf.kernel_name), "%s", ch->plan.name);
            // algorithmic work of the chain: every stage's operations; bytes of what has to cross the memory interface,
            // i.e. without the intermediate tensors that are neither kept nor re-read
            for (int k = 0; k < count; ++k) {
                const cldnn_hip_conv_info& si = ch->stage[k]->info;
                const ConvProblem& p = ch->stage[k]->p;
                inf.ops += si.ops;
                int64_t bytes = si.bytes;
                if (k > 0) bytes -= (int64_t)p.B * p.IH * p.IW * p.IFM;                  // input comes from registers
                if (!ch->keep[k]) bytes -= (int64_t)p.B * p.OH * p.OW * p.OFM;           // output stays in registers
                inf.bytes += bytes;
            }
        } catch (...) {
            cldnn_hip_conv_chain_release(ch);
            throw;
        }
        *out = ch;
    });
}

cldnn_hip_status cldnn_hip_conv_chain_release(cldnn_hip_conv_chain ch)
{
    return guarded([&] {
        CHIP_REQUIRE(ch, CLDNN_HIP_INVALID_ARG, "null chain");
        cldnn_hip_engine e = ch->engine;
        (void)hipSetDevice(e->device);
        (void)hipStreamSynchronize(e->stream);
        if (ch->packed) (void)hipFree(ch->packed);
        for (int k = 0; k < 3; ++k)
            if (ch->stage[k]) cldnn_hip_conv_release(ch->stage[k]);
        delete ch;
        cldnn_hip_engine_release(e);
    });
}

cldnn_hip_status cldnn_hip_conv_chain_enqueue(cldnn_hip_conv_chain ch, const void* input_dev, void* const* outputs_dev,
                                              const void* const* eltw_dev)
{
    return guarded([&] {
        CHIP_REQUIRE(ch && input_dev && outputs_dev, CLDNN_HIP_INVALID_ARG, "null argument");
        void* outs[3] = {nullptr, nullptr, nullptr};
        const void* el[3] = {nullptr, nullptr, nullptr};
        for (int k = 0; k < ch->count; ++k) {
            if (ch->keep[k]) {
                CHIP_REQUIRE(outputs_dev[k], CLDNN_HIP_INVALID_ARG, "a kept stage of the chain has no output buffer");
                outs[k] = outputs_dev[k];
            }
            if (ch->stage[k]->desc.fused) {
                CHIP_REQUIRE(eltw_dev && eltw_dev[k], CLDNN_HIP_INVALID_ARG, "fused stage of a chain without its second input");
                el[k] = eltw_dev[k];
            }
        }
        ch->engine->make_current();
        launch_conv_chain(ch->engine->stream, ch->in, ch->plan, ch->packed, input_dev, outs, el);
    });
}

cldnn_hip_status cldnn_hip_conv_chain_get_info(cldnn_hip_conv_chain ch, cldnn_hip_conv_info* info)
{
    return guarded([&] {
        CHIP_REQUIRE(ch && info, CLDNN_HIP_INVALID_ARG, "null argument");
        *info = ch->info;
    });
}

// One candidate of the tuner: microseconds per launch, or a negative value when the row refuses the convolution.
static float time_candidate(cldnn_hip_engine e, cldnn_hip_conv_desc d, int tile_override, const void* weights, const void* bias,
                            const float* wqf, const float* calib, const float* eltw_calib, const void* in, void* out,
                            const void* eltw, int runs)
{
    d.tile_override = tile_override;
    cldnn_hip_conv c = nullptr;
    if (cldnn_hip_conv_create(e, &d, weights, bias, wqf, calib, eltw_calib, &c) != CLDNN_HIP_SUCCESS) return -1.0f;
    if (tile_override && c->impl != CLDNN_HIP_IMPL_MFMA) {
        cldnn_hip_conv_release(c);
        return -1.0f;
    }
    float best = -1.0f;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    try {
        CHIP_CHECK(hipEventCreate(&t0));
        CHIP_CHECK(hipEventCreate(&t1));
        // creating the candidate left the device idle for a while: bring its clocks back up before timing
        const auto start = std::chrono::steady_clock::now();
        do {
            for (int i = 0; i < 10; ++i) run(c, in, out, eltw, nullptr);
            CHIP_CHECK(hipStreamSynchronize(e->stream));
        } while (std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - start).count() < 20.0);
        for (int batch = 0; batch < 3; ++batch) {
            CHIP_CHECK(hipEventRecord(t0, e->stream));
            for (int i = 0; i < runs; ++i) run(c, in, out, eltw, nullptr);
            CHIP_CHECK(hipEventRecord(t1, e->stream));
            CHIP_CHECK(hipEventSynchronize(t1));
            float ms = 0.0f;
            CHIP_CHECK(hipEventElapsedTime(&ms, t0, t1));
            const float us = ms * 1000.0f / (float)runs;
            if (best < 0.0f || us < best) best = us;
        }
    } catch (...) {
        if (t0) (void)hipEventDestroy(t0);
        if (t1) (void)hipEventDestroy(t1);
        cldnn_hip_conv_release(c);
        throw;
    }
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    cldnn_hip_conv_release(c);
    return best;
}

static void warm_device(cldnn_hip_engine e, const cldnn_hip_conv_desc& d, const void* weights, const void* bias, const float* wqf,
                        const float* calib, const float* eltw_calib, const void* in, void* out, const void* eltw, double milliseconds)
{
    cldnn_hip_conv c = nullptr;
    if (cldnn_hip_conv_create(e, &d, weights, bias, wqf, calib, eltw_calib, &c) != CLDNN_HIP_SUCCESS) return;
    try {
        const auto start = std::chrono::steady_clock::now();
        do {
            for (int i = 0; i < 20; ++i) run(c, in, out, eltw, nullptr);
            CHIP_CHECK(hipStreamSynchronize(e->stream));
        } while (std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - start).count() < milliseconds);
    } catch (...) {
        cldnn_hip_conv_release(c);
        throw;
    }
    cldnn_hip_conv_release(c);
}

cldnn_hip_status cldnn_hip_conv_tune(cldnn_hip_engine e, const cldnn_hip_conv_desc* desc, const void* weights, const void* bias,
                                     const float* wqf, const float* calib, const float* eltw_calib, int32_t runs,
                                     int32_t* best_tile_index, float* best_us, float* default_us, float* row_us)
{
    return guarded([&] {
        CHIP_REQUIRE(e && desc && weights && best_tile_index && best_us, CLDNN_HIP_INVALID_ARG, "null argument");
        CHIP_REQUIRE(runs >= 1 && runs <= 10000, CLDNN_HIP_INVALID_ARG, "tuning runs must be between 1 and 10000");
        e->make_current();
        const size_t in_bytes = tensor_elems(desc->input) * dtype_size(desc->input.dtype);
        const size_t out_bytes = tensor_elems(desc->output) * dtype_size(desc->output.dtype);
        const bool separate_eltw = desc->fused && !desc->second_input_in_output;
        const size_t el_bytes = separate_eltw ? tensor_elems(desc->eltw) * dtype_size(desc->eltw.dtype) : 0;
        void *in = nullptr, *out = nullptr, *eltw = nullptr;
        auto release = [&] {
            (void)hipStreamSynchronize(e->stream);
            if (in) (void)hipFree(in);
            if (out) (void)hipFree(out);
            if (eltw) (void)hipFree(eltw);
        };
        try {
            CHIP_CHECK(hipMalloc(&in, in_bytes ? in_bytes : 1));
            CHIP_CHECK(hipMalloc(&out, out_bytes ? out_bytes : 1));
            if (separate_eltw) CHIP_CHECK(hipMalloc(&eltw, el_bytes ? el_bytes : 1));
            // pseudo-random bytes; a float tensor gets small integers so that no NaN patterns are timed
            std::vector<uint8_t> host(std::max(in_bytes, el_bytes));
            uint32_t state = 1337u;
            for (auto& b : host) {
                state = state * 1664525u + 1013904223u;
                b = (uint8_t)(state >> 24);
            }
            if (desc->input.dtype == CLDNN_HIP_F32)
                for (size_t i = 0; i + 4 <= in_bytes; i += 4) {
                    const float v = (float)(int8_t)host[i];
                    std::memcpy(&host[i], &v, 4);
                }
            CHIP_CHECK(hipMemcpy(in, host.data(), in_bytes, hipMemcpyHostToDevice));
            if (separate_eltw) CHIP_CHECK(hipMemcpy(eltw, host.data(), el_bytes, hipMemcpyHostToDevice));
            CHIP_CHECK(hipMemset(out, 0, out_bytes));
            // the clocks of an idle device rise over tens of milliseconds: keep it busy first, or the candidates timed
            // first (the table's own choice among them) lose against the later ones
            warm_device(e, *desc, weights, bias, wqf, calib, eltw_calib, in, out, eltw, 150.0);
            const float base = time_candidate(e, *desc, 0, weights, bias, wqf, calib, eltw_calib, in, out, eltw, runs);
            CHIP_REQUIRE(base >= 0.0f, CLDNN_HIP_ERROR, std::string("the convolution cannot be created: ") + cldnn_hip_last_error());
            *best_tile_index = -1, *best_us = base;
            if (default_us) *default_us = base;
            const int rows = cldnn_hip_tile_config_count();
            for (int r = 0; r < rows; ++r) {
                const float us = desc->impl == CLDNN_HIP_IMPL_AUTO || desc->impl == CLDNN_HIP_IMPL_MFMA
                                     ? time_candidate(e, *desc, r + 1, weights, bias, wqf, calib, eltw_calib, in, out, eltw, runs)
                                     : -1.0f;
                if (row_us) row_us[r] = us;
                // a row has to win by more than the noise of the measurement to replace the table's choice
                if (us >= 0.0f && us < *best_us * 0.98f) *best_us = us, *best_tile_index = r;
            }
        } catch (...) {
            release();
            throw;
        }
        release();
    });
}

cldnn_hip_status cldnn_hip_conv_accumulators(cldnn_hip_conv c, const void* input_dev, int32_t* acc_dev)
{
    return guarded([&] {
        CHIP_REQUIRE(acc_dev, CLDNN_HIP_INVALID_ARG, "null accumulator buffer");
        CHIP_REQUIRE(c && c->epi.mode != MODE_NAT, CLDNN_HIP_INVALID_ARG, "accumulators exist in the integer modes only");
        run(c, input_dev, nullptr, nullptr, acc_dev);
    });
}

cldnn_hip_status cldnn_hip_conv_get_info(cldnn_hip_conv c, cldnn_hip_conv_info* info)
{
    return guarded([&] {
        CHIP_REQUIRE(c && info, CLDNN_HIP_INVALID_ARG, "null argument");
        *info = c->info;
    });
}

cldnn_hip_status cldnn_hip_reorder(cldnn_hip_engine e, const void* src_dev, const cldnn_hip_tensor* src, void* dst_dev,
                                   const cldnn_hip_tensor* dst)
{
    return guarded([&] {
        CHIP_REQUIRE(e && src_dev && src && dst_dev && dst, CLDNN_HIP_INVALID_ARG, "null argument");
        e->make_current();
        launch_reorder(e->stream, *src, src_dev, *dst, dst_dev);
    });
}

cldnn_hip_status cldnn_hip_copy_region(cldnn_hip_engine e, const void* src_dev, const cldnn_hip_tensor* src, void* dst_dev,
                                       const cldnn_hip_tensor* dst, int32_t offset_b, int32_t offset_f, int32_t offset_y, int32_t offset_x)
{
    return guarded([&] {
        CHIP_REQUIRE(e && src_dev && src && dst_dev && dst, CLDNN_HIP_INVALID_ARG, "null argument");
        e->make_current();
        launch_copy_region(e->stream, *src, src_dev, *dst, dst_dev, offset_b, offset_f, offset_y, offset_x);
    });
}

cldnn_hip_status cldnn_hip_activation(cldnn_hip_engine e, const void* src_dev, const cldnn_hip_tensor* src, void* dst_dev,
                                      const cldnn_hip_tensor* dst, int32_t activation, float m, float n)
{
    return guarded([&] {
        CHIP_REQUIRE(e && src_dev && src && dst_dev && dst, CLDNN_HIP_INVALID_ARG, "null argument");
        e->make_current();
        launch_pointwise(e->stream, *src, src_dev, nullptr, nullptr, *dst, dst_dev, 0, nullptr, 1.0f, activation, m, n);
    });
}

cldnn_hip_status cldnn_hip_eltwise_sum(cldnn_hip_engine e, const void* a_dev, const cldnn_hip_tensor* a, const void* b_dev,
                                       const cldnn_hip_tensor* b, void* dst_dev, const cldnn_hip_tensor* dst,
                                       int32_t quantized, const float* calib_dev, float output_quantization_factor,
                                       int32_t activation, float m, float n)
{
    return guarded([&] {
        CHIP_REQUIRE(e && a_dev && a && b_dev && b && dst_dev && dst, CLDNN_HIP_INVALID_ARG, "null argument");
        e->make_current();
        launch_pointwise(e->stream, *a, a_dev, b, b_dev, *dst, dst_dev, quantized, calib_dev, output_quantization_factor,
                         activation, m, n);
    });
}

cldnn_hip_status cldnn_hip_eltwise(cldnn_hip_engine e, const cldnn_hip_eltwise_desc* desc, const void* const* inputs_dev,
                                   const float* calib_dev, void* output_dev)
{
    return guarded([&] {
        CHIP_REQUIRE(e && desc && inputs_dev && output_dev, CLDNN_HIP_INVALID_ARG, "null argument");
        e->make_current();
        launch_eltwise(e->stream, *desc, inputs_dev, calib_dev, output_dev);
    });
}

cldnn_hip_status cldnn_hip_pooling(cldnn_hip_engine e, const cldnn_hip_pooling_desc* desc, const void* input_dev, void* output_dev)
{
    return guarded([&] {
        CHIP_REQUIRE(e && desc && input_dev && output_dev, CLDNN_HIP_INVALID_ARG, "null argument");
        e->make_current();
        launch_pooling(e->stream, *desc, input_dev, output_dev);
    });
}

int32_t cldnn_hip_pooling_out_extent(int32_t in, int32_t pad, int32_t size, int32_t stride)
{
    if (in <= 0 || size <= 0 || stride <= 0) return 0;
    const int off = -pad, extend = size > stride ? size : stride;
    // the last window may reach past the padded input once ...
    const int once = 2 * off + extend <= in + stride - 1 ? (in - 2 * off - extend + stride - 1) / stride + 1 : 1;
    // ... but has to start inside input + leading padding
    const int any = off <= in - 1 ? (in - off - 1) / stride + 1 : 1;
    return once < any ? once : any;
}

}  // extern "C"
