// Quantized convolution through the C++ API, checked against the CPU oracle.
//
// Written the way the reference's tests are (tests/test_cases/convolution_gpu_test.cpp:3741-3969,
// tests/test_cases/fused_conv_eltwise_gpu_test.cpp:169-271): allocate memories on an engine, fill them through
// pointer<T>, build a topology of input_layout / data / convolution, run a network, read the output memory.
// Exit status 0 = every case equal to the oracle bit for bit.  Needs a GPU.
#include <api/CPP/convolution.hpp>
#include <api/CPP/data.hpp>
#include <api/CPP/eltwise.hpp>
#include <api/CPP/engine.hpp>
#include <api/CPP/input_layout.hpp>
#include <api/CPP/memory.hpp>
#include <api/CPP/network.hpp>
#include <api/CPP/reorder.hpp>
#include <api/CPP/topology.hpp>
#include <api_extension/CPP/fused_conv_eltwise.hpp>

#include <cstdio>
#include <random>
#include <vector>

#include "../../oracle/refconv.h"

using namespace cldnn;

static int failures = 0;
#define EXPECT(cond, ...)                 \
    do {                                  \
        if (!(cond)) {                    \
            ++failures;                   \
            std::printf("FAILED: ");      \
            std::printf(__VA_ARGS__);     \
            std::printf("\n");            \
        }                                 \
    } while (0)

template <class T> static void set_values(const memory& mem, const std::vector<T>& v)
{
    auto ptr = mem.pointer<T>();
    EXPECT(ptr.size() >= v.size(), "memory smaller than its values");
    for (size_t i = 0; i < v.size(); ++i) ptr[i] = v[i];
}

struct problem {
    int B, IFM, H, W, OFM, K, pad;
    std::vector<uint8_t> x;
    std::vector<int8_t> w, shortcut;
    std::vector<int32_t> bias;
    std::vector<float> wqf, calib, ecal;
    int OH() const { return rc_out_extent(H, pad, K, 1, 1); }
    int OW() const { return rc_out_extent(W, pad, K, 1, 1); }
};

static problem make_problem(unsigned seed, int B, int IFM, int H, int W, int OFM, int K)
{
    problem p{};
    p.B = B, p.IFM = IFM, p.H = H, p.W = W, p.OFM = OFM, p.K = K, p.pad = K / 2;
    std::mt19937 gen(seed);
    p.x.resize((size_t)B * IFM * H * W);
    for (auto& v : p.x) v = (uint8_t)(gen() % 256);
    p.w.resize((size_t)OFM * IFM * K * K);
    for (auto& v : p.w) v = (int8_t)((int)(gen() % 255) - 127);
    p.bias.resize(OFM);
    for (auto& v : p.bias) v = (int)(gen() % 2001) - 1000;
    p.wqf.assign(OFM, 1.0f);
    p.calib.resize(OFM);
    const float sigma = std::sqrt((float)(IFM * K * K)) * 147.4f * 73.3f;
    for (auto& v : p.calib) v = 40.0f / sigma * (0.5f + (gen() % 1000) / 666.0f);
    p.shortcut.resize((size_t)B * OFM * p.OH() * p.OW());
    for (auto& v : p.shortcut) v = (int8_t)((int)(gen() % 256) - 128);
    p.ecal.resize(OFM);
    for (auto& v : p.ecal) v = 0.25f + (gen() % 1000) / 1333.0f;
    return p;
}

static std::vector<int8_t> oracle(const problem& p, bool fused)
{
    rc_desc d{};
    d.in_dt = RC_U8, d.w_dt = RC_S8, d.bias_dt = RC_I32, d.out_dt = RC_S8, d.eltw_dt = RC_S8;
    d.B = p.B, d.IFM = p.IFM, d.IH = p.H, d.IW = p.W, d.OFM = p.OFM, d.OH = p.OH(), d.OW = p.OW();
    d.FY = d.FX = p.K, d.sy = d.sx = d.dy = d.dx = 1, d.pad_y = d.pad_x = p.pad, d.groups = 1;
    d.has_wqf = d.has_calib = 1, d.iqf = d.oqf = 1.0f;
    d.act = fused ? RC_ACT_NONE : RC_ACT_RELU;
    d.fused = fused, d.non_conv_scale = 1.0f, d.eltw_act = RC_ACT_RELU, d.has_eltw_calib = fused, d.esy = d.esx = 1;
    rc_dense_bfyx(&d.in_p, p.IFM, p.H, p.W);
    rc_dense_bfyx(&d.out_p, p.OFM, d.OH, d.OW);
    rc_dense_bfyx(&d.eltw_p, p.OFM, d.OH, d.OW);
    std::vector<int8_t> out((size_t)p.B * p.OFM * d.OH * d.OW);
    int rc = rc_conv(&d, p.x.data(), p.w.data(), p.bias.data(), p.wqf.data(), p.calib.data(), fused ? p.shortcut.data() : nullptr,
                     fused ? p.ecal.data() : nullptr, out.data(), nullptr, 4);
    EXPECT(rc == 0, "oracle refused the problem");
    return out;
}

static topology conv_topology(const engine& eng, const problem& p, bool fused_primitive, bool as_eltwise)
{
    auto input = memory::allocate(eng, {data_types::u8, format::bfyx, {p.B, p.IFM, p.W, p.H}});
    (void)input;
    auto weights = memory::allocate(eng, {data_types::i8, format::bfyx, {p.OFM, p.IFM, p.K, p.K}});
    auto biases = memory::allocate(eng, {data_types::i32, format::bfyx, {1, 1, p.OFM, 1}});
    auto w_qf = memory::allocate(eng, {data_types::f32, format::bfyx, {1, 1, p.OFM, 1}});
    auto calibrations = memory::allocate(eng, {data_types::f32, format::bfyx, {1, 1, p.OFM, 1}});
    auto eltw_calib = memory::allocate(eng, {data_types::f32, format::bfyx, {1, 1, p.OFM, 1}});
    set_values(weights, p.w);
    set_values(biases, p.bias);
    set_values(w_qf, p.wqf);
    set_values(calibrations, p.calib);
    set_values(eltw_calib, p.ecal);

    topology topo(input_layout("input", {data_types::u8, format::bfyx, {p.B, p.IFM, p.W, p.H}}), data("weights", weights),
                  data("biases", biases), data("w_qf", w_qf), data("calibrations", calibrations));
    const tensor offset{0, 0, -p.pad, -p.pad};
    if (fused_primitive) {
        topo.add(input_layout("shortcut", {data_types::i8, format::bfyx, {p.B, p.OFM, p.OW(), p.OH()}}), data("eltw_calib", eltw_calib),
                 fused_conv_eltwise("conv", "input", "shortcut", eltwise_mode::sum, {"weights"}, {"biases"}, {"w_qf"}, {"calibrations"}, 1.0f,
                                    1.0f, "eltw_calib", {}, {1, 1, 1, 1}, offset, {1, 1, 1, 1}, false, 0.0f, true, 0.0f, padding(),
                                    optional_data_type(data_types::i8)));
    } else if (as_eltwise) {
        convolution conv("conv_part", "input", {"weights"}, {"biases"}, {"w_qf"}, {"calibrations"}, 1.0f, {1, 1, 1, 1}, offset);
        conv.set_output_data_type(data_types::i8);
        topo.add(input_layout("shortcut", {data_types::i8, format::bfyx, {p.B, p.OFM, p.OW(), p.OH()}}), data("eltw_calib", eltw_calib), conv,
                 eltwise("sum", "shortcut", "conv_part", "eltw_calib", eltwise_mode::sum, true), reorder("conv", "sum", format::bfyx, data_types::i8));
    } else {
        convolution conv("conv", "input", {"weights"}, {"biases"}, {"w_qf"}, {"calibrations"}, 1.0f, {1, 1, 1, 1}, offset, {1, 1, 1, 1}, true);
        conv.set_output_data_type(data_types::i8);
        topo.add(conv);
    }
    return topo;
}

static void run_case(const engine& eng, const char* name, const problem& p, bool fused_primitive, bool as_eltwise, bool optimize)
{
    const bool fused = fused_primitive || as_eltwise;
    topology topo = conv_topology(eng, p, fused_primitive, as_eltwise);
    build_options opts;
    opts.set_option(build_option::optimize_data(optimize));
    network net(eng, topo, opts);

    auto input = memory::allocate(eng, {data_types::u8, format::bfyx, {p.B, p.IFM, p.W, p.H}});
    set_values(input, p.x);
    net.set_input_data("input", input);
    if (fused) {
        auto shortcut = memory::allocate(eng, {data_types::i8, format::bfyx, {p.B, p.OFM, p.OW(), p.OH()}});
        set_values(shortcut, p.shortcut);
        net.set_input_data("shortcut", shortcut);
    }
    auto outputs = net.execute();
    EXPECT(outputs.size() == 1 && outputs.begin()->first == "conv", "%s: unexpected outputs", name);
    auto out_mem = outputs.at("conv").get_memory();
    auto out_layout = out_mem.get_layout();
    EXPECT(out_layout.format == format::bfyx && out_layout.data_type == data_types::i8, "%s: output layout", name);
    EXPECT(out_layout.size == tensor(p.B, p.OFM, p.OW(), p.OH()), "%s: output size", name);
    const std::vector<int8_t> expected = oracle(p, fused);
    auto ptr = out_mem.pointer<int8_t>();
    size_t bad = 0;
    for (size_t i = 0; i < expected.size(); ++i) bad += ptr[i] != expected[i];
    EXPECT(bad == 0, "%s: %zu of %zu outputs differ from the oracle", name, bad, expected.size());
    std::printf("%-44s %s  (%zu outputs, %zu primitives executed)\n", name, bad ? "MISMATCH" : "ok", expected.size(),
                net.get_executed_primitive_ids().size());
}

int main()
{
    try {
        engine eng;
        const problem a = make_problem(1337, 2, 64, 14, 14, 64, 3);
        const problem b = make_problem(7, 3, 32, 9, 11, 48, 1);
        run_case(eng, "conv 3x3 u8->i8 relu, as written", a, false, false, false);
        run_case(eng, "conv 3x3 u8->i8 relu, optimize_data", a, false, false, true);
        run_case(eng, "fused_conv_eltwise 1x1, as written", b, true, false, false);
        run_case(eng, "fused_conv_eltwise 1x1, optimize_data", b, true, false, true);
        run_case(eng, "conv 1x1 + eltwise, fused by the pass", b, false, true, true);

        // error behaviour: exceptions of type cldnn::error with the C status
        bool thrown = false;
        try {
            topology topo = conv_topology(eng, a, false, false);
            network net(eng, topo);
            net.set_input_data("input", memory::allocate(eng, {data_types::u8, format::bfyx, {1, 1, 1, 1}}));
        } catch (const cldnn::error& e) {
            thrown = e.status() == CLDNN_INVALID_ARG;
        }
        EXPECT(thrown, "set_input_data with a wrong layout must throw cldnn::error(CLDNN_INVALID_ARG)");
    } catch (const std::exception& e) {
        std::printf("FAILED with exception: %s\n", e.what());
        return 2;
    }
    std::printf(failures ? "%d failure(s)\n" : "all cases passed\n", failures);
    return failures ? 1 : 0;
}
