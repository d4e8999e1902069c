// Host side of the convolution chain kernel: eligibility, LDS image of the weights, launch.
#include <algorithm>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "conv_dwchain_kernel.h"

namespace chip {

namespace {

enum { ROW_P64_F64_FOR_DWCHAIN = 4 };  // the 64x64 LDS-staged row: same 64-row unit order, any feature count (K padded with zeros)
enum { ROW_WSL_P64_FOR_CHAIN = 14 };  // the 64-feature weights-stationary row: its packed stream is the LDS image's unit order
enum { CHAIN_MAX_LDS = 160 * 1024 };

int epilogue_kind(const ChainStageIn& s)
{
    const FastEpi& f = *s.fe;
    int kind = EPI_KIND_FAST;
    if (f.has_wqf && f.iqf_one && f.clamp_folded && !f.fused && !f.fc && s.epi->calib) kind = EPI_KIND_CLAMPQ;
    if (!f.has_wqf && s.epi->calib && !f.fc) {
        if (!f.fused && f.relu_folded) kind = EPI_KIND_RELU;
        if (!f.fused && f.act == CLDNN_HIP_ACT_NONE) kind = EPI_KIND_LINEAR;
        if (f.fused && f.act == CLDNN_HIP_ACT_NONE && f.eltw_relu_folded && s.epi->eltw_calib && !f.conv_sat) kind = EPI_KIND_FUSED;
        if (f.fused && f.act == CLDNN_HIP_ACT_NONE && f.eltw_act == CLDNN_HIP_ACT_NONE && !f.eltw_relu_folded) kind = EPI_KIND_SUMLIN;
    }
    return kind;
}

struct Instance {
    int nt, d, sp0, sp1, sp2, e0, e1, e2;
    void (*launch)(hipStream_t, const ChainArgs&, int, int);
};
#define CHAIN_INSTANCE(NT, D, SP0, SP1, SP2, E0, E1, E2) \
    {NT, D, SP0, SP1, SP2, E0, E1, E2, &launch_chain_instance<NT, D, SP0, SP1, SP2, E0, E1, E2>}
// What is compiled: the tails of ResNet bottlenecks with 64 mid features (3x3 -> expansion [+ residual] -> next
// reduction), with and without the third stage, residual fused or not.
const Instance g_instances[] = {
    CHAIN_INSTANCE(2, 3, 1, 4, 1, EPI_KIND_RELU, EPI_KIND_FUSED, EPI_KIND_RELU),
    CHAIN_INSTANCE(2, 3, 1, 4, 0, EPI_KIND_RELU, EPI_KIND_FUSED, EPI_KIND_RELU),
    CHAIN_INSTANCE(2, 3, 1, 4, 1, EPI_KIND_RELU, EPI_KIND_RELU, EPI_KIND_RELU),
    CHAIN_INSTANCE(2, 3, 1, 4, 0, EPI_KIND_RELU, EPI_KIND_RELU, EPI_KIND_RELU),
};

const Instance* find_instance(const ChainPlan& pl)
{
    for (const Instance& i : g_instances)
        if (i.nt == pl.nt && i.d == pl.depth && i.sp0 == pl.sp[0] && i.sp1 == pl.sp[1] && i.sp2 == pl.sp[2] && i.e0 == pl.epi[0]
            && i.e1 == pl.epi[1] && (pl.stages < 3 || i.e2 == pl.epi[2]))
            return &i;
    return nullptr;
}

}  // namespace

std::string chain_plan(const ChainStageIn* st, int n, int cus, ChainPlan* out)
{
    ChainPlan pl{};
    if (n < 2 || n > CHAIN_MAX_STAGES) return "a chain has two or three stages";
    pl.stages = n;
    const ConvProblem& p0 = *st[0].p;
    for (int k = 0; k < n; ++k) {
        const ConvProblem& p = *st[k].p;
        const std::string at = "stage " + std::to_string(k) + ": ";
        if (!st[k].fast) return at + "needs the short int8 epilogue";
        if (st[k].fe->fc) return at + "the fully_connected form is not chained";
        const bool dw0 = k == 0 && st[0].dw_wmask != nullptr;
        if (p.groups != 1 && !dw0) return at + "grouped convolution";
        if (p.in_t.format != CLDNN_HIP_FMT_FS_B_YX_FSV16 || p.out_t.format != CLDNN_HIP_FMT_FS_B_YX_FSV16) return at + "needs fs_b_yx_fsv16";
        if (st[0].dw_wmask == nullptr && (p.IFM % 64 != 0 || p.OFM % 64 != 0)) return at + "feature counts must be multiples of 64";
        if (st[0].dw_wmask != nullptr && k < 2 && p.IFM % 16 != 0) return at + "a depthwise chain needs feature counts in multiples of 16 up to the projection";
        if (st[k].fe->fused && p.eltw_t.format != CLDNN_HIP_FMT_FS_B_YX_FSV16) return at + "unblocked residual";
        if (tensor_elems(p.out_t) >= (1ull << 31) || tensor_elems(p.in_t) >= (1ull << 31)) return at + "tensor of 2 GiB or more";
        if (k > 0) {
            const ConvProblem& q = *st[k - 1].p;
            if (p.FY != 1 || p.FX != 1 || p.sy != 1 || p.sx != 1 || p.py != 0 || p.px != 0) return at + "only the first stage may be wider than 1x1";
            if (p.IFM != q.OFM || p.B != q.B || p.IH != q.OH || p.IW != q.OW) return at + "does not read the previous stage's result";
            if (p.in_dt != q.out_dt) return at + "input type differs from the previous stage's output type";
        }
        pl.sp[k] = (p.OFM + 63) / 64;
        pl.epi[k] = epilogue_kind(st[k]);
    }
    if (!conv_border_covers(p0)) return "stage 0: the input needs a zero border as wide as the padding";
    if (p0.dy != 1 || p0.dx != 1) return "stage 0: dilation";
    pl.m_total = (int64_t)p0.B * p0.OH * p0.OW;
    if (st[0].dw_wmask) {
        // ---- depthwise first stage: lane = pixel on the vector ALU, 64-pixel granules, later stages resident in LDS
        if (p0.FY != 3 || p0.FX != 3) return "stage 0: the depthwise stage of a chain is 3x3";
        if (st[0].fe->fused) return "stage 0: a fused depthwise stage is not chained";
        if (pl.sp[1] != 1) return "stage 1: the projection behind a depthwise stage has at most 64 features";
        pl.dw = 1;
        // 32-pixel granules; 16-pixel ones where that still leaves waves without work (14x14 and 7x7 planes)
        pl.nt = pl.m_total / 32 >= (int64_t)cus * 8 ? 2 : 1;
        pl.granules = (int)((pl.m_total + 16 * pl.nt - 1) / (16 * pl.nt));
        pl.units = 0;
        int vec = 0;
        for (int k = 0; k < n; ++k) {
            if (k > 0) {
                MfmaPlan mp{};
                try {
                    mp = mfma_plan(*st[k].p, ROW_P64_F64_FOR_DWCHAIN, cus);
                } catch (const error& e) {
                    return "stage " + std::to_string(k) + ": " + e.what();
                }
                pl.unit0[k] = pl.units, pl.kstride[k] = mp.ksteps;
                pl.units += pl.sp[k] * mp.ksteps;
            }
            pl.vec0[k] = vec;
            vec += 4 * pl.sp[k] * 64;
        }
        pl.ksteps0 = pl.sp[0];  // K-steps the depthwise stage delivers to stage 1
        pl.lds_bytes = pl.sp[0] * 9 * 1024 + pl.units * 4096 + vec * 4;  // diagonal-weight table, units, vectors
        if (pl.lds_bytes > CHAIN_MAX_LDS) return "the weights of the chain (" + std::to_string(pl.lds_bytes / 1024) + " KiB) do not fit into LDS";
        // workgroups a CU holds at once: by LDS, and by registers (16-pixel granules: 137-167 registers = three waves per
        // SIMD; 32-pixel granules: 206-239 = two).  The grid is what is resident, so that no workgroup waits for a slot.
        const int per_cu = std::min(pl.nt == 1 ? 3 : 2, CHAIN_MAX_LDS / pl.lds_bytes);
        int grid = cus * per_cu / 8 * 8;
        const int wanted = ((pl.granules + 3) / 4 + 7) / 8 * 8;  // at least one granule per wave
        if (grid > wanted) grid = wanted;
        if (grid < 8) grid = 8;
        pl.grid = grid;
        std::snprintf(pl.name, sizeof(pl.name), "conv_dwchain<%d stages,p%d,mid %d,spans %d-%d>", n, 16 * pl.nt, p0.OFM, pl.sp[1], n > 2 ? pl.sp[2] : 0);
        *out = pl;
        return std::string();
    }
    pl.nt = 2;
    pl.granules = (int)((pl.m_total + 16 * pl.nt - 1) / (16 * pl.nt));
    // K-steps of every stage as the weights-stationary row packs them
    MfmaPlan mp[3]{};
    for (int k = 0; k < n; ++k) {
        ConvProblem q = *st[k].p;
        try {
            mp[k] = mfma_plan(q, ROW_WSL_P64_FOR_CHAIN, cus);
        } catch (const error&) {
            // K beyond what that row keeps in LDS: only the K-step count is wanted here
            mp[k] = MfmaPlan{};
            mp[k].ksteps = (q.FY * q.FX * ((q.IFM + 15) / 16) + 3) / 4;
            mp[k].wsl_depth = 0;
        }
        if (k > 0 && mp[k].ksteps < pl.sp[k - 1]) return "stage " + std::to_string(k) + ": fewer K-steps than the previous stage has spans";
    }
    // everything in LDS, independent waves
    {
        pl.units = 0;
        int vec = 0;
        for (int k = 0; k < n; ++k) {
            pl.unit0[k] = pl.units, pl.kstride[k] = mp[k].ksteps;
            pl.units += pl.sp[k] * mp[k].ksteps;
            pl.vec0[k] = vec;
            vec += 4 * pl.sp[k] * 64;
        }
        pl.depth = mp[0].wsl_depth, pl.ksteps0 = mp[0].ksteps;
        pl.lds_bytes = pl.units * 4096 + vec * 4;
        if (mp[0].wsl_depth > 0 && pl.lds_bytes <= CHAIN_MAX_LDS && find_instance(pl)) {
            const int per_cu = pl.lds_bytes * 2 <= CHAIN_MAX_LDS ? 2 : 1;
            int grid = cus * per_cu / 8 * 8;
            const int wanted = ((pl.granules + 3) / 4 + 7) / 8 * 8;  // at least one granule per wave
            if (grid > wanted) grid = wanted;
            if (grid < 8) grid = 8;
            pl.grid = grid;
            std::snprintf(pl.name, sizeof(pl.name), "conv_chain<%d stages,p%d,d%d,spans %d-%d-%d,epi %d-%d-%d>", n, 16 * pl.nt, pl.depth,
                          pl.sp[0], pl.sp[1], pl.sp[2], pl.epi[0], pl.epi[1], n > 2 ? pl.epi[2] : -1);
            *out = pl;
            return std::string();
        }
    }
    if (mp[0].wsl_depth <= 0 || pl.lds_bytes > CHAIN_MAX_LDS)
        return "the weights of the chain (" + std::to_string(pl.units * 4) + " KiB) do not fit into LDS";
    return "no compiled instance for this chain shape";
}

size_t chain_packed_bytes(const ChainPlan& pl) { return (size_t)pl.lds_bytes + 4096; }

static void fill_stage(ChainStage& c, const ChainStageIn& in, const ChainPlan& pl, int k, void* out, const void* eltw)
{
    const ConvProblem& p = *in.p;
    c.out = out;
    c.eltw = eltw;
    CHIP_REQUIRE(!in.fe->fused || c.eltw, CLDNN_HIP_INVALID_ARG, "fused stage of a chain without its second input");
    c.OFM = p.OFM;
    c.out_off = (int32_t)p.out_p.off, c.out_pb = (int32_t)p.out_p.pb, c.out_pf = (int32_t)p.out_p.pf, c.out_py = (int32_t)p.out_p.py;
    c.el_off = (int32_t)p.eltw_p.off, c.el_pb = (int32_t)p.eltw_p.pb, c.el_pf = (int32_t)p.eltw_p.pf;
    c.el_py = (int32_t)p.eltw_p.py * p.esy, c.el_px = 16 * p.esx;  // a strided residual: the shortcut sub-sampled in place
    c.xor_mask = p.in_dt == CLDNN_HIP_U8 ? 0x80808080u : 0u;
    c.unit0 = pl.unit0[k], c.kstride = pl.kstride[k], c.vec0 = pl.vec0[k];
    c.fe = *in.fe;
    c.epi = *in.epi;
}

static void launch_dwchain(hipStream_t s, const ChainStageIn* st, const ChainPlan& pl, const void* packed_dev, const void* in,
                           void* const* outs, const void* const* eltws)
{
    const ConvProblem& p0 = *st[0].p;
    DwChainArgs a{};
    a.in = (const int8_t*)in;
    a.img = (const v4i*)packed_dev;
    a.dw_quads = pl.sp[0] * 9 * 64;
    a.units = pl.units;
    a.vec_quads = (pl.lds_bytes - a.dw_quads * 16 - pl.units * 4096) / 16;
    a.granules = pl.granules;
    a.gpw = pl.granules / (pl.grid * 4), a.grem = pl.granules % (pl.grid * 4);
    a.div_waves = make_fast_div((uint32_t)pl.grid * 4u);
    a.M = (uint32_t)pl.m_total;
    a.OHW = p0.OH * p0.OW, a.OW = p0.OW;
    a.div_ohw = make_fast_div((uint32_t)a.OHW), a.div_ow = make_fast_div((uint32_t)a.OW);
    a.sy = p0.sy, a.sx = p0.sx, a.py = p0.py, a.px = p0.px;
    a.in_off = (int32_t)p0.in_p.off, a.in_pb = (int32_t)p0.in_p.pb, a.in_pf = (int32_t)p0.in_p.pf, a.in_py = (int32_t)p0.in_p.py;
    a.tap_dy = p0.dy * (int32_t)p0.in_p.py, a.tap_dx = p0.dx * 16;
    a.CB = (p0.OFM + 15) / 16;
    a.KS = (a.CB + 3) / 4;
    a.SP2 = pl.stages > 2 ? pl.sp[2] : 0;
    for (int k = 0; k < pl.stages; ++k) fill_stage(a.st[k], st[k], pl, k, outs[k], eltws ? eltws[k] : nullptr);
    // the branch-free epilogue forms of a MobileNet block (clamp on the dequantised value, linear projection, clamp), else
    // the run-time form for every stage
    constexpr int CQ = EPI_KIND_CLAMPQ, LIN = EPI_KIND_LINEAR, SUM = EPI_KIND_SUMLIN, ANY = EPI_KIND_FAST;
    const bool ends = pl.epi[0] == CQ && (pl.stages < 3 || pl.epi[2] == CQ);
    const bool block = ends && pl.epi[1] == LIN, block_sum = ends && pl.epi[1] == SUM;  // projection without / with the block's sum
#define DWCHAIN_LAUNCH(NT, HAS2)                                                                           \
    {                                                                                                      \
        if (block) launch_dwchain_instance<NT, 1, HAS2, CQ, LIN, CQ>(s, a, pl.grid, pl.lds_bytes);         \
        else if (block_sum) launch_dwchain_instance<NT, 1, HAS2, CQ, SUM, CQ>(s, a, pl.grid, pl.lds_bytes); \
        else launch_dwchain_instance<NT, 1, HAS2, ANY, ANY, ANY>(s, a, pl.grid, pl.lds_bytes);             \
    }
    if (pl.nt == 2) {
        if (pl.stages > 2) DWCHAIN_LAUNCH(2, true) else DWCHAIN_LAUNCH(2, false)
    } else {
        if (pl.stages > 2) DWCHAIN_LAUNCH(1, true) else DWCHAIN_LAUNCH(1, false)
    }
#undef DWCHAIN_LAUNCH
    CHIP_CHECK(hipGetLastError());
}

void chain_pack_weights(const ChainStageIn* st, const ChainPlan& pl, int cus, const int8_t* const* w, const ChainVectors* vec,
                        int8_t* packed)
{
    std::memset(packed, 0, chain_packed_bytes(pl));
    const size_t dw_bytes = pl.dw ? (size_t)pl.sp[0] * 9 * 1024 : 0;
    if (pl.dw) {
        // diagonal-weight dwords [K-step][tap][fragment][lane]: lane (kq, l16) of fragment mt carries the weight of feature
        // 64 ks + 16 (l16 / 4) + 4 mt + l16 % 4 in byte l16 % 4 when kq == l16 / 4, else zero
        const ConvProblem& p0 = *st[0].p;
        int32_t* dia = reinterpret_cast<int32_t*>(packed);
        for (int ks = 0; ks < pl.sp[0]; ++ks)
            for (int tap = 0; tap < 9; ++tap)
                for (int mt = 0; mt < 4; ++mt)
                    for (int lane = 0; lane < 64; ++lane) {
                        const int kq = lane >> 4, l16 = lane & 15;
                        const int ch = ks * 64 + 16 * (l16 >> 2) + 4 * mt + (l16 & 3);
                        int32_t v = 0;
                        if (kq == (l16 >> 2) && ch < p0.OFM) v = (int32_t)((uint32_t)(uint8_t)w[0][(size_t)ch * 9 + tap] << (8 * (l16 & 3)));
                        dia[((ks * 9 + tap) * 4 + mt) * 64 + lane] = v;
                    }
    }
    packed += dw_bytes;
    // per-feature vectors behind the weight units: per stage init, calib, eltw_calib, wqf, spans * 64 entries each
    int32_t* v = reinterpret_cast<int32_t*>(packed + (size_t)pl.units * 4096);
    const float one = 1.0f;
    int32_t one_bits;
    std::memcpy(&one_bits, &one, 4);
    for (int k = 0; k < pl.stages; ++k) {
        const int n = pl.sp[k] * 64, ofm = st[k].p->OFM;
        const void* src[4] = {vec[k].acc_init, vec[k].calib, vec[k].eltw_calib, vec[k].wqf};
        for (int kind = 0; kind < 4; ++kind) {
            int32_t* dst = v + pl.vec0[k] + kind * n;
            // without calibration factors the epilogue multiplies by the output quantization factor (or by one)
            int32_t fill = kind == 0 ? 0 : one_bits;
            if (kind == 1 && !src[kind] && st[k].epi->oqf_on) std::memcpy(&fill, &st[k].epi->oqf, 4);
            for (int f = 0; f < n; ++f) dst[f] = fill;
            if (src[kind]) std::memcpy(dst, src[kind], (size_t)ofm * 4);
        }
    }
    for (int k = pl.dw ? 1 : 0; k < pl.stages; ++k) {
        const MfmaPlan mp = mfma_plan(*st[k].p, pl.dw ? ROW_P64_F64_FOR_DWCHAIN : ROW_WSL_P64_FOR_CHAIN, cus);
        std::vector<int8_t> buf(mp.packed_bytes);
        std::vector<int32_t> ktab(mp.ktab_bytes / sizeof(int32_t));
        mfma_pack_weights(*st[k].p, mp, w[k], buf.data(), ktab.data());
        std::memcpy(packed + (size_t)pl.unit0[k] * 4096, buf.data(), (size_t)pl.sp[k] * mp.ksteps * 4096);
    }
}

void launch_conv_chain(hipStream_t s, const ChainStageIn* st, const ChainPlan& pl, const void* packed_dev, const void* in,
                       void* const* outs, const void* const* eltws)
{
    if (pl.dw) return launch_dwchain(s, st, pl, packed_dev, in, outs, eltws);
    const ConvProblem& p0 = *st[0].p;
    ChainArgs a{};
    a.in = (const int8_t*)in;
    a.wpk = (const v4i*)packed_dev;
    a.units = pl.units;
    a.vec_quads = (pl.lds_bytes - pl.units * 4096) / 16;
    a.granules = pl.granules;
    a.gpw = pl.granules / (pl.grid * 4), a.grem = pl.granules % (pl.grid * 4);
    a.div_waves = make_fast_div((uint32_t)pl.grid * 4u);
    a.M = (uint32_t)pl.m_total;
    a.OHW = p0.OH * p0.OW, a.OW = p0.OW;
    a.div_ohw = make_fast_div((uint32_t)a.OHW), a.div_ow = make_fast_div((uint32_t)a.OW);
    a.sy = p0.sy, a.sx = p0.sx, a.py = p0.py, a.px = p0.px;
    a.in_off = (int32_t)p0.in_p.off, a.in_pb = (int32_t)p0.in_p.pb, a.in_pf = (int32_t)p0.in_p.pf, a.in_py = (int32_t)p0.in_p.py;
    a.ksteps0 = pl.ksteps0, a.CB = (p0.IFM + 15) / 16, a.FX = p0.FX, a.FY = p0.FY;
    a.tap_dy = p0.dy * (int32_t)p0.in_p.py, a.tap_dx = p0.dx * 16;
    for (int k = 0; k < pl.stages; ++k) fill_stage(a.st[k], st[k], pl, k, outs[k], eltws ? eltws[k] : nullptr);
    const Instance* inst = find_instance(pl);
    CHIP_REQUIRE(inst, CLDNN_HIP_ERROR, "chain without a compiled instance");
    inst->launch(s, a, pl.grid, pl.lds_bytes);
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
