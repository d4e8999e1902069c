// Host side of the int8 MFMA convolution: the gfx950 tile-config table, plans, weight
// pre-packing, eligibility of the short epilogue and the launch.
#include <algorithm>
#include <cmath>
#include <cstring>

#include "conv_halo_kernel.h"

namespace chip {

#define DECL_TILE(i) void launch_mfma_tile_##i(hipStream_t, const MfmaArgs&, int, int, bool, int);
DECL_TILE(0) DECL_TILE(1) DECL_TILE(2) DECL_TILE(3) DECL_TILE(4) DECL_TILE(5)
#undef DECL_TILE
void launch_stream(hipStream_t s, const MfmaArgs& a, int nt, int grid, int epi);
void launch_bdir_f64(hipStream_t s, const MfmaArgs& a, int nt, int grid, int lds, int epi);
void launch_bdir_f128(hipStream_t s, const MfmaArgs& a, int nt, int grid, int lds, int epi);
void launch_bdir_k2(hipStream_t s, const MfmaArgs& a, int nt, int grid, int lds, int epi);
void launch_bdir_k4(hipStream_t s, const MfmaArgs& a, int nt, int grid, int lds, int epi);
void launch_gemv(hipStream_t s, const MfmaArgs& a, int grid, int waves, int mtiles);
size_t gemv_gather_bytes(int mtiles, int ksteps);
size_t gemv_static_scratch_bytes();
void* gemv_static_scratch(int device);
#define DECL_WSL(d) void launch_wsl_d##d(hipStream_t s, const MfmaArgs& a, int nt, int grid, int lds, int epi);
DECL_WSL(1) DECL_WSL(2) DECL_WSL(3) DECL_WSL(4) DECL_WSL(6) DECL_WSL(8)
#undef DECL_WSL
void launch_halo(hipStream_t s, const HaloArgs& h, int row, int pl, int grid, int lds, int epi);

typedef void (*tile_launcher)(hipStream_t, const MfmaArgs&, int, int, bool, int);

static const TileConfig g_tiles[] = {
    {"p128_f128", 128, 128, 64},
    {"p256_f64", 256, 64, 64},
    {"p64_f128", 64, 128, 32},
    {"p128_f64", 128, 64, 32},
    {"p64_f64", 64, 64, 16},
    {"p256_f128", 256, 128, 128},
    // rows of the streaming kernel: a wave owns one span of 64 features of one tile of wave_pixels pixels
    {"stream_p16", 16, 64, 16},
    {"stream_p32", 32, 64, 32},
    // rows of the direct-activation kernel: weights through LDS, activations straight into registers;
    // a wave owns wave_pixels pixels and all tile_ofm features
    {"bdir_p64_f64", 64, 64, 16},
    {"bdir_p128_f64", 128, 64, 32},
    {"bdir_p256_f64", 256, 64, 64},
    {"bdir_p64_f128", 64, 128, 16},
    {"bdir_p128_f128", 128, 128, 32},
    {"bdir_p256_f128", 256, 128, 64},
    // rows of the weights-stationary kernel: persistent workgroups, the 64-feature weight tile resident in LDS
    {"wsl_p64", 64, 64, 16},
    {"wsl_p128", 128, 64, 32},
    {"wsl_p256", 256, 64, 64},
    // direct-activation kernel with K split over 2 or 4 groups of four waves inside the workgroup
    {"bdir_k2_p64_f64", 64, 64, 16, 2},
    {"bdir_k4_p64_f64", 64, 64, 16, 4},
    {"bdir_k2_p128_f64", 128, 64, 32, 2},
    // first layers (at most 4 input features) read b_fs_yx_fsv4: a 16-byte fragment is 4 horizontal taps x 4 features;
    // streaming kernel
    {"stem_p32", 32, 64, 32},
    // few pixels, long K (fully_connected): a workgroup owns one 16-feature fragment of a 64-feature tile and 16
    // pixels; its waves split K and stream both operands straight from global memory
    {"gemv_p16_f16", 16, 64, 16},
    // first layers with several K-steps (a 7x7 filter): 64 pixels per wave, so the weights are fetched half as often
    {"stem_p64", 64, 64, 64},
    // nine-tap stride-1 kernel with both operands in LDS (direct global -> LDS loads); persistent workgroups; a wave
    // owns 64 positions x 128 features.  tile_pixels counts positions of the bordered input.
    {"halo_p256_f128", 256, 128, 64},   // 4 waves, two workgroups per CU
    {"halo_p512_f128", 512, 128, 64},   // 8 waves, one workgroup per CU (rows too long for two patches of 256 + halo in 80 KB)
};
enum { FIRST_STREAM_ROW = 6, FIRST_BDIR_ROW = 8, FIRST_WSL_ROW = 14, FIRST_BDIRK_ROW = 17, STEM_ROW = 20, GEMV_ROW = 21, STEM_P64_ROW = 22, FIRST_HALO_ROW = 23 };
enum { HALO_RING = 4, HALO_TAPS = 9 };
enum { WSL_MAX_LDS = 160 * 1024 };
enum { MFMA_SLACK_STEPS = 40 };  // >= weight look-ahead + activation look-ahead + 3
static const tile_launcher g_launch[] = {launch_mfma_tile_0, launch_mfma_tile_1, launch_mfma_tile_2, launch_mfma_tile_3,
                                         launch_mfma_tile_4, launch_mfma_tile_5};

int tile_config_count() { return (int)(sizeof(g_tiles) / sizeof(g_tiles[0])); }
const TileConfig& tile_config(int i) { return g_tiles[i]; }

FastDiv make_fast_div(uint32_t d);
static FastDiv make_div(uint32_t d) { return make_fast_div(d); }
FastDiv make_fast_div(uint32_t d)
{
    FastDiv f{};
    if (d <= 1) {
        f.one = 1;
        return f;
    }
    uint32_t s = 0;
    while ((1ull << s) < d) ++s;              // s = ceil(log2 d) >= 1
    const unsigned p = 31 + s;
    f.mul = (uint32_t)(((1ull << p) + d - 1) / d);  // ceil(2^p / d) < 2^32
    f.shift = p - 32;
    return f;
}

// does the input buffer carry a zero border that covers every tap of every output pixel?
static bool border_covers(const ConvProblem& p);
bool conv_border_covers(const ConvProblem& p) { return border_covers(p); }
static bool border_covers(const ConvProblem& p)
{
    const cldnn_hip_tensor& t = p.in_t;
    const int hi_y = (p.OH - 1) * p.sy - p.py + (p.FY - 1) * p.dy - (p.IH - 1);
    const int hi_x = (p.OW - 1) * p.sx - p.px + (p.FX - 1) * p.dx - (p.IW - 1);
    return t.pad_lo_y >= p.py && t.pad_lo_x >= p.px && t.pad_hi_y >= hi_y && t.pad_hi_x >= hi_x;
}

// ---- the gfx950 tile-config table lookup.  Key: (pixels M, OFM, K-steps, border available, slices in fours);
// value: table row.  The entries come from sweeps of every row over every layer shape of the ResNet-50,
// VGG-16 and MobileNet-v2 stacks (bench.py --tune); they stand where the reference keeps a tuned cache file.
enum {
    ROW_P128_F128 = 0, ROW_P256_F64 = 1, ROW_P64_F128 = 2, ROW_P128_F64 = 3, ROW_P64_F64 = 4, ROW_P256_F128 = 5,
    ROW_STREAM_P16 = 6, ROW_STREAM_P32 = 7,
    ROW_BDIR_P64_F64 = 8, ROW_BDIR_P128_F64 = 9, ROW_BDIR_P256_F64 = 10, ROW_BDIR_P64_F128 = 11, ROW_BDIR_P128_F128 = 12,
    ROW_BDIR_P256_F128 = 13, ROW_WSL_P64 = 14, ROW_WSL_P128 = 15, ROW_WSL_P256 = 16,
    ROW_BDIR_K2_P64_F64 = 17, ROW_BDIR_K4_P64_F64 = 18, ROW_BDIR_K2_P128_F64 = 19, ROW_STEM_P32 = 20, ROW_GEMV = 21, ROW_STEM_P64 = 22,
    ROW_HALO_P256_F128 = 23, ROW_HALO_P512_F128 = 24
};

static int choose_lds_tile(const ConvProblem& p, int64_t m, int cus)
{
    static const int order_f128[] = {ROW_P256_F128, ROW_P128_F128, ROW_P64_F128, ROW_P256_F64, ROW_P128_F64, ROW_P64_F64};
    static const int order_f64[] = {ROW_P256_F64, ROW_P128_F64, ROW_P64_F64};
    const int* order = p.OFM > 64 ? order_f128 : order_f64;
    const int n = p.OFM > 64 ? 6 : 3;
    int best = order[n - 1];
    int64_t best_grid = -1;
    for (int i = 0; i < n; ++i) {
        const TileConfig& tc = g_tiles[order[i]];
        const int64_t grid = ((m + tc.tile_pixels - 1) / tc.tile_pixels) * ((p.OFM + tc.tile_ofm - 1) / tc.tile_ofm);
        if (grid >= 2 * (int64_t)cus) return order[i];
        if (grid > best_grid) best_grid = grid, best = order[i];
    }
    return best;
}

int mfma_choose(const ConvProblem& p, int cus)
{
    if (p.in_t.format == CLDNN_HIP_FMT_B_FS_YX_FSV4)
        return p.FY * ((p.FX + 3) / 4) > 8 ? ROW_STEM_P64 : ROW_STEM_P32;  // more than two K-steps of four 4-tap chunks
    const int64_t m = (int64_t)p.B * p.OH * p.OW;
    const int cb = (p.IFM + 15) / 16;
    const int ksteps = (p.FY * p.FX * cb + 3) / 4;
    const bool border = border_covers(p);
    const bool direct = border && cb % 4 == 0;  // the direct-activation and weights-stationary kernels apply
    const int64_t stream_waves = ((m + 31) / 32) * ((p.OFM + 63) / 64);
    const bool stream_fits = border && ksteps <= 8 && stream_waves * 2 >= 4ll * cus;
    const int stream_row = stream_waves >= 4ll * cus ? ROW_STREAM_P32 : ROW_STREAM_P16;

    // a fragment or two of pixels and a long K (fully_connected): the weights are the traffic and the tile kernels
    // would occupy one workgroup per 64 features
    if (direct && m <= 32 && ksteps >= 16) return ROW_GEMV;
    if (ksteps <= 2 || !direct) {
        // one or two K-steps (or a first layer with three input features): bound by HBM bandwidth
        if (!direct && ksteps >= 3 && m >= 500000) return choose_lds_tile(p, m, cus);  // VGG conv1
        if (stream_fits) return stream_row;
        return choose_lds_tile(p, m, cus);
    }
    if (ksteps <= 8) {
        if (m >= 16384) return ROW_WSL_P64;                       // 1x1 reductions at 56x56 and 28x28
        if (m >= 4096) {
            if (p.OFM > 1024) return ROW_P64_F128;  // a 14x14 projection together with the block's opening 1x1
            if (p.OFM >= 512) return ksteps <= 4 ? ROW_WSL_P64 : ROW_BDIR_P128_F128;  // 14x14 expansions / projections
            return stream_fits ? stream_row : ROW_BDIR_P64_F64;
        }
        if (p.OFM >= 1024 && m >= 512) return ROW_P64_F128;       // 7x7 expansions; at a few hundred pixels 64-feature tiles give more workgroups
        return stream_fits ? stream_row : ROW_BDIR_P64_F64;
    }
    // long K
    if (m >= 50000) {
        // 256 and more features: 64 pixels x 128 features per wave, two waves per SIMD (3x3 at 56x56 with 128 / 256 input features)
        if (p.OFM >= 256 && p.OFM % 128 == 0) return ROW_BDIR_P256_F128;
        if (ksteps <= 18) return p.OFM <= 128 ? ROW_WSL_P128 : ROW_WSL_P64;  // 3x3 at 56x56 .. 224x224 with 64 / 128 input features
        return p.OFM >= 128 ? ROW_P256_F128 : ROW_BDIR_P256_F64;
    }
    const int64_t grid_p128_f64 = ((m + 127) / 128) * ((p.OFM + 63) / 64);
    if (m >= 8192) {
        if (p.OFM >= 512) {
            if (m >= 20000 && p.OFM % 128 == 0) return ROW_BDIR_P256_F128;  // 3x3 at 28x28 with a batch of 32
            return ksteps >= 64 ? ROW_BDIR_P128_F128 : ROW_BDIR_P256_F64;
        }
        if (ksteps <= 9 && m >= 32768) return ROW_WSL_P64;         // 64 input features under a 3x3 filter
        if (ksteps >= 32 && m >= 16384) return ROW_BDIR_P256_F64;  // 3x3 at 56x56 with 256 features and a small batch
        if (p.FY * p.FX > 1 && grid_p128_f64 <= cus) return ROW_BDIR_P64_F64;  // one workgroup per CU or fewer: halve the tile
        return ROW_BDIR_P128_F64;                                  // 3x3 at 28x28
    }
    if (m >= 4096) return p.OFM >= 512 && ksteps >= 64 ? ROW_BDIR_P128_F64 : ROW_BDIR_P64_F64;  // 14x14
    // few pixels, K >= 2048: split K; 128-pixel tiles when they still give three workgroups to every four CUs
    if (ksteps >= 32) return m >= 2048 && grid_p128_f64 * 4 >= 3ll * cus ? ROW_BDIR_K2_P128_F64 : ROW_BDIR_K2_P64_F64;
    if (p.OFM > 2048 && m >= 512) return ROW_P64_F128;  // a 7x7 projection together with the block's opening 1x1
    if (p.OFM >= 1024 && m >= 512) return ROW_P128_F128;
    return ROW_BDIR_P64_F64;
}

// look-ahead D of the weights-stationary kernel and the K-step count padded to a multiple of it:
// least padding first, then the deepest look-ahead
static void wsl_depth(int ksteps, int* depth, int* padded)
{
    static const int depths[] = {8, 6, 4, 3, 2, 1};
    int best_d = 1, best_pad = ksteps;
    for (int d : depths) {
        const int pad = (ksteps + d - 1) / d * d;
        if (pad < best_pad || (pad == best_pad && d > best_d)) best_pad = pad, best_d = d;
    }
    // one padded step in sixteen is cheaper than a shallow look-ahead
    for (int d : depths) {
        const int pad = (ksteps + d - 1) / d * d;
        if (d > best_d && (pad - ksteps) * 16 <= ksteps) {
            best_d = d, best_pad = pad;
            break;
        }
    }
    *depth = best_d, *padded = best_pad;
}

MfmaPlan mfma_plan(const ConvProblem& p, int tile, int cus)
{
    const TileConfig& tc = g_tiles[tile];
    MfmaPlan pl{};
    pl.tile = tile;
    pl.checked = border_covers(p) ? 0 : 1;
    pl.stem = tile == STEM_ROW || tile == STEM_P64_ROW ? 1 : 0;
    CHIP_REQUIRE(pl.stem == (p.in_t.format == CLDNN_HIP_FMT_B_FS_YX_FSV4 ? 1 : 0), CLDNN_HIP_INVALID_ARG,
                 "b_fs_yx_fsv4 input goes with the first-layer row of the tile table and only with it");
    pl.stream = (tile >= FIRST_STREAM_ROW && tile < FIRST_BDIR_ROW) || pl.stem ? 1 : 0;
    pl.gemv = tile == GEMV_ROW ? 1 : 0;
    pl.halo = tile >= FIRST_HALO_ROW ? 1 : 0;
    pl.block = 256;
    pl.bdir = ((tile >= FIRST_BDIR_ROW && tile < FIRST_WSL_ROW) || tile >= FIRST_BDIRK_ROW) && !pl.stem && !pl.gemv && !pl.halo ? 1 : 0;
    pl.wsl = tile >= FIRST_WSL_ROW && tile < FIRST_BDIRK_ROW ? 1 : 0;
    CHIP_REQUIRE(!(pl.stream && pl.checked), CLDNN_HIP_INVALID_ARG,
                 "the streaming kernel needs an input whose physical zero border covers the convolution's padding");
    pl.cb = (p.IFM + 15) / 16;
    if (pl.stem) CHIP_REQUIRE(p.IFM <= 4 && p.dx == 1 && p.groups == 1, CLDNN_HIP_INVALID_ARG,
                              "the first-layer kernel takes at most 4 input features and no horizontal dilation");
    CHIP_REQUIRE(!(pl.bdir || pl.wsl || pl.gemv || pl.halo) || (!pl.checked && pl.cb % 4 == 0), CLDNN_HIP_INVALID_ARG,
                 "the direct-activation kernels need a zero border covering the padding and input features in multiples of 64");
    pl.kchunks = pl.stem ? p.FY * ((p.FX + 3) / 4) : p.FY * p.FX * pl.cb;  // first layer: a chunk is 4 horizontal taps
    pl.ksteps = (pl.kchunks + 3) / 4;
    if (pl.stream) {
        CHIP_REQUIRE(pl.ksteps <= 8, CLDNN_HIP_INVALID_ARG, "the streaming kernel handles at most 8 K-steps (K <= 512)");
        int ks = 1;
        while (ks < pl.ksteps) ks *= 2;  // compile-time K-step counts: 1, 2, 4, 8 (zero-weight padding chunks)
        pl.ksteps = ks;
    }
    if (tc.kgroups > 1) pl.ksteps = (pl.ksteps + tc.kgroups - 1) / tc.kgroups * tc.kgroups;  // zero-weight padding steps
    if (pl.wsl) {
        wsl_depth(pl.ksteps, &pl.wsl_depth, &pl.ksteps);
        CHIP_REQUIRE(pl.ksteps * 4096 <= WSL_MAX_LDS, CLDNN_HIP_INVALID_ARG,
                     "the weights-stationary kernel holds 64 x K weight bytes in LDS: K is limited to 2560");
    }
    // K order.  With the taps innermost, consecutive K-steps of a wave read the same cache lines of the input shifted
    // by one pixel (or one row), so most activation loads of a 3x3 filter hit in the CU's L1 instead of going to L2.
    // The weights-stationary and streaming kernels walk the taps with counters in (tap, slice) order.
    pl.tap_minor = !pl.stream && !pl.wsl && pl.cb % 4 == 0 && p.FY * p.FX > 1 ? 1 : 0;
    if (pl.halo) {
        const cldnn_hip_tensor& t = p.in_t;
        CHIP_REQUIRE(p.FY * p.FX == HALO_TAPS && p.sy == 1 && p.sx == 1 && p.groups == 1, CLDNN_HIP_INVALID_ARG,
                     "the staged-patch kernel takes nine-tap filters at stride 1");
        CHIP_REQUIRE(t.pad_lo_b == 0 && t.pad_hi_b == 0, CLDNN_HIP_INVALID_ARG, "the staged-patch kernel takes no batch padding");
        const int wp = t.x + t.pad_lo_x + t.pad_hi_x, hp = t.y + t.pad_lo_y + t.pad_hi_y;
        const int64_t pos_total = (int64_t)p.B * hp * wp;
        const int halo_lo = p.py * wp + p.px;
        const int halo_hi = ((p.FY - 1) * p.dy - p.py) * wp + ((p.FX - 1) * p.dx - p.px);
        CHIP_REQUIRE(halo_lo >= 0 && halo_hi >= 0, CLDNN_HIP_INVALID_ARG, "the staged-patch kernel needs taps on both sides of the anchor");
        const int waves = (tc.tile_pixels / 64) * (tc.tile_ofm / 128);
        pl.block = waves * 64;
        pl.halo_patch_len = (tc.tile_pixels + halo_lo + halo_hi + 63) / 64 * 64;
        pl.halo_ptiles = (int)((pos_total + tc.tile_pixels - 1) / tc.tile_pixels);
        // the next block's patch is requested in five steps of the current one, by every wave
        const int slots = (HALO_TAPS - HALO_RING) * waves;
        pl.halo_pl = (4 * (pl.halo_patch_len / 64) + slots - 1) / slots;
        CHIP_REQUIRE(pl.halo_pl <= 2, CLDNN_HIP_UNSUPPORTED_SIZE, "rows too long for the staged-patch kernel's request slots");
    }
    pl.ofm_tiles = (p.OFM + tc.tile_ofm - 1) / tc.tile_ofm;
    pl.m_total = (int64_t)p.B * p.OH * p.OW;
    // every 16 pixels stream all the weights again (and take 1 KB of scratch per K-step when gathered)
    CHIP_REQUIRE(!pl.gemv || pl.m_total <= 4096, CLDNN_HIP_INVALID_ARG, "the small-batch kernel takes at most 4096 output pixels");
    CHIP_REQUIRE(pl.m_total < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "more than 2^31 output pixels");
    pl.mtiles = (int)((pl.m_total + tc.tile_pixels - 1) / tc.tile_pixels);
    if (pl.halo) pl.mtiles = pl.halo_ptiles;
    // which operand do the eight dies share out?  the larger one (it is then read from memory once, not 8 times)
    const int64_t w_bytes = (int64_t)p.OFM * (p.IFM / p.groups) * p.FY * p.FX, in_bytes = (int64_t)p.B * p.IFM * p.IH * p.IW;
    pl.by_features = !pl.stream && !pl.wsl && !pl.gemv && !pl.halo && w_bytes > in_bytes && (p.OFM + tc.tile_ofm - 1) / tc.tile_ofm >= 8 ? 1 : 0;
    int64_t grid = pl.by_features ? (int64_t)((pl.ofm_tiles + 7) / 8) * 8 * pl.mtiles : (int64_t)((pl.mtiles + 7) / 8) * 8 * pl.ofm_tiles;
    if (pl.stream) grid = ((int64_t)pl.mtiles * pl.ofm_tiles + 3) / 4;  // one wave per (pixel tile, span)
    pl.lds_bytes = pl.stream ? 0 : (pl.bdir ? 3 * 4 * tc.tile_ofm * 16 : 2 * 4 * (tc.tile_ofm + tc.tile_pixels) * 16);
    if (tc.kgroups > 1)  // per-group weight buffers, later reused for the partial sums of groups 1..
        pl.lds_bytes = std::max(tc.kgroups * pl.lds_bytes, (tc.kgroups - 1) * (tc.tile_ofm / 16) * (tc.wave_pixels / 16) * 4096);
    if (pl.wsl) {
        // persistent workgroups: as many as the chip holds at once, by LDS and by registers (16 pixels per wave: 118-168
        // registers = three waves per SIMD; 32 and 64 pixels per wave: two), split evenly over the feature tiles;
        // partitions come in eights (one per accelerator die)
        pl.lds_bytes = pl.ksteps * 4096;
        const int by_regs = tc.wave_pixels == 16 ? 3 : 2;
        const int per_cu = std::max(1, std::min(by_regs, (int)WSL_MAX_LDS / pl.lds_bytes));
        int parts = std::max(8, cus * per_cu / pl.ofm_tiles / 8 * 8);
        pl.wsl_tpp = (pl.mtiles + parts - 1) / parts;
        parts = ((pl.mtiles + pl.wsl_tpp - 1) / pl.wsl_tpp + 7) / 8 * 8;
        pl.wsl_parts = parts;
        grid = (int64_t)parts * pl.ofm_tiles;
    }
    if (pl.halo) {
        pl.lds_bytes = (HALO_RING * 4 * tc.tile_ofm + 2 * 4 * pl.halo_patch_len) * 16;
        CHIP_REQUIRE(pl.lds_bytes <= WSL_MAX_LDS, CLDNN_HIP_UNSUPPORTED_SIZE, "rows too long for the staged-patch kernel's LDS");
        // persistent workgroups: as many as the chip holds at once (two waves per SIMD by registers), split evenly over
        // the feature tiles; partitions come in eights (one contiguous run of position tiles per die)
        const int by_lds = WSL_MAX_LDS / pl.lds_bytes, by_regs = 8 / (pl.block / 64);
        const int per_cu = std::max(1, std::min(by_lds, by_regs));
        int parts = std::max(8, cus * per_cu / pl.ofm_tiles / 8 * 8);
        parts = std::min(parts, (pl.halo_ptiles + 7) / 8 * 8);
        pl.halo_parts = parts;
        grid = (int64_t)parts * pl.ofm_tiles;
    }
    if (pl.gemv) {
        // one workgroup per 16-feature fragment and 16 pixels; 4, 8 or 16 waves split K, at least eight steps (one
        // look-ahead window) each
        grid = (int64_t)pl.mtiles * pl.ofm_tiles * 4;
        pl.gemv_waves = pl.ksteps >= 128 ? 16 : (pl.ksteps >= 64 ? 8 : 4);
        pl.lds_bytes = 16 * 1024;
    }
    CHIP_REQUIRE(grid < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "convolution too large for one launch");
    pl.grid = (int)grid;
    // the tile kernel requests operands up to MFMA_SLACK_STEPS K-steps past the end (zero weights there)
    pl.packed_bytes = ((size_t)pl.ofm_tiles * pl.ksteps + MFMA_SLACK_STEPS) * 4 * tc.tile_ofm * 16;
    pl.ktab_bytes = (size_t)(pl.ksteps + MFMA_SLACK_STEPS) * 4 * sizeof(int32_t);
    CHIP_REQUIRE((p.FY - 1) * p.dy < 1024 && (p.FX - 1) * p.dx < 1024 && pl.cb < 2048, CLDNN_HIP_UNSUPPORTED_SIZE,
                 "filter extent or feature count beyond the tap table encoding");
    // 32-bit offsets inside the kernel
    CHIP_REQUIRE(tensor_elems(p.in_t) < (1ull << 31) && tensor_elems(p.out_t) * dtype_size(p.out_dt) < (1ull << 31),
                 CLDNN_HIP_UNSUPPORTED_SIZE, "tensor of 2 GiB or more");
    return pl;
}

void mfma_pack_weights(const ConvProblem& p, const MfmaPlan& pl, const int8_t* w, int8_t* packed, int32_t* ktab)
{
    const TileConfig& tc = g_tiles[pl.tile];
    const int BN = tc.tile_ofm;
    std::memset(packed, 0, pl.packed_bytes);
    auto row_of = [&](int f) {
        const int fl = f % BN, span = fl / 64, o = fl % 64;
        if (pl.halo) {
            // 32-row tiles of the 32x32x32 matrix instruction: row 8g + 4h + i holds feature 16h + 4g + i of the tile
            const int tile = fl / 32, q = fl % 32;
            return tile * 32 + ((q % 16) / 4) * 8 + (q / 16) * 4 + (q % 4);
        }
        return span * 64 + ((o % 16) / 4) * 16 + (o / 16) * 4 + (o % 4);  // permuted row inside the span
    };
    if (pl.stem) {
        // k-chunk = (filter row, group of 4 horizontal taps); byte = (tap in group) * 4 + feature; absent taps / features stay zero
        const int fxg = (p.FX + 3) / 4;
        for (int kc = 0; kc < (pl.ksteps + MFMA_SLACK_STEPS) * 4; ++kc) ktab[kc] = 0;  // offsets are computed in the kernel
        for (int f = 0; f < p.OFM; ++f)
            for (int fy = 0; fy < p.FY; ++fy)
                for (int fx = 0; fx < p.FX; ++fx)
                    for (int ch = 0; ch < p.IFM; ++ch) {
                        const int kc = fy * fxg + fx / 4, ks = kc / 4, kq = kc % 4;
                        packed[((((size_t)(f / BN) * pl.ksteps + ks) * 4 + kq) * BN + row_of(f)) * 16 + (fx % 4) * 4 + ch] =
                            w[(((size_t)f * p.IFM + ch) * p.FY + fy) * p.FX + fx];
                    }
        return;
    }
    // k-chunk -> (tap, feature slice): tap-major with the slices innermost, or groups of 4 slices with the taps innermost
    const int taps = p.FY * p.FX;
    auto chunk_tap = [&](int kc) { return pl.tap_minor ? (kc / 4) % taps : kc / pl.cb; };
    auto chunk_slice = [&](int kc) { return pl.tap_minor ? (kc / 4) / taps * 4 + kc % 4 : kc % pl.cb; };
    for (int kc = 0; kc < (pl.ksteps + MFMA_SLACK_STEPS) * 4; ++kc) {
        if (kc >= pl.kchunks) {
            ktab[kc] = pl.checked ? (int32_t)0x80000000 : 0;  // padding chunk: zero weights
            continue;
        }
        const int tap = chunk_tap(kc), cb = chunk_slice(kc);
        const int fyd = (tap / p.FX) * p.dy, fxd = (tap % p.FX) * p.dx;
        if (pl.checked) ktab[kc] = fyd | (fxd << 10) | (cb << 20);
        else ktab[kc] = (int32_t)(cb * p.in_p.pf + fyd * p.in_p.py + fxd * 16);
    }
    for (int f = 0; f < p.OFM; ++f) {
        const int nt = f / BN;
        const int row = row_of(f);
        for (int kc = 0; kc < pl.kchunks; ++kc) {
            const int tap = chunk_tap(kc), cb = chunk_slice(kc);
            const int ks = kc / 4, kq = kc % 4;
            int8_t* dst = packed + ((((size_t)nt * pl.ksteps + ks) * 4 + kq) * BN + row) * 16;
            for (int c = 0; c < 16; ++c) {
                const int ch = cb * 16 + c;
                if (ch < p.IFM) dst[c] = w[((size_t)f * p.IFM + ch) * p.FY * p.FX + tap];
            }
        }
    }
}

static bool tame(const float* v, int n)
{
    for (int i = 0; i < n; ++i)
        if (!(std::fabs(v[i]) < 1.0e9f)) return false;  // also rejects NaN
    return true;
}

// Can the short epilogue reproduce the long one bit for bit?  Decided once per convolution.
bool mfma_fast_epilogue(const ConvProblem& p, const Epilogue& e, const float* calib, const float* ecal, const float* wqf,
                        FastEpi* out)
{
    FastEpi F{};
    if (e.mode != MODE_Q || e.round_even) return false;
    if (e.fc) {
        // the fully_connected form has a short version for a float bias and no / relu activation
        if (!e.bias || e.bias_dt != CLDNN_HIP_F32 || e.fused || e.out_dt != CLDNN_HIP_S8) return false;
        if (!(e.act == CLDNN_HIP_ACT_NONE || e.act == CLDNN_HIP_ACT_RELU)) return false;
        F.fc = 1;
    } else if (e.bias) {
        return false;  // an int32 bias is folded into the accumulator start; a float bias takes the long path
    }
    if (!(e.out_dt == CLDNN_HIP_S8 || e.out_dt == CLDNN_HIP_U8)) return false;
    if (e.split_f > 0) {
        // Two convolutions in one launch: only the branch-free clamp form is written for it.  It needs per-feature
        // output factors that are finite (and not negative where a relu is folded into the clamp), unit weight factors,
        // and none / relu on both sides.
        auto plain = [](int act) { return act == CLDNN_HIP_ACT_NONE || act == CLDNN_HIP_ACT_RELU; };
        if (e.fc || e.fused || !calib || !plain(e.act) || !plain(e.act2) || !tame(calib, p.OFM)) return false;
        if (e.iqf != 1.0f) return false;
        if (wqf)
            for (int f = 0; f < p.OFM; ++f)
                if (wqf[f] != 1.0f) return false;
        for (int f = 0; f < p.OFM; ++f)
            if ((f < e.split_f ? e.act : e.act2) == CLDNN_HIP_ACT_RELU && !(calib[f] >= 0.0f)) return false;
        F.hi = e.out_dt == CLDNN_HIP_S8 ? 127.0f : 255.0f;
        const float type_lo = e.out_dt == CLDNN_HIP_S8 ? -128.0f : 0.0f;
        F.lo = e.act == CLDNN_HIP_ACT_RELU ? 0.0f : type_lo;
        F.lo2 = e.act2 == CLDNN_HIP_ACT_RELU ? 0.0f : type_lo;
        F.split_valid = p.OFM - e.split_f;
        F.act = CLDNN_HIP_ACT_NONE;  // what is left of the activations is in the bounds
        F.iqf = 1.0f, F.iqf_one = 1;
        *out = F;
        return true;
    }
    if (!(e.act == CLDNN_HIP_ACT_NONE || e.act == CLDNN_HIP_ACT_RELU || e.act == CLDNN_HIP_ACT_CLAMP)) return false;
    if (e.act == CLDNN_HIP_ACT_CLAMP && !(e.act_m <= e.act_n)) return false;  // the median form needs ordered bounds
    // factors small enough that no product can overflow into inf * 0
    if (calib && !tame(calib, p.OFM)) return false;
    if (ecal && !tame(ecal, p.OFM)) return false;
    if (wqf && !tame(wqf, p.OFM)) return false;
    if (!tame(&e.iqf, 1) || !tame(&e.oqf, 1) || !tame(&e.act_m, 1) || !tame(&e.act_n, 1)) return false;
    F.lo = e.out_dt == CLDNN_HIP_S8 ? -128.0f : 0.0f;
    F.hi = e.out_dt == CLDNN_HIP_S8 ? 127.0f : 255.0f;
    F.iqf = e.iqf;
    F.act = e.act, F.act_m = e.act_m, F.act_n = e.act_n;
    F.has_wqf = 0;
    if (wqf) {
        bool unit = e.iqf == 1.0f;
        for (int f = 0; f < p.OFM && unit; ++f) unit = wqf[f] == 1.0f;
        F.has_wqf = unit ? 0 : 1;  // x * 1.0f * 1.0f == x
    }
    F.fused = e.fused;
    if (e.fused) {
        if (e.ncs_on) return false;
        if (!(e.eltw_dt == CLDNN_HIP_S8 || e.eltw_dt == CLDNN_HIP_U8) || p.eltw_p.fsv != 16) return false;
        if (!(e.eltw_act == CLDNN_HIP_ACT_NONE || e.eltw_act == CLDNN_HIP_ACT_RELU || e.eltw_act == CLDNN_HIP_ACT_CLAMP))
            return false;
        if (!tame(&e.eltw_m, 1) || !tame(&e.eltw_n, 1)) return false;
        F.eltw_act = e.eltw_act, F.eltw_m = e.eltw_m, F.eltw_n = e.eltw_n;
        F.conv_sat = e.conv_sat ? 1 : 0;
        F.conv_lo = e.conv_sat == 1 ? -128.0f : 0.0f, F.conv_hi = e.conv_sat == 1 ? 127.0f : 255.0f;
        F.has_ecal = ecal ? 1 : 0;
        F.eltw_u8 = e.eltw_dt == CLDNN_HIP_U8;
        if (e.eltw_act == CLDNN_HIP_ACT_CLAMP && !(e.eltw_m <= e.eltw_n)) return false;
        if (e.eltw_act == CLDNN_HIP_ACT_RELU) {
            bool nonneg = true;
            if (ecal)
                for (int f = 0; f < p.OFM && nonneg; ++f) nonneg = ecal[f] >= 0.0f;
            F.eltw_relu_folded = nonneg ? 1 : 0;
        }
    } else if (e.act == CLDNN_HIP_ACT_RELU) {
        bool nonneg = true;
        if (calib)
            for (int f = 0; f < p.OFM && nonneg; ++f) nonneg = calib[f] >= 0.0f;
        else if (e.oqf_on) nonneg = e.oqf >= 0.0f;
        F.relu_folded = nonneg ? 1 : 0;
    } else if (e.act == CLDNN_HIP_ACT_CLAMP && !F.fc && e.act_m >= 0.0f) {
        // x in [m, n], factor >= 0: 0 <= x * factor <= n * factor (rounding is monotonic), so if n * factor is inside the
        // output range the second clamp does nothing and the value rounds like a non-negative number
        bool inside = true;
        auto ok = [&](float factor) { return factor >= 0.0f && e.act_n * factor <= F.hi; };
        if (calib)
            for (int f = 0; f < p.OFM && inside; ++f) inside = ok(calib[f]);
        else inside = ok(e.oqf_on ? e.oqf : 1.0f);
        F.clamp_folded = inside ? 1 : 0;
    }
    F.iqf_one = e.iqf == 1.0f ? 1 : 0;
    *out = F;
    return true;
}

// a filter of one tap puts the 16 pixels' bytes of a K-step side by side already
size_t mfma_gather_bytes(const ConvProblem& p, const MfmaPlan& pl)
{
    return pl.gemv && p.FY * p.FX > 1 ? gemv_gather_bytes(pl.mtiles, pl.ksteps) : 0;
}

size_t mfma_static_scratch_bytes() { return gemv_static_scratch_bytes(); }
void* mfma_static_scratch(int device) { return gemv_static_scratch(device); }

void launch_conv_mfma(hipStream_t s, const ConvProblem& p, const MfmaPlan& pl, const MfmaBuffers& wb,
                      const int32_t* acc_init, const Epilogue& epi, const FastEpi* fast, const void* in, const void* eltw,
                      void* out, int32_t* raw)
{
    const TileConfig& tc = g_tiles[pl.tile];
    MfmaArgs a{};
    a.in = (const int8_t*)in;
    a.wpk = (const v4i*)wb.packed;
    a.ktab = wb.ktab;
    a.acc_init = acc_init;
    a.out = out;
    a.eltw = eltw;
    a.raw = raw;
    a.M = (uint32_t)pl.m_total;
    a.OFM = p.OFM, a.ofm_tiles = pl.ofm_tiles, a.mtiles = pl.mtiles;
    a.OHW = p.OH * p.OW, a.OW = p.OW, a.OH = p.OH, a.IH = p.IH, a.IW = p.IW;
    a.div_ohw = make_div((uint32_t)a.OHW), a.div_ow = make_div((uint32_t)a.OW);
    a.div_mtiles = make_div((uint32_t)a.mtiles), a.div_ofm_tiles = make_div((uint32_t)a.ofm_tiles);
    a.sy = p.sy, a.sx = p.sx, a.py = p.py, a.px = p.px, a.esy = p.esy, a.esx = p.esx;
    a.in_off = (int32_t)p.in_p.off, a.in_pb = (int32_t)p.in_p.pb, a.in_pf = (int32_t)p.in_p.pf, a.in_py = (int32_t)p.in_p.py;
    a.out_off = (int32_t)p.out_p.off, a.out_pb = (int32_t)p.out_p.pb, a.out_pf = (int32_t)p.out_p.pf;
    a.out_py = (int32_t)p.out_p.py;
    a.el_off = (int32_t)p.eltw_p.off, a.el_pb = (int32_t)p.eltw_p.pb, a.el_pf = (int32_t)p.eltw_p.pf;
    a.el_py = (int32_t)p.eltw_p.py;
    a.ksteps = pl.ksteps;
    a.CB = pl.cb, a.FX = p.FX, a.kchunks = pl.kchunks;
    a.tap_dy = p.dy * (int32_t)p.in_p.py, a.tap_dx = p.dx * 16;
    a.div_cb = make_div((uint32_t)pl.cb), a.div_fx = make_div((uint32_t)p.FX);
    a.wsl_parts = pl.wsl_parts, a.wsl_tpp = pl.wsl_tpp, a.FY = p.FY;
    a.by_features = pl.by_features;
    a.px_bytes = 16;
    if (pl.stem) {
        // the streaming kernel's tap arithmetic with "taps" = groups of 4 horizontal taps, 16 bytes apart
        a.px_bytes = 4;
        a.CB = 1, a.FX = (p.FX + 3) / 4, a.kchunks = pl.kchunks;
        a.tap_dx = 16;
        a.div_cb = make_div(1u), a.div_fx = make_div((uint32_t)a.FX);
        a.linear = 0;
    }
    {
        // dense tensors and a 1x1 / stride-1 convolution: pixel m sits at byte m * 16 of every feature slice
        auto dense = [](const cldnn_hip_tensor& t) {
            return t.pad_lo_y == 0 && t.pad_lo_x == 0 && t.pad_hi_y == 0 && t.pad_hi_x == 0;
        };
        a.linear = !pl.stem && p.FY == 1 && p.FX == 1 && p.sy == 1 && p.sx == 1 && p.py == 0 && p.px == 0 && dense(p.in_t)
                   && dense(p.out_t) && p.out_dt != CLDNN_HIP_F32
                   && (!epi.fused || (dense(p.eltw_t) && p.esy == 1 && p.esx == 1 && p.eltw_t.y == p.OH && p.eltw_t.x == p.OW));
    }
    a.xor_mask = p.in_dt == CLDNN_HIP_U8 ? 0x80808080u : 0u;
    a.epi = epi;
    int kind = EPI_KIND_GENERIC;
    if (fast && !raw) {
        a.fe = *fast;
        kind = EPI_KIND_FAST;
        // the branch-free forms
        if (!fast->has_wqf && epi.calib && !fast->fc) {
            if (!fast->fused && fast->relu_folded) kind = EPI_KIND_RELU;
            if (!fast->fused && fast->act == CLDNN_HIP_ACT_NONE) kind = EPI_KIND_LINEAR;
            if (fast->fused && fast->act == CLDNN_HIP_ACT_NONE && fast->eltw_relu_folded && epi.eltw_calib && !fast->conv_sat)
                kind = EPI_KIND_FUSED;
        }
    }
    a.bpk = (const v4i*)wb.gather;
    if (pl.halo) {
        HaloArgs h{};
        h.m = a;
        const cldnn_hip_tensor& t = p.in_t;
        h.Wp = t.x + t.pad_lo_x + t.pad_hi_x;
        h.YXp = h.Wp * (t.y + t.pad_lo_y + t.pad_hi_y);
        h.pos_total = p.B * h.YXp;
        h.div_yxp = make_div((uint32_t)h.YXp), h.div_wp = make_div((uint32_t)h.Wp);
        h.pad_lo_y = t.pad_lo_y, h.pad_lo_x = t.pad_lo_x;
        h.halo_lo = p.py * h.Wp + p.px;
        h.patch_len = pl.halo_patch_len, h.cps = pl.halo_patch_len / 64;
        h.div_cps = make_div((uint32_t)h.cps);
        h.blocks = pl.cb / 4;
        h.ptiles = pl.halo_ptiles, h.parts = pl.halo_parts;
        h.tpp = pl.halo_ptiles / pl.halo_parts, h.trem = pl.halo_ptiles % pl.halo_parts;
        h.div_parts = make_div((uint32_t)pl.halo_parts);
        for (int k = 0; k < HALO_TAPS; ++k)
            h.tap[k] = h.halo_lo + ((k / p.FX) * p.dy - p.py) * h.Wp + ((k % p.FX) * p.dx - p.px);
        launch_halo(s, h, pl.tile - FIRST_HALO_ROW, pl.halo_pl, pl.grid, pl.lds_bytes, kind);
    }
    else if (pl.gemv) launch_gemv(s, a, pl.grid, pl.gemv_waves, pl.mtiles);  // element-wise epilogue only
    else if (pl.stream) launch_stream(s, a, tc.wave_pixels / 16, pl.grid, kind);
    else if (pl.bdir && tc.kgroups == 2) launch_bdir_k2(s, a, tc.wave_pixels / 16, pl.grid, pl.lds_bytes, kind);
    else if (pl.bdir && tc.kgroups == 4) launch_bdir_k4(s, a, tc.wave_pixels / 16, pl.grid, pl.lds_bytes, kind);
    else if (pl.bdir && tc.tile_ofm == 64) launch_bdir_f64(s, a, tc.wave_pixels / 16, pl.grid, pl.lds_bytes, kind);
    else if (pl.bdir) launch_bdir_f128(s, a, tc.wave_pixels / 16, pl.grid, pl.lds_bytes, kind);
    else if (pl.wsl) {
        const int nt = tc.wave_pixels / 16;
        switch (pl.wsl_depth) {
        case 1: launch_wsl_d1(s, a, nt, pl.grid, pl.lds_bytes, kind); break;
        case 2: launch_wsl_d2(s, a, nt, pl.grid, pl.lds_bytes, kind); break;
        case 3: launch_wsl_d3(s, a, nt, pl.grid, pl.lds_bytes, kind); break;
        case 4: launch_wsl_d4(s, a, nt, pl.grid, pl.lds_bytes, kind); break;
        case 6: launch_wsl_d6(s, a, nt, pl.grid, pl.lds_bytes, kind); break;
        default: launch_wsl_d8(s, a, nt, pl.grid, pl.lds_bytes, kind); break;
        }
    }
    else g_launch[pl.tile](s, a, pl.grid, pl.lds_bytes, pl.checked != 0, kind);
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
