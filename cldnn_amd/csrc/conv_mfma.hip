// Dense quantized convolution as an implicit GEMM on the gfx950 int8 matrix cores.
//
//   D[ofm][pixel] = sum_k W[ofm][k] * X[pixel][k],   k = (tap, input feature)
//
// computed with v_mfma_i32_16x16x64_i8: the A operand is a 16(ofm) x 64(k) weight tile, the
// B operand a 64(k) x 16(pixel) activation tile; every lane feeds 16 consecutive k bytes of one
// row / column, and that is exactly one 16-feature slice of one pixel in fs_b_yx_fsv16 memory
// (one 128-bit load, one 128-bit LDS read, no byte shuffling anywhere).
//
// Workgroup = 256 threads = 4 waves, output tile BM pixels x BN features; each wave owns
// 64 features x WP pixels.  Per K-step (4 k-chunks = 64 k values) the workgroup stages
// BN x 64 weight bytes and BM x 64 activation bytes in LDS (double buffered, one barrier
// per step).  Pixels are the linear index over (batch, oy, ox), so a tile may span rows and
// images; taps outside the image read as zero.
//
// u8 activations: the MFMA multiplies signed bytes, so activations are fed as (a ^ 0x80) = a - 128
// and the accumulators start from 128 * sum(w[f]) (+ the int32 bias), which is exact in int32.
//
// Weight rows are stored permuted inside each 64-feature span so that a lane's 16 accumulators
// of one pixel are 16 CONSECUTIVE features: the int8 result is written with one 128-bit store.
#include "epilogue.h"
#include "kernels.h"

#include <cstring>
#include <vector>

namespace chip {

typedef int v4i __attribute__((ext_vector_type(4)));

struct MfmaArgs {
    const int8_t* in;
    const int8_t* wpk;
    const int32_t* ktab;
    const int32_t* acc_init;  // [ofm_tiles * BN], natural feature order, zero padded
    void* out;
    const void* eltw;
    int32_t* raw;
    Pitch in_p, out_p, eltw_p;
    int B, IH, IW, OH, OW, OFM, OHW;
    int64_t M;
    int sy, sx, py, px, esy, esx;
    int ksteps;
    uint32_t xor_mask;  // 0x80808080 for u8 activations, 0 for s8
    Epilogue epi;
    // EPI_FAST parameters
    float fast_lo, fast_hi;
};

static const TileConfig g_tiles[] = {
    {"mfma_i8_p128_f128", 128, 128, 64},
    {"mfma_i8_p256_f64", 256, 64, 64},
    {"mfma_i8_p64_f128", 64, 128, 32},
    {"mfma_i8_p128_f64", 128, 64, 32},
    {"mfma_i8_p64_f64", 64, 64, 16},
    {"mfma_i8_p256_f128", 256, 128, 128},
};
int tile_config_count() { return (int)(sizeof(g_tiles) / sizeof(g_tiles[0])); }
const TileConfig& tile_config(int i) { return g_tiles[i]; }

// ktab entry: bits 0..9 = fy*dilation_y, 10..19 = fx*dilation_x, 20..30 = feature slice, bit 31 = padding chunk
__host__ __device__ inline int32_t ktab_pack(int fyd, int fxd, int cb) { return fyd | (fxd << 10) | (cb << 20); }

template <int BM, int BN, int WP, int EPI>
__global__ void __launch_bounds__(256) conv_mfma_kernel(MfmaArgs a)
{
    constexpr int NT = WP / 16;        // pixel tiles per wave
    constexpr int WAVES_F = BN / 64;   // waves along features
    constexpr int A_LOADS = BN / 64;   // 16-byte weight chunks per thread per K-step
    constexpr int B_LOADS = BM / 64;   // 16-byte activation chunks per thread per K-step
    constexpr int KC_STRIDE = 256 / BM;  // k-chunk distance between a thread's activation loads
    static_assert((BM / WP) * WAVES_F == 4, "tile must map onto 4 waves");

    extern __shared__ __align__(16) unsigned char smem[];
    v4i* ldsA = reinterpret_cast<v4i*>(smem);                 // [2][4 * BN]
    v4i* ldsB = reinterpret_cast<v4i*>(smem) + 2 * 4 * BN;    // [2][4 * BM]

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = t >> 6;
    const int wave_f = wave % WAVES_F;
    const int wave_p = wave / WAVES_F;

    // feature tiles vary fastest so that workgroups sharing activation pixels run together
    const int ofm_tiles = (a.OFM + BN - 1) / BN;
    const int ntile = blockIdx.x % ofm_tiles;
    const int64_t m0 = (int64_t)(blockIdx.x / ofm_tiles) * BM;

    // ---- this thread's activation pixel
    const int lp = t % BM;
    const int kc0 = t / BM;
    const int64_t m_ld = m0 + lp;
    const bool ld_valid = m_ld < a.M;
    int iy0, ix0;
    int64_t in_base;
    {
        const int64_t mm = ld_valid ? m_ld : 0;
        const int b = (int)(mm / a.OHW);
        const int r = (int)(mm % a.OHW);
        const int oy = r / a.OW, ox = r % a.OW;
        iy0 = oy * a.sy - a.py;
        ix0 = ox * a.sx - a.px;
        in_base = a.in_p.off + (int64_t)b * a.in_p.pb;
    }
    const v4i* wsrc = reinterpret_cast<const v4i*>(a.wpk) + (int64_t)ntile * a.ksteps * (4 * BN) + t;

    v4i ra[A_LOADS], rb[B_LOADS];

    auto load_global = [&](int ks) {
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) ra[j] = wsrc[(int64_t)ks * (4 * BN) + j * 256];
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) {
            const int kc = ks * 4 + kc0 + j * KC_STRIDE;
            const int e = a.ktab[kc];
            const int iy = iy0 + (e & 1023), ix = ix0 + ((e >> 10) & 1023);
            const int cb = (e >> 20) & 2047;
            const bool ok = ld_valid && e >= 0 && iy >= 0 && iy < a.IH && ix >= 0 && ix < a.IW;
            v4i v = {0, 0, 0, 0};
            if (ok) {
                const int64_t off = in_base + (int64_t)cb * a.in_p.pf + (int64_t)iy * a.in_p.py + (int64_t)ix * 16;
                v = *reinterpret_cast<const v4i*>(a.in + off);
            }
            rb[j] = v;
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) ldsA[buf * 4 * BN + t + j * 256] = ra[j];
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) ldsB[buf * 4 * BM + (kc0 + j * KC_STRIDE) * BM + lp] = rb[j];
    };

    // ---- accumulators start from the per-feature constant (u8 offset correction + int32 bias)
    v4i acc[4][NT];
    {
        const int g = lane >> 4;
        const int fbase = ntile * BN + wave_f * 64 + g * 16;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
            const v4i init = *reinterpret_cast<const v4i*>(a.acc_init + fbase + mt * 4);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = init;
        }
    }

    load_global(0);
    store_lds(0);
    __syncthreads();

    const int arow = wave_f * 64 + (lane & 15);
    const int bcol = wave_p * WP + (lane & 15);
    const int kq = lane >> 4;
    const v4i xm = {(int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask};

    for (int ks = 0; ks < a.ksteps; ++ks) {
        const int buf = ks & 1;
        if (ks + 1 < a.ksteps) load_global(ks + 1);

        v4i fa[4], fb[NT];
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) fa[mt] = ldsA[buf * 4 * BN + kq * BN + arow + mt * 16];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) fb[nt] = ldsB[buf * 4 * BM + kq * BM + bcol + nt * 16] ^ xm;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                acc[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[mt], fb[nt], acc[mt][nt], 0, 0, 0);

        if (ks + 1 < a.ksteps) store_lds(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane (g, col) holds, for each pixel tile, features fs*16 .. fs*16+15 of one pixel
    const int g = lane >> 4;
    const int f0 = ntile * BN + wave_f * 64 + g * 16;
    if (f0 >= a.OFM) return;
    const int fs = f0 >> 4;
    const Epilogue& e = a.epi;

#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int64_t m = m0 + wave_p * WP + nt * 16 + (lane & 15);
        if (m >= a.M) continue;
        const int b = (int)(m / a.OHW);
        const int r = (int)(m % a.OHW);
        const int oy = r / a.OW, ox = r % a.OW;

        if (EPI == EPI_RAW) {
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int f = f0 + mt * 4 + i;
                    if (f < a.OFM) a.raw[(((int64_t)b * a.OFM + f) * a.OH + oy) * a.OW + ox] = acc[mt][nt][i];
                }
            continue;
        }

        const int64_t obase = a.out_p.off + (int64_t)b * a.out_p.pb + (int64_t)fs * a.out_p.pf
                              + (int64_t)oy * a.out_p.py + (int64_t)ox * a.out_p.px;
        int64_t ebase = 0;
        if (e.fused)
            ebase = a.eltw_p.off + (int64_t)b * a.eltw_p.pb + (int64_t)fs * a.eltw_p.pf
                    + (int64_t)(oy * a.esy) * a.eltw_p.py + (int64_t)(ox * a.esx) * a.eltw_p.px;

        if (EPI == EPI_FAST) {
            // relu, non-negative per-feature scale, unit wqf/iqf, int8 output, optional int8 residual with
            // unit scale + relu: cvt, mul, clamp, +0.49999997 and truncate.
            // trunc(y + pred(0.5)) == round-half-away(y) for 0 <= y < 2^22.
            v4i ev4 = {0, 0, 0, 0};
            if (e.fused) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
            v4i packed;
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                const float4 cal = *reinterpret_cast<const float4*>(e.calib + f0 + mt * 4);
                const float cs[4] = {cal.x, cal.y, cal.z, cal.w};
                float4 ecal = {1.f, 1.f, 1.f, 1.f};
                if (e.fused && e.eltw_calib) ecal = *reinterpret_cast<const float4*>(e.eltw_calib + f0 + mt * 4);
                const float ecs[4] = {ecal.x, ecal.y, ecal.z, ecal.w};
                unsigned word = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float v = (float)acc[mt][nt][i] * cs[i];
                    int q;
                    if (!e.fused) {
                        v = fminf(fmaxf(v, 0.0f), a.fast_hi);
                        q = (int)(v + 0.49999997f);
                    } else {
                        // conv part: relu is absent in the fused form handled here (act == none):
                        // round half away on a signed value, then add the residual
                        float rr = truncf(v + copysignf(0.49999997f, v));
                        int ebyte = (int)(int8_t)((unsigned)ev4[mt] >> (8 * i));
                        if (e.eltw_dt == CLDNN_HIP_U8) ebyte &= 255;
                        float s = rr + (float)ebyte;
                        s = fmaxf(s, 0.0f) * ecs[i];
                        s = fminf(fmaxf(s, a.fast_lo), a.fast_hi);
                        q = (int)(s + copysignf(0.49999997f, s));
                    }
                    word |= ((unsigned)q & 255u) << (8 * i);
                }
                packed[mt] = (int)word;
            }
            *reinterpret_cast<v4i*>((int8_t*)a.out + obase) = packed;
            continue;
        }

        // generic epilogue
        const bool out8 = e.out_dt == CLDNN_HIP_S8 || e.out_dt == CLDNN_HIP_U8;
        v4i packed = {0, 0, 0, 0};
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int ci = mt * 4 + i;
                const int f = f0 + ci;
                EpiOut o;
                o.f = 0.f, o.i = 0;
                if (f < a.OFM) {
                    float ev = 0.f;
                    if (e.fused) ev = load_as_float(a.eltw, e.eltw_dt, ebase + ci);
                    o = epilogue_generic(e, acc[mt][nt][i], f, ev);
                }
                if (out8) packed[mt] |= (int)(((unsigned)o.i & 255u) << (8 * i));
                else store_out(a.out, e.out_dt, obase + ci, o);
            }
        if (out8) *reinterpret_cast<v4i*>((int8_t*)a.out + obase) = packed;
    }
}

// ------------------------------------------------------------------------------------------ host side
MfmaPlan mfma_plan(const ConvProblem& p, int tile)
{
    const TileConfig& tc = g_tiles[tile];
    MfmaPlan pl{};
    pl.tile = tile;
    pl.cb = (p.IFM + 15) / 16;
    pl.kchunks = p.FY * p.FX * pl.cb;
    pl.ksteps = (pl.kchunks + 3) / 4;
    pl.ofm_tiles = (p.OFM + tc.tile_ofm - 1) / tc.tile_ofm;
    pl.m_total = (int64_t)p.B * p.OH * p.OW;
    const int64_t mtiles = (pl.m_total + tc.tile_pixels - 1) / tc.tile_pixels;
    const int64_t grid = mtiles * pl.ofm_tiles;
    CHIP_REQUIRE(grid < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "convolution too large for one launch");
    pl.grid = (int)grid;
    pl.lds_bytes = 2 * 4 * (tc.tile_ofm + tc.tile_pixels) * 16;
    pl.packed_bytes = (size_t)pl.ofm_tiles * pl.ksteps * 4 * tc.tile_ofm * 16;
    pl.ktab_bytes = (size_t)pl.ksteps * 4 * sizeof(int32_t);
    CHIP_REQUIRE((p.FY - 1) * p.dy < 1024 && (p.FX - 1) * p.dx < 1024 && pl.cb < 2048, CLDNN_HIP_UNSUPPORTED_SIZE,
                 "filter extent or feature count beyond the tap table encoding");
    return pl;
}

void mfma_pack_weights(const ConvProblem& p, const MfmaPlan& pl, const int8_t* w, int8_t* packed, int32_t* ktab)
{
    const TileConfig& tc = g_tiles[pl.tile];
    const int BN = tc.tile_ofm;
    std::memset(packed, 0, pl.packed_bytes);
    // k-chunk order: tap-major, feature slice minor
    for (int kc = 0; kc < pl.ksteps * 4; ++kc) {
        if (kc >= pl.kchunks) {
            ktab[kc] = (int32_t)0x80000000;
            continue;
        }
        const int tap = kc / pl.cb, cb = kc % pl.cb;
        ktab[kc] = ktab_pack((tap / p.FX) * p.dy, (tap % p.FX) * p.dx, cb);
    }
    for (int f = 0; f < p.OFM; ++f) {
        const int nt = f / BN, fl = f % BN;
        const int span = fl / 64, o = fl % 64;
        const int row = span * 64 + ((o % 16) / 4) * 16 + (o / 16) * 4 + (o % 4);  // permuted row inside the span
        for (int kc = 0; kc < pl.kchunks; ++kc) {
            const int tap = kc / pl.cb, cb = kc % pl.cb;
            const int ks = kc / 4, kq = kc % 4;
            int8_t* dst = packed + ((((size_t)nt * pl.ksteps + ks) * 4 + kq) * BN + row) * 16;
            for (int c = 0; c < 16; ++c) {
                const int ch = cb * 16 + c;
                if (ch < p.IFM) dst[c] = w[((size_t)f * p.IFM + ch) * p.FY * p.FX + tap];
            }
        }
    }
}

template <int BM, int BN, int WP>
static void launch_tile(hipStream_t s, const MfmaArgs& a, int grid, int lds, int epi)
{
    switch (epi) {
    case EPI_RAW:
        hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WP, EPI_RAW>), dim3(grid), dim3(256), lds, s, a);
        break;
    case EPI_FAST:
        hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WP, EPI_FAST>), dim3(grid), dim3(256), lds, s, a);
        break;
    default:
        hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WP, EPI_GENERIC>), dim3(grid), dim3(256), lds, s, a);
        break;
    }
}

// Can the short epilogue reproduce the generic one bit for bit?  (decided per convolution at creation)
bool mfma_fast_epilogue_ok(const ConvProblem& p, const Epilogue& e, const float* calib_host, const float* ecal_host,
                           const float* wqf_host, int ofm)
{
    if (e.mode != MODE_Q || e.round_even) return false;
    if (e.bias) return false;  // int32 bias is folded into the accumulator start; a float bias needs the long path
    if (!(e.out_dt == CLDNN_HIP_S8 || e.out_dt == CLDNN_HIP_U8)) return false;
    if (!calib_host) return false;
    if (e.iqf != 1.0f) return false;
    if (wqf_host)
        for (int f = 0; f < ofm; ++f)
            if (wqf_host[f] != 1.0f) return false;
    for (int f = 0; f < ofm; ++f)
        if (!(calib_host[f] >= 0.0f) || !(calib_host[f] < 3.0e38f)) return false;
    if (!e.fused) return e.act == CLDNN_HIP_ACT_RELU;
    // fused: conv result without activation, int8 residual with unit scale, relu, optional non-negative scale
    if (e.act != CLDNN_HIP_ACT_NONE || e.eltw_act != CLDNN_HIP_ACT_RELU || e.ncs_on) return false;
    if (!(e.eltw_dt == CLDNN_HIP_S8 || e.eltw_dt == CLDNN_HIP_U8)) return false;
    if (p.eltw_p.fsv != 16 || p.esy != 1 || p.esx != 1) return false;
    if (ecal_host)
        for (int f = 0; f < ofm; ++f)
            if (!(ecal_host[f] >= 0.0f) || !(ecal_host[f] < 3.0e38f)) return false;
    return true;
}

void launch_conv_mfma(hipStream_t s, const ConvProblem& p, const MfmaPlan& pl, const MfmaBuffers& wb,
                         const int32_t* acc_init, const Epilogue& epi, int epi_kind, const void* in, const void* eltw,
                         void* out, int32_t* raw)
{
    const TileConfig& tc = g_tiles[pl.tile];
    MfmaArgs a{};
    a.in = (const int8_t*)in;
    a.wpk = wb.packed;
    a.ktab = wb.ktab;
    a.acc_init = acc_init;
    a.out = out;
    a.eltw = eltw;
    a.raw = raw;
    a.in_p = p.in_p, a.out_p = p.out_p, a.eltw_p = p.eltw_p;
    a.B = p.B, a.IH = p.IH, a.IW = p.IW, a.OH = p.OH, a.OW = p.OW, a.OFM = p.OFM, a.OHW = p.OH * p.OW;
    a.M = pl.m_total;
    a.sy = p.sy, a.sx = p.sx, a.py = p.py, a.px = p.px, a.esy = p.esy, a.esx = p.esx;
    a.ksteps = pl.ksteps;
    a.xor_mask = p.in_dt == CLDNN_HIP_U8 ? 0x80808080u : 0u;
    a.epi = epi;
    a.fast_lo = epi.out_dt == CLDNN_HIP_S8 ? -128.0f : 0.0f;
    a.fast_hi = epi.out_dt == CLDNN_HIP_S8 ? 127.0f : 255.0f;
    const int g = pl.grid, l = pl.lds_bytes;
    if (tc.tile_pixels == 128 && tc.tile_ofm == 128) launch_tile<128, 128, 64>(s, a, g, l, epi_kind);
    else if (tc.tile_pixels == 256 && tc.tile_ofm == 64) launch_tile<256, 64, 64>(s, a, g, l, epi_kind);
    else if (tc.tile_pixels == 64 && tc.tile_ofm == 128) launch_tile<64, 128, 32>(s, a, g, l, epi_kind);
    else if (tc.tile_pixels == 128 && tc.tile_ofm == 64) launch_tile<128, 64, 32>(s, a, g, l, epi_kind);
    else if (tc.tile_pixels == 64 && tc.tile_ofm == 64) launch_tile<64, 64, 16>(s, a, g, l, epi_kind);
    else if (tc.tile_pixels == 256 && tc.tile_ofm == 128) launch_tile<256, 128, 128>(s, a, g, l, epi_kind);
    else throw error(CLDNN_HIP_ERROR, "tile configuration without a kernel instance");
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
