// Dense 3x3 (nine-tap) stride-1 convolution with BOTH matrix operands staged in LDS by direct global->LDS loads.
//
// The direct-activation kernels fetch every activation fragment once per filter tap and every weight fragment once
// per wave.  Here a workgroup copies, per block of 64 input features, the contiguous stretch of the input that its
// output positions reach with any tap (the "patch": tile + halo) into LDS ONCE and reads all nine taps from there, so
// the activations cross the L2 -> CU path once instead of nine times; weights travel through an LDS ring shared by
// the waves of the workgroup.  Both copies are global_load_lds_dwordx4: no staging registers, so a wave keeps a
// 64 position x 128 feature tile (128 accumulators) with two waves per SIMD, and the look-ahead is bounded by LDS
// space, not by registers.
//
// Positions.  The input lies in fs_b_yx_fsv16 with a physical zero border that covers the padding: one feature slice
// is a contiguous array of B * Yp * Xp positions of 16 bytes (Yp, Xp: extents with border).  Output position q is
// the input position of the same index, so filter tap (fy, fx) is the constant distance
// (fy * dy - py) * Xp + (fx * dx - px) for every q, across rows and images.  Positions that fall on the border are
// computed (from whatever their taps reach) and not stored: 7 % of the matrix work at 56 x 56, 15 % at 28 x 28.
//
// Workgroups are persistent: each owns one tile of BN features and a contiguous run of position tiles and streams
// (tile, feature block) pairs without draining: the next pair's patch lands in the other patch buffer while the
// current one is multiplied, the weight ring never stops, and the requantisation of a finished tile overlaps the
// loads of the next.
#pragma once
#include <type_traits>

#include "conv_mfma_kernel.h"

namespace chip {

struct HaloArgs {
    MfmaArgs m;
    int32_t pos_total;         // B * Yp * Xp
    int32_t Wp, YXp;           // positions per padded row / padded image
    FastDiv div_yxp, div_wp;
    int32_t pad_lo_y, pad_lo_x;  // physical border in front of row 0 / column 0
    int32_t halo_lo;           // positions in front of a tile that its taps reach
    int32_t patch_len;         // positions per slice of a patch (multiple of 64)
    int32_t cps;               // patch_len / 64: wave-loads per slice
    FastDiv div_cps;
    int32_t blocks;            // blocks of 64 input features
    int32_t ptiles, parts;     // position tiles; workgroups per feature tile (multiple of 8)
    int32_t tap[9];            // halo_lo + distance of tap k, in positions (>= 0)
};

template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

typedef const __attribute__((address_space(1))) void* halo_gptr;
typedef __attribute__((address_space(3))) void* halo_lptr;

// MT x NT fragments per wave (16 features x 16 positions each), WP x WF waves per workgroup, R stages in the weight
// ring, PL patch wave-loads per wave in each of the first PSTEPS steps of a block.
template <int MT, int NT, int WP, int WF, int R, int PL, int EPI, int DBG = 0>
__global__ void __launch_bounds__(WP * WF * 64) conv_halo_kernel(HaloArgs h)
{
    constexpr int TAPS = 9;
    constexpr int LA = R - 2;                 // weight look-ahead in steps
    constexpr int PSTEPS = TAPS - 1 - LA;     // steps of a block that request patch chunks of the next block
    constexpr int WAVES = WP * WF;
    constexpr int BN = WF * MT * 16, BM = WP * NT * 16;
    constexpr int STAGE = 4 * BN;             // 16-byte units per ring stage
    constexpr int WL = STAGE / 64 / WAVES;    // weight wave-loads per wave and step
    constexpr int SPANS = MT / 4;
    constexpr int BAR_MT = MT - 3;            // the step's barrier sits behind this fragment row
    static_assert(WL * 64 * WAVES == STAGE && WL >= 1, "weight stage must split evenly over the waves");
    static_assert(MT % 4 == 0 && MT >= 4, "whole 64-feature spans per wave");
    const MfmaArgs& a = h.m;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave_p = wave % WP, wave_f = wave / WP;
    const int kq = lane >> 4, l16 = lane & 15;

    // Workgroup ids are dealt round-robin to the eight dies.  A die takes a contiguous eighth of the partitions with
    // all their feature tiles adjacent in time: neighbouring position tiles share their halos, feature tiles their
    // whole patch, through that die's L2.
    const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
    const int part = xcd * (h.parts >> 3) + jj / a.ofm_tiles;
    const int ntile = jj % a.ofm_tiles;
    const int t_begin = (int)((long long)part * h.ptiles / h.parts);
    const int t_end = (int)((long long)(part + 1) * h.ptiles / h.parts);
    if (t_begin >= t_end) return;

    extern __shared__ __align__(16) unsigned char smem[];
    v4i* ring = reinterpret_cast<v4i*>(smem);  // [R][STAGE]
    v4i* patch = ring + R * STAGE;             // [2][4 slices][patch_len]
    const int patch_v4 = 4 * h.patch_len;

    const int a_lane = kq * BN + wave_f * MT * 16 + l16;
    const int b_lane = kq * h.patch_len + wave_p * NT * 16 + l16;
    const v4i* wsrc = a.wpk + (size_t)ntile * a.ksteps * STAGE + wave * WL * 64 + lane;
    const v4i xm = {(int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask};

    auto issue_weights = [&](int ks, int stage) {
#pragma unroll
        for (int q = 0; q < WL; ++q)
            __builtin_amdgcn_global_load_lds((halo_gptr)(wsrc + (size_t)ks * STAGE + q * 64),
                                             (halo_lptr)(ring + stage * STAGE + (wave * WL + q) * 64), 16, 0, 0);
    };
    // chunk c of the patch of (position tile, feature block) -> buffer buf: 64 positions of one slice
    auto issue_patch = [&](int c, int tile, int cb, int buf) {
        c = min(c, 4 * h.cps - 1);  // spare request slots repeat the last chunk
        const int sl = (int)h.div_cps.div((uint32_t)c);
        const int i = c - sl * h.cps;
        int p = tile * BM - h.halo_lo + i * 64 + lane;
        p = min(max(p, 0), h.pos_total - 1);  // only positions that are never stored reach outside the tensor
        const int8_t* src = a.in + (size_t)(cb * 4 + sl) * (size_t)a.in_pf + (size_t)p * 16;
        __builtin_amdgcn_global_load_lds((halo_gptr)src, (halo_lptr)(patch + buf * patch_v4 + sl * h.patch_len + i * 64), 16, 0, 0);
    };

    v4i acc[MT][NT];
    auto reset_acc = [&]() {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int f = ntile * BN + ((wave_f * MT + mt) >> 2) * 64 + kq * 16 + (mt & 3) * 4;
            const v4i init = *reinterpret_cast<const v4i*>(a.acc_init + f);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = init;
        }
    };

    // ---- prologue: the first patch, the first LA + 1 weight stages
    for (int c = wave; c < 4 * h.cps; c += WAVES) issue_patch(c, t_begin, 0, 0);
    step_fence();
#pragma unroll
    for (int u = 0; u <= LA; ++u) issue_weights(u, u);
    step_fence();
    reset_acc();
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(LA * WL) : "memory");

    int rd_stage = 0;        // ring stage of the current step
    int wnext = LA + 1;      // K-step of the tile whose weights are requested next
    int pbuf = 0;            // patch buffer of the current block
    v4i fa[4], fb[NT], fbn[NT];
    {
        const v4i* st = ring + a_lane;
        const v4i* pt = patch + b_lane + h.tap[0];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) fbn[nt] = pt[nt * 16];
        fa[0] = st[0];
        fa[1] = st[16];
    }

    for (int tile = t_begin; tile < t_end; ++tile) {
        for (int cb = 0; cb < h.blocks; ++cb) {
            const bool last_cb = cb + 1 == h.blocks;
            const int cb_n = last_cb ? 0 : cb + 1;
            const int tile_n = last_cb ? tile + 1 : tile;
            static_for<0, TAPS>([&](auto ic) {
                constexpr int S = decltype(ic)::value;
                // loads younger than the weights of the next step when this step's barrier is reached
                constexpr int YOUNGER = [] {
                    int n = (LA - 1) * WL;
                    for (int i = 0; i < LA; ++i) n += ((S - LA + i + TAPS) % TAPS) < PSTEPS ? PL : 0;
                    return n;
                }();
                const v4i* st = ring + rd_stage * STAGE + a_lane;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) fb[nt] = fbn[nt] ^ xm;
                step_fence();
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    if (mt + 2 < MT) fa[(mt + 2) & 3] = st[(mt + 2) * 16];
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        acc[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[mt & 3], fb[nt], acc[mt][nt], 0, 0, 0);
                    step_fence();
                    if (mt == BAR_MT) {
                        // behind this barrier the next step's weights and (at a block's last step) the next patch are
                        // in LDS for every wave, and nobody reads the ring stage of the previous step any more
                        if constexpr (DBG & 1) { if constexpr (!(DBG & 2)) asm volatile("s_barrier" ::: "memory"); }
                        else if constexpr (DBG & 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(YOUNGER) : "memory");
                        else asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(YOUNGER) : "memory");
                        const int nx_stage = rd_stage + 1 == R ? 0 : rd_stage + 1;
                        const int wr_stage = rd_stage == 0 ? R - 1 : rd_stage - 1;
                        if constexpr (!(DBG & 4)) issue_weights(wnext, wr_stage);
                        wnext = wnext + 1 == a.ksteps ? 0 : wnext + 1;
                        if constexpr (S < PSTEPS && !(DBG & 8)) {
#pragma unroll
                            for (int i = 0; i < PL; ++i) issue_patch((S * WAVES + wave) * PL + i, tile_n, cb_n, pbuf ^ 1);
                        }
                        step_fence();
                        // first fragments of the next step
                        const int nbuf = S == TAPS - 1 ? pbuf ^ 1 : pbuf;
                        const v4i* pt = patch + nbuf * patch_v4 + b_lane + h.tap[(S + 1) % TAPS];
                        const v4i* sn = ring + nx_stage * STAGE + a_lane;
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt) fbn[nt] = pt[nt * 16];
                        fa[0] = sn[0];
                        fa[1] = sn[16];
                        step_fence();
                    }
                }
                rd_stage = rd_stage + 1 == R ? 0 : rd_stage + 1;
            });
            pbuf ^= 1;
        }

        // ---- requantise and store the tile: lane (kq, l16) holds 16 consecutive features of one position per fragment
        uint32_t ob[NT], eb[NT];
        PixelPos pos[NT];
        bool ok[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const uint32_t q = (uint32_t)tile * BM + (uint32_t)(wave_p * NT * 16 + nt * 16 + l16);
            const uint32_t b = h.div_yxp.div(q);
            const uint32_t r = q - b * (uint32_t)h.YXp;
            const uint32_t yp = h.div_wp.div(r);
            const int oy = (int)yp - h.pad_lo_y, ox = (int)(r - yp * (uint32_t)h.Wp) - h.pad_lo_x;
            ok[nt] = q < (uint32_t)h.pos_total && (uint32_t)oy < (uint32_t)a.OH && (uint32_t)ox < (uint32_t)a.OW;
            pos[nt] = PixelPos{b, (uint32_t)oy, (uint32_t)ox};
            ob[nt] = (uint32_t)(a.out_off + (int)b * a.out_pb + oy * a.out_py + ox * 16);
            eb[nt] = (uint32_t)(a.el_off + (int)b * a.el_pb + oy * a.esy * a.el_py + ox * a.esx * 16);
        }
#pragma unroll
        for (int sp = 0; sp < SPANS; ++sp) {
            const int f0 = ntile * BN + (wave_f * SPANS + sp) * 64 + kq * 16;
            if (f0 >= a.OFM) continue;
            const int fs = f0 >> 4;
            const int valid = a.OFM - f0;
            LaneScales sc;
            load_scales<EPI>(a, f0, sc);
            const v4i(&acc_sp)[4][NT] = *reinterpret_cast<const v4i(*)[4][NT]>(&acc[sp * 4]);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (ok[nt]) {
                    const int obase = (int)ob[nt] + fs * a.out_pf, ebase = (int)eb[nt] + fs * a.el_pf;
                    v4i ev4 = {0, 0, 0, 0};
                    if constexpr (EPI == EPI_KIND_FUSED) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
                    else if constexpr (EPI == EPI_KIND_FAST)
                        if (a.fe.fused) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
                    finish_pixel<NT, EPI>(a, acc_sp, nt, f0, valid, obase, ebase, sc, ev4, pos[nt].b, pos[nt].oy, pos[nt].ox);
                }
            }
        }
        reset_acc();
    }
    // requests past the end of the workgroup's work are still on their way into its LDS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int MT, int NT, int WP, int WF, int R, int PL, int DBG = 0>
void launch_halo_instance(hipStream_t s, const HaloArgs& h, int grid, int lds, int epi)
{
    const dim3 g(grid), b(WP * WF * 64);
#define HALO_LAUNCH(KIND)                                                                                           \
    {                                                                                                               \
        static std::once_flag allowed;                                                                              \
        std::call_once(allowed, [] {                                                                                \
            CHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_halo_kernel<MT, NT, WP, WF, R, PL, KIND, DBG>), \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));                \
        });                                                                                                         \
        hipLaunchKernelGGL((conv_halo_kernel<MT, NT, WP, WF, R, PL, KIND, DBG>), g, b, lds, s, h);                       \
    }
    switch (epi) {
    case EPI_KIND_RELU: HALO_LAUNCH(EPI_KIND_RELU) break;
    case EPI_KIND_FUSED: HALO_LAUNCH(EPI_KIND_FUSED) break;
    case EPI_KIND_LINEAR: HALO_LAUNCH(EPI_KIND_LINEAR) break;
    case EPI_KIND_FAST: HALO_LAUNCH(EPI_KIND_FAST) break;
    default: HALO_LAUNCH(EPI_KIND_GENERIC) break;
    }
#undef HALO_LAUNCH
}

}  // namespace chip
