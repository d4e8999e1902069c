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
//
// Measured on VGG-16's layers at batch 16 and 32, this kernel is within 5 % of the best other row of the tile table on
// every layer and better than it on none by more than the noise: its loop keeps the matrix pipe 70-75 % busy, but a launch
// of such a layer spends about 12 us outside the loop (launch, start skew, prologue, a 3.6 us epilogue of 128 outputs
// per lane, and a last round of tiles that is four fifths full).  The built-in table therefore never selects its rows;
// a tuning cache or tile_override may.
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
    int32_t tpp, trem;         // ptiles / parts and the remainder
    FastDiv div_parts;         // partition p starts at tile p * tpp + (p * trem) / parts = floor(p * ptiles / parts)
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

typedef int v16i __attribute__((ext_vector_type(16)));

// LDS read issued behind the compiler's back: the destination register is written when the data arrives, which the caller
// establishes with lds_wait (LDS reads of a wave return in order, so a count of younger reads names the one waited for)
template <int OFFSET>
__device__ __forceinline__ void lds_read(v4i& dst, uint32_t byte_address)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(byte_address), "n"(OFFSET));
}
template <int YOUNGER>
__device__ __forceinline__ void lds_wait(v4i& needed)
{
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(needed) : "n"(YOUNGER));
}
__device__ __forceinline__ uint32_t lds_offset(const void* p)
{
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// The matrix instruction here is v_mfma_i32_32x32x32_i8: a 32 feature x 32 position tile per instruction, 32 k values
// (two feature slices of one tap: lanes 0-31 bring the 16 bytes of the first, lanes 32-63 those of the second, for both
// operands alike).  Against the 16x16x64 form it needs half as many instructions per multiply-accumulate, which leaves
// the issue port free for the LDS reads and the sign flips of the step (measured on a loop with both operands from LDS,
// one barrier per step and two waves per SIMD: matrix pipe 91 % busy against 80 %).  A lane's 16 accumulators of a tile
// are the features 8g + 4h + i (g = 0..3, i = 0..3, h = lane / 32) of position lane % 32; the weight rows of every 32-row
// tile are stored permuted (row 8g + 4h + i holds feature 16h + 4g + i), so that the lane ends with 16 CONSECUTIVE
// features of its position: one 16-byte store into fs_b_yx_fsv16, as in the other kernels.
//
// MT x NT tiles per wave (32 features x 32 positions each), WP x WF waves per workgroup, R stages in the weight ring,
// PL patch wave-loads per wave in each of the first PSTEPS steps of a block.
template <int MT, int NT, int WP, int WF, int R, int PL, int EPI>
__global__ void __launch_bounds__(WP * WF * 64) conv_halo_kernel(HaloArgs h)
{
    constexpr int TAPS = 9;
    constexpr int PSTEPS = TAPS - R;          // steps of a block that request patch chunks of the next block
    constexpr int WAVES = WP * WF;
    constexpr int BN = WF * MT * 32, BM = WP * NT * 32;
    constexpr int STAGE = 4 * BN;             // 16-byte units per ring stage
    constexpr int WL = STAGE / 64 / WAVES;    // weight wave-loads per wave and step
    constexpr int FRAGS = 2 * MT;             // weight fragments of a step: two k-halves x MT tiles
    static_assert(WL * 64 * WAVES == STAGE && WL >= 1, "weight stage must split evenly over the waves");
    static_assert(MT == 4 && NT == 2 && R == 4, "the read schedule of the main loop is written out for this shape");
    const MfmaArgs& a = h.m;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave_p = wave % WP, wave_f = wave / WP;
    const int half = lane >> 5, l32 = lane & 31;
    // Everything the prologue and the loop read from the argument block is requested here, behind ONE wait: left to
    // itself the compiler fetches arguments where they are first used, four dependent round trips to memory (about
    // 0.4 us each) before the first operand request goes out.
    asm volatile("" ::"s"(a.in), "s"(a.wpk), "s"(a.acc_init), "s"(a.ofm_tiles), "s"(a.div_ofm_tiles.mul), "s"(a.div_ofm_tiles.shift), "s"(a.div_ofm_tiles.one), "s"(a.ksteps), "s"(a.in_pf), "s"(a.xor_mask),
                 "s"(h.pos_total), "s"(h.halo_lo), "s"(h.patch_len), "s"(h.cps), "s"(h.div_cps.mul), "s"(h.div_cps.shift),
                 "s"(h.div_cps.one), "s"(h.blocks), "s"(h.ptiles), "s"(h.parts), "s"(h.tap[0]), "s"(h.tap[1]), "s"(h.tap[2]),
                 "s"(h.tap[3]), "s"(h.tap[4]), "s"(h.tap[5]), "s"(h.tap[6]), "s"(h.tap[7]), "s"(h.tap[8]));

    // Workgroup ids are dealt round-robin to the eight dies.  A die takes a contiguous eighth of the partitions with
    // all their feature tiles adjacent in time: neighbouring position tiles share their halos, feature tiles their
    // whole patch, through that die's L2.
    const int xcd = blockIdx.x & 7, jj = blockIdx.x >> 3;
    const int jj_by_f = (int)a.div_ofm_tiles.div((uint32_t)jj);
    const int part = xcd * (h.parts >> 3) + jj_by_f;
    const int ntile = jj - jj_by_f * a.ofm_tiles;
    const int t_begin = (int)((uint32_t)part * (uint32_t)h.tpp + h.div_parts.div((uint32_t)part * (uint32_t)h.trem));
    const int t_end = (int)((uint32_t)(part + 1) * (uint32_t)h.tpp + h.div_parts.div((uint32_t)(part + 1) * (uint32_t)h.trem));
    if (t_begin >= t_end) return;

    extern __shared__ __align__(16) unsigned char smem[];
    v4i* ring = reinterpret_cast<v4i*>(smem);  // [R][4 slices][BN rows]
    v4i* patch = ring + R * STAGE;             // [2][4 slices][patch_len]
    const int patch_v4 = 4 * h.patch_len;

    // fragment (k-half kh, tile) of a lane: slice 2 * kh + half
    const int a_lane = half * BN + wave_f * MT * 32 + l32;
    const int b_lane = half * h.patch_len + wave_p * NT * 32 + l32;
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

    v16i acc[MT][NT];
    auto reset_acc = [&]() {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int f = ntile * BN + (wave_f * MT + mt) * 32 + half * 16;
            v16i init;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const v4i v = *reinterpret_cast<const v4i*>(a.acc_init + f + g * 4);
                init[g * 4 + 0] = v[0], init[g * 4 + 1] = v[1], init[g * 4 + 2] = v[2], init[g * 4 + 3] = v[3];
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = init;
        }
    };

    // ---- prologue: the first patch, the first R weight stages; the accumulator start values are requested behind
    // them (the wait below then covers most of those too: loads complete in order)
    for (int c = wave; c < 4 * h.cps; c += WAVES) issue_patch(c, t_begin, 0, 0);
    step_fence();
#pragma unroll
    for (int u = 0; u < R; ++u) issue_weights(u, u);
    step_fence();
    reset_acc();
    step_fence();
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((R - 2) * WL) : "memory");

    // ---- main loop.  LDS reads are issued by hand (the compiler does not see them) and waited for by count: the reads of
    // a step are a fixed sequence, returned in order, so "at most N outstanding" names exactly the fragment that is
    // needed.  Per step and wave, in issue order: weight fragments 4..7 of this step (one in front of each of the
    // first four fragments' matrix instructions), then, spread over the last four fragments, the next step's four
    // activation fragments and its weight fragments 0..3.  Every fragment is requested 256 matrix-pipe clocks or more
    // before its first use; nothing is read behind the step's barrier that the step itself still needs.
    const uint32_t a_lane_b = lds_offset(ring) + (uint32_t)a_lane * 16u;
    const uint32_t b_lane_b = lds_offset(patch) + (uint32_t)b_lane * 16u;
    const uint32_t kh_bytes = 2u * (uint32_t)h.patch_len * 16u;   // from a k-half's slices to the next one's
    constexpr int KH_A = 2 * BN * 16;                             // the same for the weights
    int rd_stage = 0;        // ring stage of the current step
    int wnext = R % TAPS;    // K-step of the tile whose weights are requested next (ksteps is a multiple of TAPS >= R)
    int pbuf = 0;            // patch buffer of the current block
    v4i fa[FRAGS], fb[2][NT], fbn[2][NT];
    {
        const uint32_t b0 = b_lane_b + (uint32_t)h.tap[0] * 16u, b1 = b0 + kh_bytes;
        lds_read<0>(fbn[0][0], b0), lds_read<512>(fbn[0][1], b0), lds_read<0>(fa[0], a_lane_b);
        lds_read<0>(fbn[1][0], b1), lds_read<512>(fbn[1][1], b1), lds_read<512>(fa[1], a_lane_b);
        lds_read<1024>(fa[2], a_lane_b), lds_read<1536>(fa[3], a_lane_b);
    }
    auto mma = [&](int j) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            acc[j % MT][nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[j], fb[j / MT][nt], acc[j % MT][nt], 0, 0, 0);
    };

    for (int tile = t_begin; tile < t_end; ++tile) {
        for (int cb = 0; cb < h.blocks; ++cb) {
            const bool last_cb = cb + 1 == h.blocks;
            const int cb_n = last_cb ? 0 : cb + 1;
            const int tile_n = last_cb ? tile + 1 : tile;
            static_for<0, TAPS>([&](auto ic) {
                constexpr int S = decltype(ic)::value;
                // requests younger than the weights of step + 2 when this step's barrier is reached: the weights of
                // step + 3 and the patch chunks of the last two steps
                constexpr int YOUNGER = WL + (((S + TAPS - 2) % TAPS) < PSTEPS ? PL : 0) + (((S + TAPS - 1) % TAPS) < PSTEPS ? PL : 0);
                const int nx_stage = rd_stage + 1 == R ? 0 : rd_stage + 1;
                const uint32_t a_cur = a_lane_b + (uint32_t)(rd_stage * STAGE * 16);
                const uint32_t a_nxt = a_lane_b + (uint32_t)(nx_stage * STAGE * 16);
                const int nbuf = S == TAPS - 1 ? pbuf ^ 1 : pbuf;
                const uint32_t b_nxt0 = b_lane_b + (uint32_t)(nbuf * patch_v4 + h.tap[(S + 1) % TAPS]) * 16u;
                const uint32_t b_nxt1 = b_nxt0 + kh_bytes;
                // this step's activation fragments and its first weight fragment have landed (three younger reads)
                asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(fbn[0][0]), "+v"(fbn[0][1]), "+v"(fbn[1][0]), "+v"(fbn[1][1]), "+v"(fa[0]));
#pragma unroll
                for (int kh = 0; kh < 2; ++kh)
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) fb[kh][nt] = fbn[kh][nt] ^ xm;
                step_fence();
                lds_read<KH_A + 0>(fa[4], a_cur);
                mma(0);
                step_fence();
                lds_read<KH_A + 512>(fa[5], a_cur);
                lds_wait<4>(fa[1]);
                mma(1);
                step_fence();
                lds_read<KH_A + 1024>(fa[6], a_cur);
                lds_wait<4>(fa[2]);
                mma(2);
                step_fence();
                lds_read<KH_A + 1536>(fa[7], a_cur);
                lds_wait<4>(fa[3]);
                mma(3);
                step_fence();
                lds_read<0>(fbn[0][0], b_nxt0), lds_read<512>(fbn[0][1], b_nxt0), lds_read<0>(fa[0], a_nxt);
                lds_wait<6>(fa[4]);
                mma(4);
                step_fence();
                lds_read<0>(fbn[1][0], b_nxt1), lds_read<512>(fbn[1][1], b_nxt1), lds_read<512>(fa[1], a_nxt);
                lds_wait<8>(fa[5]);
                mma(5);
                step_fence();
                lds_read<1024>(fa[2], a_nxt);
                lds_wait<8>(fa[6]);
                mma(6);
                step_fence();
                lds_read<1536>(fa[3], a_nxt);
                lds_wait<8>(fa[7]);
                // Every read of this step's ring stage has completed in this wave.  Behind the barrier that holds for all
                // waves, so the stage can be refilled (with the weights of step + 4); and the weights of step + 2 and the
                // patch chunks requested up to three steps ago are in LDS for everybody.
                asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(YOUNGER) : "memory");
                issue_weights(wnext, rd_stage);
                wnext = wnext + 1 == a.ksteps ? 0 : wnext + 1;
                if constexpr (S < PSTEPS) {
#pragma unroll
                    for (int i = 0; i < PL; ++i) issue_patch((S * WAVES + wave) * PL + i, tile_n, cb_n, pbuf ^ 1);
                }
                step_fence();
                mma(7);
                step_fence();
                rd_stage = nx_stage;
            });
            pbuf ^= 1;
        }
        // the compiler's own waits in the epilogue count LDS and scalar-memory returns together: start it with nothing of
        // ours outstanding (the first fragments of the next tile, requested above)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        // ---- requantise and store the tile: a lane holds 16 consecutive features of one position per tile
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const uint32_t q = (uint32_t)tile * BM + (uint32_t)(wave_p * NT * 32 + nt * 32 + l32);
            const uint32_t b = h.div_yxp.div(q);
            const uint32_t r = q - b * (uint32_t)h.YXp;
            const uint32_t yp = h.div_wp.div(r);
            const int oy = (int)yp - h.pad_lo_y, ox = (int)(r - yp * (uint32_t)h.Wp) - h.pad_lo_x;
            const bool ok = q < (uint32_t)h.pos_total && (uint32_t)oy < (uint32_t)a.OH && (uint32_t)ox < (uint32_t)a.OW;
            if (!ok) continue;
            const int ob = a.out_off + (int)b * a.out_pb + oy * a.out_py + ox * 16;
            const int eb = a.el_off + (int)b * a.el_pb + oy * a.esy * a.el_py + ox * a.esx * 16;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int f0 = ntile * BN + (wave_f * MT + mt) * 32 + half * 16;
                if (f0 >= a.OFM) continue;
                const int fs = f0 >> 4;
                const int valid = a.OFM - f0;
                LaneScales sc;
                load_scales<EPI>(a, f0, sc);
                v4i one[4][1];
#pragma unroll
                for (int c = 0; c < 16; ++c) one[c >> 2][0][c & 3] = acc[mt][nt][c];
                const int obase = ob + fs * a.out_pf, ebase = eb + fs * a.el_pf;
                v4i ev4 = {0, 0, 0, 0};
                if constexpr (EPI == EPI_KIND_FUSED) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
                else if constexpr (EPI == EPI_KIND_FAST)
                    if (a.fe.fused) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
                finish_pixel<1, EPI>(a, one, 0, f0, valid, obase, ebase, sc, ev4, b, (uint32_t)oy, (uint32_t)ox);
            }
        }
        reset_acc();
    }
    // requests past the end of the workgroup's work are still on their way into its LDS
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

template <int MT, int NT, int WP, int WF, int R, int PL>
void launch_halo_instance(hipStream_t s, const HaloArgs& h, int grid, int lds, int epi)
{
    const dim3 g(grid), b(WP * WF * 64);
#define HALO_LAUNCH(KIND)                                                                                           \
    {                                                                                                               \
        static std::once_flag allowed;                                                                              \
        std::call_once(allowed, [] {                                                                                \
            CHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_halo_kernel<MT, NT, WP, WF, R, PL, KIND>), \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));                \
        });                                                                                                         \
        hipLaunchKernelGGL((conv_halo_kernel<MT, NT, WP, WF, R, PL, KIND>), g, b, lds, s, h);                       \
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
