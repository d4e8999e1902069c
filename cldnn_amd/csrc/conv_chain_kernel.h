// A chain of up to three quantized convolutions in ONE launch: a spatial convolution (3x3 ...) followed by one
// or two 1x1 / stride-1 convolutions that consume its result, e.g. the tail of a ResNet bottleneck
//     3x3 (mid -> mid)  ->  1x1 expansion (mid -> 4 mid) + residual  ->  1x1 reduction of the next block (4 mid -> mid).
//
// Why it needs no shared memory between the stages: with weight rows permuted as the tile kernels store them, the
// 16 accumulators a lane holds after v_mfma_i32_16x16x64_i8 are 16 CONSECUTIVE features of one pixel; requantised
// and packed they are 16 bytes = exactly the lane's share of the B operand (64 k-values x 16 pixels) of the next
// 1x1 convolution, whose K index is the previous stage's feature index.  A wave that computes all features of a
// stage for its 16*NT pixels therefore feeds the next stage straight from its registers: the intermediate tensor
// is never written (unless somebody else reads it) and never read back.
//
// Work split: persistent workgroups of four INDEPENDENT waves.  All weights of all stages (a few tens of KB) and
// the per-feature vectors are copied into LDS once per workgroup; after that a wave walks over its own range of
// 16*NT-pixel granules without any barrier.  Feature counts are multiples of 64.  Stage 0 reads its activations straight from global memory, D K-steps
// ahead of their use, and the look-ahead runs across granule boundaries (as in the weights-stationary kernel).
// Every stage has its own epilogue kind, per-feature vectors, output tensor and (optional) residual tensor.
#pragma once
#include <mutex>

#include "conv_chain.h"
#include "conv_mfma_kernel.h"

namespace chip {

enum { CHAIN_MAX_STAGES = 3 };

struct ChainStage {
    void* out;                 // nullptr: the result of this stage is not materialised
    const void* eltw;          // residual operand of a fused stage
    int32_t OFM;
    int32_t out_off, out_pb, out_pf, out_py;  // elements
    int32_t el_off, el_pb, el_pf, el_py, el_px;  // elements; el_py / el_px carry the residual's stride (a sub-sampled shortcut)
    uint32_t xor_mask;         // applied to the fragments this stage READS (0x80808080: its input is u8)
    int32_t unit0;             // first 4 KB weight unit of the stage inside the LDS image
    int32_t kstride;           // units per 64-feature span (K-steps incl. zero padding)
    int32_t vec0;              // first dword of the stage's vectors in LDS: init, calib, eltw_calib, wqf (spans * 64 each)
    FastEpi fe;
    Epilogue epi;
};

struct ChainArgs {
    const int8_t* in;
    const v4i* wpk;            // LDS image: weight units [unit][kq][64 rows] x 16 bytes, then the per-feature vectors
    int32_t units;
    int32_t vec_quads;         // 16-byte pieces of per-feature vectors behind the units
    int32_t granules;          // ceil(M / (16 * NT))
    int32_t gpw, grem;         // granules / waves of the grid and the remainder
    FastDiv div_waves;         // wave w starts at granule w * gpw + (w * grem) / waves = floor(w * granules / waves)
    uint32_t M;
    int32_t OHW, OW;
    FastDiv div_ohw, div_ow;
    int32_t sy, sx, py, px;
    int32_t in_off, in_pb, in_pf, in_py;  // bytes
    int32_t ksteps0, CB, FX, FY, tap_dy, tap_dx;
    ChainStage st[CHAIN_MAX_STAGES];
};

__device__ __forceinline__ PixelPos chain_pixel_pos(const ChainArgs& a, uint32_t m)
{
    PixelPos p;
    p.b = a.div_ohw.div(m);
    const uint32_t r = m - p.b * a.OHW;
    p.oy = a.div_ow.div(r);
    p.ox = r - p.oy * a.OW;
    return p;
}

__device__ __forceinline__ void chain_tap_advance(const ChainArgs& a, TapWalk& w, int cb4)
{
    w.sg += 1;
    w.off += 4 * a.in_pf;
    if (w.sg == cb4) {
        w.sg = 0;
        w.off += a.tap_dx - cb4 * 4 * a.in_pf;
        w.fx += 1;
        if (w.fx == a.FX) {
            w.fx = 0;
            w.off += a.tap_dy - a.FX * a.tap_dx;
            w.fy += 1;
        }
    }
}

// the lane's 16 per-feature values of one vector kind, from the LDS copy
__device__ __forceinline__ void chain_vec16(const int32_t* ldsV, int at, float (&dst)[16])
{
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const v4i q = *reinterpret_cast<const v4i*>(ldsV + at + d * 4);
        dst[d * 4 + 0] = __int_as_float(q[0]), dst[d * 4 + 1] = __int_as_float(q[1]);
        dst[d * 4 + 2] = __int_as_float(q[2]), dst[d * 4 + 3] = __int_as_float(q[3]);
    }
}

template <int EPI>
__device__ __forceinline__ void chain_scales(const ChainStage& st, const int32_t* ldsV, int spans, int f0, LaneScales& sc)
{
    if constexpr (EPI == EPI_KIND_RELU || EPI == EPI_KIND_LINEAR) {
        chain_vec16(ldsV, st.vec0 + spans * 64 + f0, sc.cal);
    } else if constexpr (EPI == EPI_KIND_CLAMPQ) {
        chain_vec16(ldsV, st.vec0 + spans * 64 + f0, sc.cal);
        chain_vec16(ldsV, st.vec0 + 3 * spans * 64 + f0, sc.wq);
    } else if constexpr (EPI == EPI_KIND_FUSED || EPI == EPI_KIND_SUMLIN) {
        chain_vec16(ldsV, st.vec0 + spans * 64 + f0, sc.cal);
        chain_vec16(ldsV, st.vec0 + 2 * spans * 64 + f0, sc.ecal);
    } else {  // EPI_KIND_FAST: absent vectors were filled with their neutral values by the host
        chain_vec16(ldsV, st.vec0 + spans * 64 + f0, sc.cal);
        chain_vec16(ldsV, st.vec0 + 2 * spans * 64 + f0, sc.ecal);
        chain_vec16(ldsV, st.vec0 + 3 * spans * 64 + f0, sc.wq);
    }
}

template <int EPI>
constexpr bool chain_reads_residual()
{
    return EPI == EPI_KIND_FUSED || EPI == EPI_KIND_FAST || EPI == EPI_KIND_SUMLIN;
}

// SP0 / SP1 / SP2: 64-feature spans of the three stages (SP2 == 0: two stages).  D: activation look-ahead of stage 0.
template <int NT, int D, int SP0, int SP1, int SP2, int EPI0, int EPI1, int EPI2>
__global__ void __launch_bounds__(256) conv_chain_kernel(ChainArgs a)
{
    constexpr int WP = NT * 16;
    constexpr int EVD = SP1 < 4 ? SP1 : 4;  // residual look-ahead of stage 1, in spans
    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int kq = lane >> 4;
    const int l16 = lane & 15;
    const ChainStage& s0 = a.st[0];
    const ChainStage& s1 = a.st[1];
    const ChainStage& s2 = a.st[2];

    extern __shared__ __align__(16) unsigned char smem[];
    v4i* ldsW = reinterpret_cast<v4i*>(smem);                              // [units][4][64]
    int32_t* ldsV = reinterpret_cast<int32_t*>(smem + (size_t)a.units * 4096);  // per-feature vectors
    {
        // one bulk copy: the image holds the weight units and, behind them, the per-feature vectors of all stages
        // (absent vectors filled with their neutral values by the host); all requests of a thread are in flight at once
        const int total = a.units * 256 + a.vec_quads;
        constexpr int BATCH = 20;
        for (int i = t; i < total; i += BATCH * 256) {
            v4i r[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u) r[u] = a.wpk[min(i + u * 256, total - 1)];
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                if (i + u * 256 < total) ldsW[i + u * 256] = r[u];
        }
    }

    // Every die gets one contiguous run of workgroups, every wave one contiguous range of granules: rows that
    // share filter taps stay inside one die's L2.  (A shared counter that hands out granules one by one was tried:
    // device-scope atomics on a handful of addresses take about 0.2 us each, one after the other, which cost four
    // times what the better balance saved.)
    const int per_xcd = gridDim.x >> 3;  // the grid is a multiple of 8
    const uint32_t vb = (blockIdx.x & 7u) * (uint32_t)per_xcd + (blockIdx.x >> 3);
    // (a 64-bit division of two run-time values here costs every wave a few hundred instructions before its first request)
    const uint32_t gw = vb * 4u + (uint32_t)wave;
    const int g_begin = (int)(gw * (uint32_t)a.gpw + a.div_waves.div(gw * (uint32_t)a.grem));
    const int g1 = (int)((gw + 1) * (uint32_t)a.gpw + a.div_waves.div((gw + 1) * (uint32_t)a.grem));

    const v4i xm0 = {(int)s0.xor_mask, (int)s0.xor_mask, (int)s0.xor_mask, (int)s0.xor_mask};
    const v4i xm1 = {(int)s1.xor_mask, (int)s1.xor_mask, (int)s1.xor_mask, (int)s1.xor_mask};
    const v4i xm2 = {(int)s2.xor_mask, (int)s2.xor_mask, (int)s2.xor_mask, (int)s2.xor_mask};
    const int cb4 = a.CB >> 2;

    struct Refs {
        uint32_t boff[NT];
        int o0[NT], o1[NT], e1[NT], o2[NT], e0[NT], e2[NT];
    };
    auto setup = [&](int g, Refs& r) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const uint32_t m = (uint32_t)g * WP + nt * 16 + l16;
            const bool ok = g < g1 && m < a.M;
            const PixelPos pp = chain_pixel_pos(a, ok ? m : 0);
            r.boff[nt] = (uint32_t)(a.in_off + (int)pp.b * a.in_pb + ((int)pp.oy * a.sy - a.py) * a.in_py
                                    + ((int)pp.ox * a.sx - a.px) * 16 + kq * a.in_pf);
            auto at = [&](const ChainStage& st) {
                return st.out_off + (int)pp.b * st.out_pb + kq * st.out_pf + (int)pp.oy * st.out_py + (int)pp.ox * 16;
            };
            auto res = [&](const ChainStage& st) {
                return st.el_off + (int)pp.b * st.el_pb + kq * st.el_pf + (int)pp.oy * st.el_py + (int)pp.ox * st.el_px;
            };
            r.o0[nt] = ok && s0.out ? at(s0) : -1;
            r.o1[nt] = ok && s1.out ? at(s1) : -1;
            r.o2[nt] = SP2 > 0 && ok && s2.out ? at(s2) : -1;
            r.e0[nt] = res(s0), r.e1[nt] = res(s1), r.e2[nt] = SP2 > 0 ? res(s2) : 0;
        }
    };
    auto load_b = [&](const Refs& r, const TapWalk& w, v4i (&xb)[NT]) {
        const int8_t* base = a.in + (w.fy < a.FY ? w.off : 0);  // padded K-steps read tap 0 (their weights are zero)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) xb[nt] = *reinterpret_cast<const v4i*>(base + r.boff[nt]);
    };
    auto unit = [&](const ChainStage& st, int span, int ks) { return ldsW + (size_t)(st.unit0 + span * st.kstride + ks) * 256; };
    auto residual = [&](const ChainStage& st, int ebase, int span) {
        v4i v = {0, 0, 0, 0};
        if (st.fe.fused) v = *reinterpret_cast<const v4i*>((const int8_t*)st.eltw + ebase + span * 4 * st.el_pf);
        return v;
    };

    if (g_begin >= g1) {
        __syncthreads();
        return;
    }
    Refs cur, nxt;
    v4i rb[D][NT];
    TapWalk walk;  // tap of the next activation request
    setup(g_begin, cur);
    tap_reset(walk);
#pragma unroll
    for (int d = 0; d < D; ++d) {
        load_b(cur, walk, rb[d]);
        chain_tap_advance(a, walk, cb4);
    }
    __syncthreads();  // weights and vectors are in LDS; no barrier after this point

    for (int g = g_begin; g < g1; ++g) {
        setup(g + 1, nxt);
        // residual of stage 1 for the first spans: requested now, used after the whole of stage 0
        v4i ev1[EVD][NT];
        if constexpr (chain_reads_residual<EPI1>()) {
#pragma unroll
            for (int s = 0; s < EVD; ++s)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) ev1[s][nt] = residual(s1, cur.e1[nt], s);
        }

        // ---------------- stage 0: the spatial convolution, all SP0 spans at once
        v4i acc0[SP0 * 4][NT];
#pragma unroll
        for (int sp = 0; sp < SP0; ++sp)
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                const v4i init = *reinterpret_cast<const v4i*>(ldsV + s0.vec0 + sp * 64 + kq * 16 + mt * 4);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc0[sp * 4 + mt][nt] = init;
            }
        v4i fa_cur[SP0 * 4], fa_nxt[SP0 * 4];
        auto load_a0 = [&](int ks, v4i (&fa)[SP0 * 4]) {
#pragma unroll
            for (int sp = 0; sp < SP0; ++sp)
#pragma unroll
                for (int mt = 0; mt < 4; ++mt) fa[sp * 4 + mt] = unit(s0, sp, ks)[kq * 64 + mt * 16 + l16];
        };
        auto step = [&](int ks, int d, const Refs& refill_from) {
            load_a0(ks + 1 < a.ksteps0 ? ks + 1 : 0, fa_nxt);
            v4i fb[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) fb[nt] = rb[d][nt] ^ xm0;
#pragma unroll
            for (int m = 0; m < SP0 * 4; ++m)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    acc0[m][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa_cur[m], fb[nt], acc0[m][nt], 0, 0, 0);
            load_b(refill_from, walk, rb[d]);
            chain_tap_advance(a, walk, cb4);
#pragma unroll
            for (int m = 0; m < SP0 * 4; ++m) fa_cur[m] = fa_nxt[m];
            step_fence();
        };
        load_a0(0, fa_cur);
        for (int ks0 = 0; ks0 + D < a.ksteps0; ks0 += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) step(ks0 + d, d, cur);
        }
        tap_reset(walk);  // the last D steps request the first D steps of the next granule
#pragma unroll
        for (int d = 0; d < D; ++d) step(a.ksteps0 - D + d, d, nxt);

        // requantise stage 0: the packed results ARE the B fragments of stage 1 (K-step = span)
        v4i bf0[SP0][NT];
#pragma unroll
        for (int sp = 0; sp < SP0; ++sp) {
            const int f0 = sp * 64 + kq * 16;
            LaneScales sc;
            chain_scales<EPI0>(s0, ldsV, SP0, f0, sc);
            const v4i(&acc_sp)[4][NT] = *reinterpret_cast<const v4i(*)[4][NT]>(&acc0[sp * 4]);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                v4i ev = {0, 0, 0, 0};
                if constexpr (chain_reads_residual<EPI0>()) ev = residual(s0, cur.e0[nt], sp);
                const v4i packed = epilogue_fast16<NT, EPI0>(s0, acc_sp, nt, sc.wq, sc.cal, sc.ecal, ev, 16);
                if (cur.o0[nt] >= 0) *reinterpret_cast<v4i*>((int8_t*)s0.out + cur.o0[nt] + sp * 4 * s0.out_pf) = packed;
                bf0[sp][nt] = packed ^ xm1;
            }
        }

        // ---------------- stage 1 span by span; every finished span is one K-step of stage 2
        v4i acc2[SP2 > 0 ? SP2 * 4 : 1][NT];
        if constexpr (SP2 > 0) {
#pragma unroll
            for (int sp = 0; sp < SP2; ++sp)
#pragma unroll
                for (int mt = 0; mt < 4; ++mt) {
                    const v4i init = *reinterpret_cast<const v4i*>(ldsV + s2.vec0 + sp * 64 + kq * 16 + mt * 4);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) acc2[sp * 4 + mt][nt] = init;
                }
        }
#pragma unroll
        for (int s = 0; s < SP1; ++s) {
            const int f0 = s * 64 + kq * 16;
            v4i acc1[4][NT];
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                const v4i init = *reinterpret_cast<const v4i*>(ldsV + s1.vec0 + f0 + mt * 4);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc1[mt][nt] = init;
            }
#pragma unroll
            for (int ks = 0; ks < SP0; ++ks) {
                v4i fa[4];
#pragma unroll
                for (int mt = 0; mt < 4; ++mt) fa[mt] = unit(s1, s, ks)[kq * 64 + mt * 16 + l16];
#pragma unroll
                for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        acc1[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[mt], bf0[ks][nt], acc1[mt][nt], 0, 0, 0);
            }
            LaneScales sc;
            chain_scales<EPI1>(s1, ldsV, SP1, f0, sc);
            v4i bf1[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                v4i ev = {0, 0, 0, 0};
                if constexpr (chain_reads_residual<EPI1>()) ev = ev1[s % EVD][nt];
                const v4i packed = epilogue_fast16<NT, EPI1>(s1, acc1, nt, sc.wq, sc.cal, sc.ecal, ev, 16);
                if (cur.o1[nt] >= 0) *reinterpret_cast<v4i*>((int8_t*)s1.out + cur.o1[nt] + s * 4 * s1.out_pf) = packed;
                bf1[nt] = packed ^ xm2;
            }
            if constexpr (chain_reads_residual<EPI1>()) {
                if constexpr (SP1 > EVD) {
                    if (s + EVD < SP1) {
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt) ev1[s % EVD][nt] = residual(s1, cur.e1[nt], s + EVD);
                    }
                }
            }
            if constexpr (SP2 > 0) {
#pragma unroll
                for (int sp = 0; sp < SP2; ++sp) {
                    v4i fa[4];
#pragma unroll
                    for (int mt = 0; mt < 4; ++mt) fa[mt] = unit(s2, sp, s)[kq * 64 + mt * 16 + l16];
#pragma unroll
                    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
                            acc2[sp * 4 + mt][nt] =
                                __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[mt], bf1[nt], acc2[sp * 4 + mt][nt], 0, 0, 0);
                }
            }
        }

        // ---------------- stage 2 epilogue
        if constexpr (SP2 > 0) {
#pragma unroll
            for (int sp = 0; sp < SP2; ++sp) {
                const int f0 = sp * 64 + kq * 16;
                LaneScales sc;
                chain_scales<EPI2>(s2, ldsV, SP2, f0, sc);
                const v4i(&acc_sp)[4][NT] = *reinterpret_cast<const v4i(*)[4][NT]>(&acc2[sp * 4]);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    if (cur.o2[nt] < 0) continue;
                    v4i ev = {0, 0, 0, 0};
                    if constexpr (chain_reads_residual<EPI2>()) ev = residual(s2, cur.e2[nt], sp);
                    const v4i packed = epilogue_fast16<NT, EPI2>(s2, acc_sp, nt, sc.wq, sc.cal, sc.ecal, ev, 16);
                    *reinterpret_cast<v4i*>((int8_t*)s2.out + cur.o2[nt] + sp * 4 * s2.out_pf) = packed;
                }
            }
        }
        cur = nxt;
    }
}

template <int NT, int D, int SP0, int SP1, int SP2, int EPI0, int EPI1, int EPI2>
void launch_chain_instance(hipStream_t s, const ChainArgs& a, int grid, int lds)
{
    // more than 64 KiB of dynamic LDS has to be allowed per kernel, once
    static std::once_flag allowed;
    std::call_once(allowed, [] {
        CHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_chain_kernel<NT, D, SP0, SP1, SP2, EPI0, EPI1, EPI2>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    });
    hipLaunchKernelGGL((conv_chain_kernel<NT, D, SP0, SP1, SP2, EPI0, EPI1, EPI2>), dim3(grid), dim3(256), lds, s, a);
}

}  // namespace chip
