// A depthwise 3x3 convolution and the one or two 1x1 convolutions behind it in ONE launch: the tail of a MobileNet
// block and the head of the next one,
//     depthwise 3x3 (mid -> mid)  ->  1x1 projection (mid -> few)  ->  1x1 expansion of the next block (few -> 6 few).
// The depthwise result (as large as the expanded tensor it reads) and the projection's input never touch memory.
//
// The depthwise stage runs on the MATRIX cores, which the 1x1 stages leave almost idle, so that the vector ALU is
// free for the three requantisation epilogues (they are what bounds these layers).  One v_mfma_i32_16x16x64_i8 per
// filter tap and 16-feature fragment: B is what the dense kernels feed anyway -- lane (kq, l16) holds the 16 features
// of slice kq of pixel l16, shifted by the tap -- and A is DIAGONAL: row r of fragment mt stands for feature
// 16 * (r / 4) + 4 * mt + r % 4 of the K-step's 64 features (the row order that leaves a lane with 16 consecutive
// features), and its only non-zero weight sits at exactly that feature's k position.  In register terms the lane
// (kq, l16) of such an A fragment is one dword (weight << 8 * (l16 % 4), or zero unless kq == l16 / 4) in slot mt of
// four; the host precomputes that dword per (K-step, tap, fragment, lane) and the kernel keeps the table in LDS.
// Nine taps times four fragments give the 64 depthwise features of a K-step for 16 pixels; their requantised, packed
// result is the B fragment of the projection's K-step, and from there on the chain is the dense one.
//
// Work split as in the dense chain: persistent workgroups of four independent waves, granules of 16 * NT pixels, the
// activation taps requested D steps ahead (also across granules), all weights and per-feature vectors in LDS.
#pragma once
#include "conv_chain_kernel.h"

namespace chip {

struct DwChainArgs {
    const int8_t* in;
    const v4i* img;            // LDS image: diagonal-weight dwords [KS][9][4][64], units of stage 1 [SP1][KS], units of
                               // stage 2 [SP2][SP1], per-feature vectors of stages 0, 1, 2
    int32_t dw_quads;          // 16-byte pieces of the diagonal-weight table (KS * 9 * 64)
    int32_t units, vec_quads;
    int32_t granules;          // ceil(M / (16 * NT))
    int32_t gpw, grem;         // granules / waves of the grid and the remainder
    FastDiv div_waves;         // wave w starts at granule w * gpw + (w * grem) / waves = floor(w * granules / waves)
    uint32_t M;
    int32_t OHW, OW;
    FastDiv div_ohw, div_ow;
    int32_t sy, sx, py, px;
    int32_t in_off, in_pb, in_pf, in_py;  // bytes
    int32_t tap_dy, tap_dx;
    int32_t CB;                // 16-feature slices of the depthwise stage
    int32_t KS;                // K-steps of stage 1 = ceil(CB / 4)
    int32_t SP2;               // 64-feature spans of stage 2 (0: two stages)
    ChainStage st[CHAIN_MAX_STAGES];
};

// EPI0 / EPI1 / EPI2: epilogue kinds of the three stages, fixed at compile time where the stages have one of the
// branch-free forms (a MobileNet block: CLAMPQ, LINEAR, CLAMPQ), else the run-time form FAST for all of them
template <int NT, int SP1, bool HAS2, int EPI0, int EPI1, int EPI2>
__global__ void __launch_bounds__(256) conv_dwchain_kernel(DwChainArgs a)
{
    constexpr int WP = NT * 16;
    constexpr int D = 3;  // look-ahead in taps; the nine taps of a K-step are three rounds
    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int kq = lane >> 4;
    const int l16 = lane & 15;
    const ChainStage& s0 = a.st[0];
    const ChainStage& s1 = a.st[1];
    const ChainStage& s2 = a.st[2];

    extern __shared__ __align__(16) unsigned char smem[];
    const int32_t* ldsD = reinterpret_cast<const int32_t*>(smem);                         // [KS][9][4][64] dwords
    v4i* ldsW = reinterpret_cast<v4i*>(smem + (size_t)a.dw_quads * 16);                    // [units][4][64]
    const int32_t* ldsV = reinterpret_cast<const int32_t*>(smem + (size_t)a.dw_quads * 16 + (size_t)a.units * 4096);
    {
        v4i* dst = reinterpret_cast<v4i*>(smem);
        const int total = a.dw_quads + a.units * 256 + a.vec_quads;
        constexpr int BATCH = 8;
        for (int i = t; i < total; i += BATCH * 256) {
            v4i r[BATCH];
#pragma unroll
            for (int u = 0; u < BATCH; ++u) r[u] = a.img[min(i + u * 256, total - 1)];
#pragma unroll
            for (int u = 0; u < BATCH; ++u)
                if (i + u * 256 < total) dst[i + u * 256] = r[u];
        }
    }

    const int per_xcd = gridDim.x >> 3;  // the grid is a multiple of 8
    const uint32_t vb = (blockIdx.x & 7u) * (uint32_t)per_xcd + (blockIdx.x >> 3);
    const uint32_t gw = vb * 4u + (uint32_t)wave;
    const int g_begin = (int)(gw * (uint32_t)a.gpw + a.div_waves.div(gw * (uint32_t)a.grem));
    const int g_end = (int)((gw + 1) * (uint32_t)a.gpw + a.div_waves.div((gw + 1) * (uint32_t)a.grem));
    if (g_begin >= g_end) {
        __syncthreads();
        return;
    }

    const v4i xm0 = {(int)s0.xor_mask, (int)s0.xor_mask, (int)s0.xor_mask, (int)s0.xor_mask};
    const v4i xm1 = {(int)s1.xor_mask, (int)s1.xor_mask, (int)s1.xor_mask, (int)s1.xor_mask};
    const v4i xm2 = {(int)s2.xor_mask, (int)s2.xor_mask, (int)s2.xor_mask, (int)s2.xor_mask};

    struct Refs {
        uint32_t boff[NT];  // byte offset of the lane's pixel at tap (0, 0), slice 0
        int o0[NT], o1[NT], e1[NT], o2[NT];
    };
    auto setup = [&](int g, Refs& r) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const uint32_t m = (uint32_t)g * WP + nt * 16 + l16;
            const bool ok = g < g_end && m < a.M;
            const PixelPos pp = [&] {
                PixelPos q;
                const uint32_t mm = ok ? m : 0;
                q.b = a.div_ohw.div(mm);
                const uint32_t rr = mm - q.b * a.OHW;
                q.oy = a.div_ow.div(rr);
                q.ox = rr - q.oy * a.OW;
                return q;
            }();
            r.boff[nt] = (uint32_t)(a.in_off + (int)pp.b * a.in_pb + ((int)pp.oy * a.sy - a.py) * a.in_py + ((int)pp.ox * a.sx - a.px) * 16);
            auto at = [&](const ChainStage& st) {
                return st.out_off + (int)pp.b * st.out_pb + kq * st.out_pf + (int)pp.oy * st.out_py + (int)pp.ox * 16;
            };
            r.o0[nt] = ok && s0.out ? at(s0) : -1;
            r.o1[nt] = ok && s1.out ? at(s1) : -1;
            r.o2[nt] = HAS2 && ok && s2.out ? at(s2) : -1;
            r.e1[nt] = s1.el_off + (int)pp.b * s1.el_pb + kq * s1.el_pf + (int)pp.oy * s1.el_py + (int)pp.ox * s1.el_px;
        }
    };
    // walk over the (K-step, tap) sequence of the activation requests: the lane's slice of K-step ks is 4 * ks + kq; a
    // slice past the end (a partly filled last K-step) reads slice 0, its diagonal weights are zero
    struct Walk {
        int ks, fy, fx;
    };
    auto walk_reset = [](Walk& w) { w.ks = 0, w.fy = 0, w.fx = 0; };
    auto walk_advance = [&](Walk& w) {
        if (++w.fx == 3) {
            w.fx = 0;
            if (++w.fy == 3) w.fy = 0, ++w.ks;
        }
    };
    auto load_b = [&](const Refs& r, const Walk& w, v4i (&xb)[NT]) {
        const int ks = w.ks < a.KS ? w.ks : 0;
        const int slice = ks * 4 + kq;
        const int8_t* base = a.in + ((slice < a.CB ? slice : 0) * a.in_pf + w.fy * a.tap_dy + w.fx * a.tap_dx);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) xb[nt] = *reinterpret_cast<const v4i*>(base + r.boff[nt]);
    };
    auto unit = [&](const ChainStage& st, int span, int ks) { return ldsW + (size_t)(st.unit0 + span * st.kstride + ks) * 256; };

    Refs cur, nxt;
    v4i rb[D][NT];
    Walk walk;
    setup(g_begin, cur);
    walk_reset(walk);
#pragma unroll
    for (int d = 0; d < D; ++d) {
        load_b(cur, walk, rb[d]);
        walk_advance(walk);
    }
    __syncthreads();  // table, weights and vectors are in LDS; no barrier after this point

    for (int g = g_begin; g < g_end; ++g) {
        setup(g + 1, nxt);
        // residual of the projection (a fused sum): requested now, used after the whole depthwise stage
        v4i ev1[SP1][NT];
#pragma unroll
        for (int sp = 0; sp < SP1; ++sp)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                ev1[sp][nt] = v4i{0, 0, 0, 0};
                if constexpr (chain_reads_residual<EPI1>())
                    if (s1.fe.fused && sp * 64 + kq * 16 < s1.OFM)
                        ev1[sp][nt] = *reinterpret_cast<const v4i*>((const int8_t*)s1.eltw + cur.e1[nt] + sp * 4 * s1.el_pf);
            }
        v4i acc1[SP1 * 4][NT];
#pragma unroll
        for (int sp = 0; sp < SP1; ++sp)
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                const v4i init = *reinterpret_cast<const v4i*>(ldsV + s1.vec0 + sp * 64 + kq * 16 + mt * 4);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc1[sp * 4 + mt][nt] = init;
            }

        for (int ks = 0; ks < a.KS; ++ks) {
            // ---------------- stage 0: 64 depthwise features of the granule's pixels
            v4i acc0[4][NT];
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                const v4i init = *reinterpret_cast<const v4i*>(ldsV + s0.vec0 + ks * 64 + kq * 16 + mt * 4);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) acc0[mt][nt] = init;
            }
            const bool last_ks = ks + 1 == a.KS;
#pragma unroll
            for (int t0 = 0; t0 < 9; t0 += D) {
                if (last_ks && t0 + D == 9) walk_reset(walk);  // the last round requests the next granule's first taps
#pragma unroll
                for (int d = 0; d < D; ++d) {
                    const int tap = t0 + d;
                    const int32_t* dia = ldsD + ((ks * 9 + tap) * 4) * 64 + lane;
#pragma unroll
                    for (int mt = 0; mt < 4; ++mt) {
                        v4i fa = {0, 0, 0, 0};
                        fa[mt] = dia[mt * 64];
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
                            acc0[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa, rb[d][nt] ^ xm0, acc0[mt][nt], 0, 0, 0);
                    }
                    load_b(last_ks && t0 + D == 9 ? nxt : cur, walk, rb[d]);
                    walk_advance(walk);
                    step_fence();
                }
            }
            // requantise: the packed results are the B fragment of stage 1's K-step ks
            const int f0 = ks * 64 + kq * 16;
            LaneScales sc;
            chain_scales<EPI0>(s0, ldsV, a.KS, f0, sc);
            v4i bf0[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const v4i none = {0, 0, 0, 0};
                v4i packed = epilogue_fast16<NT, EPI0>(s0, acc0, nt, sc.wq, sc.cal, sc.ecal, none, 16);
                if (f0 >= s0.OFM) packed = v4i{0, 0, 0, 0};
                else if (cur.o0[nt] >= 0) *reinterpret_cast<v4i*>((int8_t*)s0.out + cur.o0[nt] + ks * 4 * s0.out_pf) = packed;
                bf0[nt] = packed ^ xm1;
            }
            // ---------------- stage 1 accumulates this K-step
#pragma unroll
            for (int sp = 0; sp < SP1; ++sp)
#pragma unroll
                for (int mt = 0; mt < 4; ++mt) {
                    const v4i fa = unit(s1, sp, ks)[kq * 64 + mt * 16 + l16];
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
                        acc1[sp * 4 + mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa, bf0[nt], acc1[sp * 4 + mt][nt], 0, 0, 0);
                }
        }

        // ---------------- stage 1 epilogue: the packed results are the B fragments of stage 2 (K-step = span)
        v4i bf1[SP1][NT];
#pragma unroll
        for (int sp = 0; sp < SP1; ++sp) {
            const int f0 = sp * 64 + kq * 16;
            LaneScales sc;
            chain_scales<EPI1>(s1, ldsV, SP1, f0, sc);
            const v4i(&acc_sp)[4][NT] = *reinterpret_cast<const v4i(*)[4][NT]>(&acc1[sp * 4]);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                v4i packed = epilogue_fast16<NT, EPI1>(s1, acc_sp, nt, sc.wq, sc.cal, sc.ecal, ev1[sp][nt], s1.OFM - f0);
                if (f0 >= s1.OFM) packed = v4i{0, 0, 0, 0};
                else if (cur.o1[nt] >= 0) *reinterpret_cast<v4i*>((int8_t*)s1.out + cur.o1[nt] + sp * 4 * s1.out_pf) = packed;
                bf1[sp][nt] = packed ^ xm2;
            }
        }

        // ---------------- stage 2, span by span
        if constexpr (HAS2) {
            for (int sp = 0; sp < a.SP2; ++sp) {
                const int f0 = sp * 64 + kq * 16;
                v4i acc2[4][NT];
#pragma unroll
                for (int mt = 0; mt < 4; ++mt) {
                    const v4i init = *reinterpret_cast<const v4i*>(ldsV + s2.vec0 + f0 + mt * 4);
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) acc2[mt][nt] = init;
                }
#pragma unroll
                for (int ks = 0; ks < SP1; ++ks)
#pragma unroll
                    for (int mt = 0; mt < 4; ++mt) {
                        const v4i fa = unit(s2, sp, ks)[kq * 64 + mt * 16 + l16];
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
                            acc2[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa, bf1[ks][nt], acc2[mt][nt], 0, 0, 0);
                    }
                if (f0 >= s2.OFM) continue;
                LaneScales sc;
                chain_scales<EPI2>(s2, ldsV, a.SP2, f0, sc);
                const v4i none = {0, 0, 0, 0};
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    if (cur.o2[nt] < 0) continue;
                    const v4i packed = epilogue_fast16<NT, EPI2>(s2, acc2, nt, sc.wq, sc.cal, sc.ecal, none, s2.OFM - f0);
                    *reinterpret_cast<v4i*>((int8_t*)s2.out + cur.o2[nt] + sp * 4 * s2.out_pf) = packed;
                }
            }
        }
        cur = nxt;
    }
}

template <int NT, int SP1, bool HAS2, int EPI0, int EPI1, int EPI2>
void launch_dwchain_instance(hipStream_t s, const DwChainArgs& a, int grid, int lds)
{
    static std::once_flag allowed;
    std::call_once(allowed, [] {
        CHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_dwchain_kernel<NT, SP1, HAS2, EPI0, EPI1, EPI2>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    });
    hipLaunchKernelGGL((conv_dwchain_kernel<NT, SP1, HAS2, EPI0, EPI1, EPI2>), dim3(grid), dim3(256), lds, s, a);
}

}  // namespace chip
