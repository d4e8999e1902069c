// Dense quantized convolution as an implicit GEMM on the gfx950 int8 matrix cores.
//
//   D[ofm][pixel] = sum_k W[ofm][k] * X[pixel][k],   k = (tap, input feature)
//
// computed with v_mfma_i32_16x16x64_i8: the A operand is a 16(ofm) x 64(k) weight tile, the
// B operand a 64(k) x 16(pixel) activation tile; every lane feeds 16 consecutive k bytes of one
// row / column, and that is exactly one 16-feature slice of one pixel in fs_b_yx_fsv16 memory
// (one 128-bit load, no byte shuffling anywhere).
//
// Two kernels share this mapping and the epilogue:
//   conv_mfma_kernel    workgroup = 4 waves, output tile BM pixels x BN features, each wave 64 features x
//                       WP pixels; per K-step (4 k-chunks = 64 k values) the workgroup stages BN x 64
//                       weight bytes and BM x 64 activation bytes in LDS (double buffered, one barrier per
//                       step).  For long K (3x3 and wide 1x1 layers), where operand reuse matters.
//   conv_stream_kernel  no LDS, no barriers: every wave loads its own fragments straight from global
//                       memory and walks over all output features.  For short K, where the layer is bound
//                       by HBM bandwidth and what matters is the number of independent requests in flight.
// Pixels are the linear index over (batch, oy, ox), so a tile may span rows and images.
// Two addressing modes:
//   !CHECKED  the input buffer carries a physical zero border at least as wide as the convolution's
//             padding, so tap (fy, fx, slice) is a constant byte offset from the pixel: ktab[kc].
//   CHECKED   taps outside the image are detected per load and read as zero (tile kernel only).
//
// u8 activations: the MFMA multiplies signed bytes, so activations are fed as (a ^ 0x80) = a - 128
// and the accumulators start from 128 * sum(w[f]) (+ the int32 bias), which is exact in int32.
//
// Weight rows are stored permuted inside each 64-feature span so that a lane's 16 accumulators
// of one pixel are 16 CONSECUTIVE features: the int8 result is written with one 128-bit store.
#pragma once
#include <mutex>

#include "epilogue.h"
#include "kernels.h"

namespace chip {

typedef int v4i __attribute__((ext_vector_type(4)));

// q = n / d for 0 <= n < 2^31 by multiply-high and shift
struct FastDiv {
    uint32_t mul, shift, one;
    __device__ __forceinline__ uint32_t div(uint32_t n) const { return one ? n : (__umulhi(n, mul) >> shift); }
};

FastDiv make_fast_div(uint32_t d);  // host

struct MfmaArgs {
    const int8_t* in;
    const v4i* wpk;
    const int32_t* ktab;
    const int32_t* acc_init;  // [ofm_tiles * BN], natural feature order, zero padded
    void* out;
    const void* eltw;
    int32_t* raw;
    uint32_t M;
    int32_t OFM, ofm_tiles, mtiles;
    int32_t OHW, OW, OH, IH, IW;
    FastDiv div_ohw, div_ow;
    int32_t sy, sx, py, px, esy, esx;
    int32_t in_off, in_pb, in_pf, in_py;       // bytes
    int32_t out_off, out_pb, out_pf, out_py;   // elements
    int32_t el_off, el_pb, el_pf, el_py;       // elements
    int32_t ksteps;
    // streaming kernel: tap offsets by arithmetic, dense-tensor shortcut
    int32_t CB, FX, kchunks, tap_dy, tap_dx, linear;
    // weights-stationary kernel: pixel-tile partitions per feature tile, tiles per partition, filter rows
    int32_t wsl_parts, wsl_tpp, FY;
    // 1: the eight accelerator dies split the FEATURE tiles between them (weights are the larger operand)
    int32_t by_features;
    // bytes per pixel of one input slice: 16 (fs_b_yx_fsv16) or 4 (b_fs_yx_fsv4, first layers; streaming kernel only)
    int32_t px_bytes;
    FastDiv div_cb, div_fx;
    // workgroup id -> (pixel tile, feature tile): a plain division of two kernel arguments costs a wave some forty
    // instructions with four trips between the vector and the scalar unit, before its first load is requested
    FastDiv div_mtiles, div_ofm_tiles;
    uint32_t xor_mask;  // 0x80808080 for u8 activations, 0 for s8
    const v4i* bpk;     // small-batch kernel: scratch for the activations in fragment order (nullptr: read them in place)
    FastEpi fe;
    Epilogue epi;
};

// epilogue kinds.  GENERIC: every mode and output type, element by element.  FAST: int8 output in the
// float-requantisation mode, options chosen by run-time flags.  RELU / FUSED: the two forms the ResNet /
// VGG stacks consist of, with nothing left to decide at run time:
//   RELU   clamp(acc * cal, 0, hi)                                    (relu, scales >= 0, unit wqf)
//   FUSED  clamp((round(acc * cal) + residual) * ecal, 0, hi)         (residual relu, scales >= 0)
//   LINEAR clamp(acc * cal, lo, hi)                                   (no activation, unit wqf; with two convolutions in one
//                                                                      launch lo is 0 for the features of the one with a relu)
//   CLAMPQ clamp(acc * wqf, m, n) * cal, rounded                      (folded clamp{m, n} with 0 <= m, e.g. ReLU6 on the
//                                                                      dequantised value; unit input factor; chain kernels)
//   SUMLIN clamp((sat(round(acc * cal)) + residual) * ecal, lo, hi)    (residual sum without activation, the rounded
//                                                                      convolution result optionally saturated first, unit
//                                                                      wqf; a MobileNet projection; chain kernels)
enum { EPI_KIND_GENERIC = 0, EPI_KIND_FAST = 1, EPI_KIND_RELU = 2, EPI_KIND_FUSED = 3, EPI_KIND_LINEAR = 4, EPI_KIND_CLAMPQ = 5,
       EPI_KIND_SUMLIN = 6 };
template <int EPI> struct epi_is_short { static constexpr bool value = EPI != EPI_KIND_GENERIC; };

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains every outstanding
// global load (loads and stores share one counter on this architecture), which would serialise the
// K loop on memory latency; the K loop shares nothing through global memory.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// Keeps the instruction scheduler from moving work across the boundary of two K-steps.  Without it the
// compiler hoists register-only work on the operands of a LATE step (the sign flip of u8 activations) to the
// top of the unrolled loop, which makes it wait for the newest outstanding load there and drains the whole
// look-ahead queue once per loop iteration.
__device__ __forceinline__ void step_fence() { __builtin_amdgcn_sched_barrier(0); }

// Instruction order inside one K-step: after each of the M matrix instructions (16 clocks in the matrix pipe, 4 to
// issue) the scheduler is told to place a share of the step's other work -- R LDS reads, W LDS writes, V global
// loads, VALU register work -- so that it issues in the shadow of the matrix pipe instead of in front of it.  The
// memory operations go behind the first half of the matrix instructions, so that their latency has passed when the
// step ends in a wait and a barrier.
template <int I, int M, int R, int W, int V, int VALU>
__device__ __forceinline__ void interleave_step()
{
    if constexpr (I < M) {
        constexpr int H = (M + 1) / 2;  // slots that take memory operations
        constexpr int i0 = I < H ? I : H, i1 = I + 1 < H ? I + 1 : H;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        constexpr int r = i1 * R / H - i0 * R / H, w = i1 * W / H - i0 * W / H, v = i1 * V / H - i0 * V / H;
        constexpr int va = (I + 1) * VALU / M - I * VALU / M;
        if constexpr (w > 0) __builtin_amdgcn_sched_group_barrier(0x200, w, 0);
        if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);
        if constexpr (v > 0) __builtin_amdgcn_sched_group_barrier(0x020, v, 0);
        if constexpr (va > 0) __builtin_amdgcn_sched_group_barrier(0x002, va, 0);
        interleave_step<I + 1, M, R, W, V, VALU>();
    }
}

// A load whose value is never used: it brings the line towards the CU while other work runs, so that the real load
// later hits in cache.  The loaded register must stay reserved until the load has landed: keep_until_here(token) goes
// behind a point where younger loads have been waited for (loads complete in order).
__device__ __forceinline__ int touch_line(const void* p)
{
    int token;
    asm volatile("global_load_dword %0, %1, off" : "=v"(token) : "v"(p) : "memory");
    return token;
}
__device__ __forceinline__ void keep_until_here(int token) { asm volatile("" ::"v"(token)); }

// The epilogue's per-feature factors of features [f_base, f_base + BN) (BN <= 128): one touch covers 512 bytes.
struct EarlyTouch {
    int t0, t1;
};
template <int BN, int EPI, class Args>
__device__ __forceinline__ EarlyTouch touch_scales(const Args& a, int f_base, int lane)
{
    EarlyTouch e{0, 0};
    if constexpr (EPI == EPI_KIND_RELU || EPI == EPI_KIND_FUSED || EPI == EPI_KIND_LINEAR) {
        const int f = f_base + ((lane * 2) & (BN - 1));
        e.t0 = touch_line(a.epi.calib + f);
        if constexpr (EPI == EPI_KIND_FUSED) e.t1 = touch_line(a.epi.eltw_calib + f);
    }
    return e;
}
__device__ __forceinline__ void keep_until_here(const EarlyTouch& e)
{
    keep_until_here(e.t0);
    keep_until_here(e.t1);
}

// Uniform table lookups go through the scalar data path (constant address space): a vector load here
// would sit in the same in-order counter as the prefetched operand loads and force them to drain.
typedef const int32_t __attribute__((address_space(4))) * const_i32_ptr;
__device__ __forceinline__ int32_t scalar_table_load(const int32_t* table, int index)
{
    return ((const_i32_ptr)(uintptr_t)table)[index];
}

__device__ __forceinline__ float rha(float v) { return truncf(v + copysignf(0.49999997f, v)); }
// median of three: one instruction; equals min(max(x, lo), hi) for lo <= hi and x not NaN
__device__ __forceinline__ float med3(float x, float lo, float hi) { return __builtin_amdgcn_fmed3f(x, lo, hi); }
__device__ __forceinline__ float relu1(float x) { return __builtin_amdgcn_fmed3f(x, 0.0f, __builtin_inff()); }

// Sixteen values inside [0, 255.5) -> four dwords of bytes, one instruction per value.  v_cvt_pk_u8_f32 converts with
// the wave's rounding mode and inserts the byte into a dword; with the mode set to round-toward-zero it gives, for every
// float from -inf to +inf, what the truncating conversion of the value clamped to [0, 255] gives (all 2^32 bit patterns
// but the NaNs were compared on the device).  Only the conversions run in that mode: the first asm takes every value as
// an input, so the arithmetic that made them (rounded to nearest even, as the reference's) is complete before the mode
// changes, and it hands out the zero that every dword starts from, so no conversion can start before it; the second asm
// takes the four dwords.  The scheduling fences keep unrelated float arithmetic of the surrounding code out of the window.
__device__ __forceinline__ void pack_nonneg16(const float (&v)[16], v4i& packed)
{
    unsigned w0, w1, w2, w3;
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 3\n\tv_mov_b32 %0, 0"
                 : "=v"(w0)
                 : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]), "v"(v[8]), "v"(v[9]),
                   "v"(v[10]), "v"(v[11]), "v"(v[12]), "v"(v[13]), "v"(v[14]), "v"(v[15]));
    w1 = w2 = w3 = w0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        w0 = __builtin_amdgcn_cvt_pk_u8_f32(v[i], i, w0);
        w1 = __builtin_amdgcn_cvt_pk_u8_f32(v[4 + i], i, w1);
        w2 = __builtin_amdgcn_cvt_pk_u8_f32(v[8 + i], i, w2);
        w3 = __builtin_amdgcn_cvt_pk_u8_f32(v[12 + i], i, w3);
    }
    asm volatile("s_setreg_imm32_b32 hwreg(HW_REG_MODE, 0, 2), 0" : "+v"(w0), "+v"(w1), "+v"(w2), "+v"(w3));
    __builtin_amdgcn_sched_barrier(0);
    packed[0] = (int)w0, packed[1] = (int)w1, packed[2] = (int)w2, packed[3] = (int)w3;
}
// four values inside [-128, 255] -> one dword of bytes
__device__ __forceinline__ int pack_signed(const float* v)
{
    const unsigned q0 = (unsigned)(int)v[0] & 255u, q1 = (unsigned)(int)v[1] & 255u, q2 = (unsigned)(int)v[2] & 255u;
    const unsigned q3 = (unsigned)(int)v[3];
    return (int)(q0 | (q1 << 8) | (q2 << 16) | (q3 << 24));
}

// Placed at the top of a conditional block of plain arithmetic, this keeps the branch a branch.  Without it the
// compiler evaluates the block for every value whatever the condition says and selects afterwards: three extra
// instructions per output for the two residual types, two and a half for the mask below.
__device__ __forceinline__ void keep_branch() { asm volatile(""); }

// partly filled last feature slice: the padding features stay zero
__device__ __forceinline__ void zero_padding_features(v4i& packed, int valid)
{
    if (valid < 16) {
        // the masks depend on `valid` alone; unless it passes through the asm they are computed ahead of the branch, for
        // every wave (16 compares and selects), whether a slice is partly filled or not
        asm volatile("" : "+v"(valid));
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            unsigned keep = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (d * 4 + i < valid) keep |= 255u << (8 * i);
            packed[d] &= (int)keep;
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Short epilogue for int8 outputs in the float-requantisation mode.  Same operations in the same
// order as the long form, with three exact rewrites: "round then saturate" becomes "clamp then round"
// (the bounds are integers), round-half-away is trunc(x + copysign(0.49999997f, x)), and
// max(0, x) * s becomes clamp(x * s, 0, hi) when s >= 0.  The truncating float->int conversion
// completes the rounding.
template <int NT, int EPI, class Args>
__device__ __forceinline__ v4i epilogue_fast16(const Args& a, const v4i (&acc)[4][NT], int nt, const float (&wq)[16],
                                               const float (&cal)[16], const float (&ecal)[16], const v4i& ev4,
                                               int valid)
{
    const FastEpi& F = a.fe;
    float v[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) v[c] = (float)acc[c >> 2][nt][c & 3];
    if constexpr (EPI == EPI_KIND_LINEAR) {
        v4i packed;
        const float lo = valid <= F.split_valid ? F.lo2 : F.lo;
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const float y = med3(v[c] * cal[c], lo, F.hi);
            v[c] = y + copysignf(0.49999997f, y);
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) packed[d] = pack_signed(v + d * 4);
        zero_padding_features(packed, valid);
        return packed;
    }
    if constexpr (EPI == EPI_KIND_SUMLIN) {
        // the run-time form's steps for a sum without activation, in the same order; ecal[] holds ones where the sum has
        // no calibration factors
        v4i packed;
        // without the saturation the bounds are infinite: one instruction that changes nothing instead of a select
        const float clo = F.conv_sat ? F.conv_lo : -__builtin_inff(), chi = F.conv_sat ? F.conv_hi : __builtin_inff();
        float e[16];
        if (F.eltw_u8) {
            keep_branch();
#pragma unroll
            for (int c = 0; c < 16; ++c) e[c] = (float)(((unsigned)ev4[c >> 2] >> (8 * (c & 3))) & 255u);
        } else {
            keep_branch();
#pragma unroll
            for (int c = 0; c < 16; ++c) e[c] = (float)(int)(int8_t)((unsigned)ev4[c >> 2] >> (8 * (c & 3)));
        }
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            const float r = med3(rha(v[c] * cal[c]), clo, chi);
            const float y = med3((r + e[c]) * ecal[c], F.lo, F.hi);
            v[c] = y + copysignf(0.49999997f, y);
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) packed[d] = pack_signed(v + d * 4);
        zero_padding_features(packed, valid);
        return packed;
    }
    if constexpr (EPI == EPI_KIND_CLAMPQ) {
        // clamp{m, n} on the dequantised value, then the calibration: the result lies in [0, n * factor], which the host
        // has checked to be inside the output range (the clamp_folded case of the run-time form below)
        v4i packed;
#pragma unroll
        for (int c = 0; c < 16; ++c) v[c] = med3(v[c] * wq[c], F.act_m, F.act_n) * cal[c] + 0.49999997f;
        pack_nonneg16(v, packed);
        zero_padding_features(packed, valid);
        return packed;
    }
    if constexpr (EPI == EPI_KIND_RELU || EPI == EPI_KIND_FUSED) {
        v4i packed;
        if constexpr (EPI == EPI_KIND_RELU) {
#pragma unroll
            for (int c = 0; c < 16; ++c) v[c] = med3(v[c] * cal[c], 0.0f, F.hi) + 0.49999997f;
        } else {
            if (F.eltw_u8) {
                keep_branch();
#pragma unroll
                for (int c = 0; c < 16; ++c)
                    v[c] = rha(v[c] * cal[c]) + (float)(((unsigned)ev4[c >> 2] >> (8 * (c & 3))) & 255u);
            } else {
                keep_branch();
#pragma unroll
                for (int c = 0; c < 16; ++c)
                    v[c] = rha(v[c] * cal[c]) + (float)(int)(int8_t)((unsigned)ev4[c >> 2] >> (8 * (c & 3)));
            }
#pragma unroll
            for (int c = 0; c < 16; ++c) v[c] = med3(v[c] * ecal[c], 0.0f, F.hi) + 0.49999997f;
        }
        pack_nonneg16(v, packed);
        zero_padding_features(packed, valid);
        return packed;
    }
    if (F.has_wqf) {
        if (F.iqf_one) {
#pragma unroll
            for (int c = 0; c < 16; ++c) v[c] = v[c] * wq[c];
        } else {
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                v[c] = v[c] * wq[c];
                v[c] = v[c] * F.iqf;
            }
        }
    }
    v4i packed;
    bool finished = false;
    if (F.clamp_folded) {
        // clamp{m, n} on the dequantised value (ReLU6), then the calibration: the result lies in [0, n * factor], which
        // the host has checked to be inside the output range
#pragma unroll
        for (int c = 0; c < 16; ++c) v[c] = med3(v[c], F.act_m, F.act_n) * cal[c] + 0.49999997f;
        pack_nonneg16(v, packed);
    } else if (F.fc) {
        // reference fully_connected_gpu_bfyx_ref.cl:63-84: (char)round((acc * wqf * iqf + bias) * factor), then the
        // activation on the char; ecal[] holds the bias
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            unsigned word = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = d * 4 + i;
                float x = v[c] + ecal[c];
                x = x * cal[c];
                int q = (int)(signed char)(int)rha(x);
                if (F.act == CLDNN_HIP_ACT_RELU) q = q > 0 ? q : 0;
                word |= ((unsigned)q & 255u) << (8 * i);
            }
            packed[d] = (int)word;
        }
    } else if (F.relu_folded) {
#pragma unroll
        for (int c = 0; c < 16; ++c) v[c] = med3(v[c] * cal[c], 0.0f, F.hi) + 0.49999997f;
        pack_nonneg16(v, packed);
    } else {
        if (F.act == CLDNN_HIP_ACT_RELU) {
#pragma unroll
            for (int c = 0; c < 16; ++c) v[c] = relu1(v[c]);
        } else if (F.act == CLDNN_HIP_ACT_CLAMP) {
#pragma unroll
            for (int c = 0; c < 16; ++c) v[c] = med3(v[c], F.act_m, F.act_n);
        }
#pragma unroll
        for (int c = 0; c < 16; ++c) v[c] = v[c] * cal[c];
        if (F.fused) {
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                float r = rha(v[c]);
                if (F.conv_sat) r = med3(r, F.conv_lo, F.conv_hi);
                const unsigned word = (unsigned)ev4[c >> 2];
                const float e = F.eltw_u8 ? (float)((word >> (8 * (c & 3))) & 255u)
                                          : (float)(int)(int8_t)(word >> (8 * (c & 3)));
                v[c] = r + e;
            }
            if (F.eltw_relu_folded) {
#pragma unroll
                for (int c = 0; c < 16; ++c) v[c] = med3(v[c] * ecal[c], 0.0f, F.hi) + 0.49999997f;
                pack_nonneg16(v, packed);
                finished = true;
            } else if (F.eltw_act == CLDNN_HIP_ACT_RELU) {
#pragma unroll
                for (int c = 0; c < 16; ++c) v[c] = relu1(v[c]);
            } else if (F.eltw_act == CLDNN_HIP_ACT_CLAMP) {
#pragma unroll
                for (int c = 0; c < 16; ++c) v[c] = med3(v[c], F.eltw_m, F.eltw_n);
            }
            if (!finished && F.has_ecal) {
#pragma unroll
                for (int c = 0; c < 16; ++c) v[c] = v[c] * ecal[c];
            }
        }
        if (!finished) {
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                const float y = med3(v[c], F.lo, F.hi);
                v[c] = y + copysignf(0.49999997f, y);
            }
#pragma unroll
            for (int d = 0; d < 4; ++d) packed[d] = pack_signed(v + d * 4);
        }
    }
    zero_padding_features(packed, valid);
    return packed;
}

// per-lane requantisation factors of the 16 features a lane finishes
struct LaneScales {
    float wq[16], cal[16], ecal[16];
};

template <int EPI, class Args>
__device__ __forceinline__ void load_scales(const Args& a, int f0, LaneScales& sc)
{
    if constexpr (EPI == EPI_KIND_RELU || EPI == EPI_KIND_FUSED || EPI == EPI_KIND_LINEAR) {
        // these kinds are only chosen when the vectors they read exist
        const Epilogue& e = a.epi;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const float4 c4 = *reinterpret_cast<const float4*>(e.calib + f0 + d * 4);
            sc.cal[d * 4 + 0] = c4.x, sc.cal[d * 4 + 1] = c4.y, sc.cal[d * 4 + 2] = c4.z, sc.cal[d * 4 + 3] = c4.w;
            if constexpr (EPI == EPI_KIND_FUSED) {
                const float4 e4 = *reinterpret_cast<const float4*>(e.eltw_calib + f0 + d * 4);
                sc.ecal[d * 4 + 0] = e4.x, sc.ecal[d * 4 + 1] = e4.y, sc.ecal[d * 4 + 2] = e4.z, sc.ecal[d * 4 + 3] = e4.w;
            }
        }
    } else if constexpr (EPI == EPI_KIND_FAST) {
        const Epilogue& e = a.epi;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            float4 c4 = {1.f, 1.f, 1.f, 1.f}, w4 = c4, e4 = c4;
            if (e.calib) c4 = *reinterpret_cast<const float4*>(e.calib + f0 + d * 4);
            else if (e.oqf_on) c4 = make_float4(e.oqf, e.oqf, e.oqf, e.oqf);
            if (a.fe.has_wqf) w4 = *reinterpret_cast<const float4*>(e.wqf + f0 + d * 4);
            if (a.fe.has_ecal) e4 = *reinterpret_cast<const float4*>(e.eltw_calib + f0 + d * 4);
            if (a.fe.fc) e4 = *reinterpret_cast<const float4*>((const float*)e.bias + f0 + d * 4);  // never fused: the slot is free
            sc.cal[d * 4 + 0] = c4.x, sc.cal[d * 4 + 1] = c4.y, sc.cal[d * 4 + 2] = c4.z, sc.cal[d * 4 + 3] = c4.w;
            sc.wq[d * 4 + 0] = w4.x, sc.wq[d * 4 + 1] = w4.y, sc.wq[d * 4 + 2] = w4.z, sc.wq[d * 4 + 3] = w4.w;
            sc.ecal[d * 4 + 0] = e4.x, sc.ecal[d * 4 + 1] = e4.y, sc.ecal[d * 4 + 2] = e4.z, sc.ecal[d * 4 + 3] = e4.w;
        }
    }
}

// Finish the 16 features [f0, f0+16) of one pixel held in acc[.][nt] and store them.
// obase / ebase: element offsets of (pixel, feature slice) in the output / residual tensor.
template <int NT, int EPI>
__device__ __forceinline__ void finish_pixel(const MfmaArgs& a, const v4i (&acc)[4][NT], int nt, int f0, int valid,
                                             int obase, int ebase, const LaneScales& sc, const v4i& ev4, uint32_t b,
                                             uint32_t oy, uint32_t ox)
{
    const Epilogue& e = a.epi;
    if constexpr (EPI != EPI_KIND_GENERIC) {
        const v4i packed = epilogue_fast16<NT, EPI>(a, acc, nt, sc.wq, sc.cal, sc.ecal, ev4, valid);
        *reinterpret_cast<v4i*>((int8_t*)a.out + obase) = packed;
    } else {
        if (a.raw) {
#pragma unroll
            for (int c = 0; c < 16; ++c)
                if (c < valid) a.raw[(((size_t)b * a.OFM + f0 + c) * a.OH + oy) * a.OW + ox] = acc[c >> 2][nt][c & 3];
        } else {
            const bool out8 = e.out_dt == CLDNN_HIP_S8 || e.out_dt == CLDNN_HIP_U8;
            v4i packed = {0, 0, 0, 0};
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                EpiOut o;
                o.f = 0.f, o.i = 0;
                if (c < valid) {
                    float ev = 0.f;
                    if (e.fused) ev = load_as_float(a.eltw, e.eltw_dt, ebase + c);
                    o = epilogue_generic(e, acc[c >> 2][nt][c & 3], f0 + c, ev);
                }
                if (out8) packed[c >> 2] |= (int)(((unsigned)o.i & 255u) << (8 * (c & 3)));
                else store_out(a.out, e.out_dt, obase + c, o);
            }
            if (out8) *reinterpret_cast<v4i*>((int8_t*)a.out + obase) = packed;
        }
    }
}

struct PixelPos {
    uint32_t b, oy, ox;
};

// Everything a kernel reads from the argument block, fetched behind one wait.  Left to itself the compiler fetches an
// argument where it is first used, and a wave makes five or six dependent round trips to memory (a few hundred
// nanoseconds each) before its first operand request goes out, and one or two more in front of its epilogue.
__device__ __forceinline__ void fetch_arguments(const MfmaArgs& a)
{
    asm volatile("" ::"s"(a.in), "s"(a.wpk), "s"(a.ktab), "s"(a.acc_init), "s"(a.out), "s"(a.eltw), "s"(a.M), "s"(a.OFM),
                 "s"(a.ofm_tiles), "s"(a.mtiles), "s"(a.OHW), "s"(a.OW), "s"(a.div_ohw.mul), "s"(a.div_ohw.shift),
                 "s"(a.div_ohw.one), "s"(a.div_ow.mul), "s"(a.div_ow.shift), "s"(a.div_ow.one), "s"(a.sy), "s"(a.sx), "s"(a.py),
                 "s"(a.px), "s"(a.esy), "s"(a.esx));
    asm volatile("" ::"s"(a.in_off), "s"(a.in_pb), "s"(a.in_pf), "s"(a.in_py), "s"(a.out_off), "s"(a.out_pb), "s"(a.out_pf),
                 "s"(a.out_py), "s"(a.el_off), "s"(a.el_pb), "s"(a.el_pf), "s"(a.el_py), "s"(a.ksteps), "s"(a.CB), "s"(a.FX),
                 "s"(a.kchunks), "s"(a.tap_dy), "s"(a.tap_dx), "s"(a.linear), "s"(a.px_bytes), "s"(a.by_features));
    asm volatile("" ::"s"(a.div_cb.mul), "s"(a.div_cb.shift), "s"(a.div_cb.one), "s"(a.div_fx.mul), "s"(a.div_fx.shift),
                 "s"(a.div_fx.one), "s"(a.div_mtiles.mul), "s"(a.div_mtiles.shift), "s"(a.div_mtiles.one), "s"(a.div_ofm_tiles.mul),
                 "s"(a.div_ofm_tiles.shift), "s"(a.div_ofm_tiles.one), "s"(a.xor_mask), "s"(a.wsl_parts), "s"(a.wsl_tpp), "s"(a.FY),
                 "s"(a.epi.calib), "s"(a.epi.eltw_calib), "s"(a.epi.wqf), "s"(a.fe.hi), "s"(a.fe.lo));
}

__device__ __forceinline__ PixelPos pixel_pos(const MfmaArgs& a, uint32_t m)
{
    PixelPos p;
    p.b = a.div_ohw.div(m);
    const uint32_t r = m - p.b * a.OHW;
    p.oy = a.div_ow.div(r);
    p.ox = r - p.oy * a.OW;
    return p;
}

// =====================================================================================================
// LDS-staged tile kernel (long K: 3x3 and wide 1x1 layers)
// =====================================================================================================
// K-steps of global-load lookahead in the tile kernel, by 16-byte loads per thread and step (even)
#define MFMA_PREFETCH_DISTANCE(loads) ((loads) <= 2 ? 8 : ((loads) <= 4 ? 4 : 2))

template <int BM, int BN, int WP, bool CHECKED, int EPI>
__global__ void __launch_bounds__(256) conv_mfma_kernel(MfmaArgs a)
{
    fetch_arguments(a);
    constexpr int NT = WP / 16;         // pixel tiles per wave
    constexpr int WAVES_F = BN / 64;    // waves along features
    constexpr int A_LOADS = BN / 64;    // 16-byte weight chunks per thread per K-step
    constexpr int B_LOADS = BM / 64;    // 16-byte activation chunks per thread per K-step
    constexpr int KC_STRIDE = 256 / BM; // k-chunk distance between a thread's activation loads
    static_assert((BM / WP) * WAVES_F == 4, "tile must map onto 4 waves");

    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wave_f = wave % WAVES_F;
    const int wave_p = wave / WAVES_F;
    const int kq = lane >> 4;
    const int l16 = lane & 15;

    // Workgroup ids are dealt round-robin to the eight accelerator dies, each with its own L2 that starts
    // cold.  The dies split the tiles of the SMALLER operand's counterpart between them, so the larger operand
    // is fetched from memory once in total and only the smaller one once per die: by default a die takes every
    // eighth pixel tile with all its feature tiles (adjacent in time, they share the activations through L2);
    // with by_features it takes every eighth feature tile with all pixel tiles (sharing the weights).
    const int xcd = blockIdx.x & 7;
    const int j = blockIdx.x >> 3;
    const int j_by_m = (int)a.div_mtiles.div((uint32_t)j), j_by_f = (int)a.div_ofm_tiles.div((uint32_t)j);
    const int ptile = a.by_features ? j - j_by_m * a.mtiles : j_by_f * 8 + xcd;
    const int ntile = a.by_features ? j_by_m * 8 + xcd : j - j_by_f * a.ofm_tiles;
    if (ptile >= a.mtiles || ntile >= a.ofm_tiles) return;
    const uint32_t m0 = (uint32_t)ptile * BM;

    v4i acc[4][NT];
    {
        const int fbase = ntile * BN + wave_f * 64 + kq * 16;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
            const v4i init = *reinterpret_cast<const v4i*>(a.acc_init + fbase + mt * 4);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = init;
        }
    }
    const v4i xm = {(int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask};

    extern __shared__ __align__(16) unsigned char smem[];
    v4i* ldsA = reinterpret_cast<v4i*>(smem);               // [2][4 * BN]
    v4i* ldsB = reinterpret_cast<v4i*>(smem) + 2 * 4 * BN;  // [2][4 * BM]

    const int lp = t % BM;
    const int kc0 = __builtin_amdgcn_readfirstlane(t / BM);
    const bool ld_valid = m0 + lp < a.M;
    int iy0, ix0, pix_off;
    {
        const PixelPos pp = pixel_pos(a, ld_valid ? m0 + lp : 0);
        iy0 = (int)pp.oy * a.sy - a.py;
        ix0 = (int)pp.ox * a.sx - a.px;
        pix_off = a.in_off + (int)pp.b * a.in_pb + iy0 * a.in_py + ix0 * 16;
    }
    const v4i* wsrc = a.wpk + (size_t)ntile * a.ksteps * (4 * BN) + t;

    // Global loads run D K-steps ahead of the multiply: D register sets in rotation.  With one workgroup
    // per CU (small layers) nothing else hides the memory latency, so the distance has to.  The main loop
    // is free of branches (the weight stream and the tap table carry D+1 zero steps of slack), which lets
    // the compiler wait for exactly the oldest set instead of draining the queue.
    constexpr int D = MFMA_PREFETCH_DISTANCE(A_LOADS + B_LOADS);
    v4i ra[D][A_LOADS], rb[D][B_LOADS];
    auto load_global = [&](int ks, v4i (&xa)[A_LOADS], v4i (&xb)[B_LOADS]) {
#pragma unroll
        for (int q = 0; q < A_LOADS; ++q) xa[q] = wsrc[(size_t)ks * (4 * BN) + q * 256];
#pragma unroll
        for (int q = 0; q < B_LOADS; ++q) {
            const int e = scalar_table_load(a.ktab, ks * 4 + kc0 + q * KC_STRIDE);
            if constexpr (!CHECKED) {
                xb[q] = *reinterpret_cast<const v4i*>(a.in + (pix_off + e));
            } else {
                const int iy = iy0 + (e & 1023), ix = ix0 + ((e >> 10) & 1023);
                const int cb = (e >> 20) & 2047;
                const bool ok = ld_valid && e >= 0 && iy >= 0 && iy < a.IH && ix >= 0 && ix < a.IW;
                v4i v = {0, 0, 0, 0};
                if (ok)
                    v = *reinterpret_cast<const v4i*>(a.in + (pix_off + cb * a.in_pf + (e & 1023) * a.in_py
                                                              + ((e >> 10) & 1023) * 16));
                xb[q] = v;
            }
        }
    };
    auto store_lds = [&](int buf, const v4i (&xa)[A_LOADS], const v4i (&xb)[B_LOADS]) {
#pragma unroll
        for (int q = 0; q < A_LOADS; ++q) ldsA[buf * 4 * BN + t + q * 256] = xa[q];
#pragma unroll
        for (int q = 0; q < B_LOADS; ++q) ldsB[buf * 4 * BM + (kc0 + q * KC_STRIDE) * BM + lp] = xb[q];
    };
    const int arow = wave_f * 64 + l16;
    const int bcol = wave_p * WP + l16;
    auto compute = [&](int buf) {
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
    };

#pragma unroll
    for (int d = 0; d < D; ++d) load_global(d, ra[d], rb[d]);
    store_lds(0, ra[0], rb[0]);
    load_global(D, ra[0], rb[0]);
    lds_barrier();
    const int main_steps = (a.ksteps / D) * D;
    for (int ks0 = 0; ks0 < main_steps; ks0 += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int ks = ks0 + d;
            compute(d & 1);  // D is even: the LDS buffer of step ks is ks & 1 == d & 1
            // K-step ks+1 sits in set (d+1)%D, requested D-1 steps ago; refill the set with step ks+1+D
            store_lds((d & 1) ^ 1, ra[(d + 1) % D], rb[(d + 1) % D]);
            load_global(ks + 1 + D, ra[(d + 1) % D], rb[(d + 1) % D]);
            lds_barrier();
            step_fence();
        }
    }
    const int rest = a.ksteps - main_steps;  // < D steps left; their operands are already on the way
#pragma unroll
    for (int d = 0; d < D - 1; ++d) {
        if (d < rest) {
            compute(d & 1);
            store_lds((d & 1) ^ 1, ra[(d + 1) % D], rb[(d + 1) % D]);
            lds_barrier();
            step_fence();
        }
    }

    // ---- epilogue: lane (kq, l16) holds, for each pixel tile, features f0 .. f0+15 of one pixel
    const int f0 = ntile * BN + wave_f * 64 + kq * 16;
    if (f0 >= a.OFM) return;
    const int fs = f0 >> 4;
    const int valid = a.OFM - f0;  // >= 16 except in the last, partly filled slice
    LaneScales sc;
    load_scales<EPI>(a, f0, sc);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const uint32_t m = m0 + wave_p * WP + nt * 16 + l16;
        if (m < a.M) {
            const PixelPos pp = pixel_pos(a, m);
            const int obase = a.out_off + (int)pp.b * a.out_pb + fs * a.out_pf + (int)pp.oy * a.out_py + (int)pp.ox * 16;
            const int ebase = a.el_off + (int)pp.b * a.el_pb + fs * a.el_pf + (int)(pp.oy * a.esy) * a.el_py
                              + (int)(pp.ox * a.esx) * 16;
            v4i ev4 = {0, 0, 0, 0};
            if constexpr (EPI == EPI_KIND_FUSED) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
            else if constexpr (EPI == EPI_KIND_FAST)
                if (a.fe.fused) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
            finish_pixel<NT, EPI>(a, acc, nt, f0, valid, obase, ebase, sc, ev4, pp.b, pp.oy, pp.ox);
        }
    }
}

// =====================================================================================================
// Direct-activation tile kernel (long K, input with a zero border, feature slices a multiple of 4)
// =====================================================================================================
// Same output tile and weight stream as the LDS-staged kernel, but only the WEIGHTS go through LDS.  A wave
// owns 16*NT pixels and ALL BN features of the tile, so its activation fragments are private to it: lane
// (kq, l16) loads the 16 bytes of slice s0+kq of its pixel straight from global memory into the register
// the MFMA reads (per K-step: one scalar tap offset + one per-lane 32-bit offset, no address arithmetic in
// the vector unit).  Against the LDS-staged kernel this removes the activation store + load through LDS and
// makes every weight fragment read from LDS feed NT matrix instructions: with BN = 64 a wave issues 4 LDS
// reads per 4*NT MFMAs (the LDS-staged 64x64 tile: 5 reads per 4 MFMAs), so the LDS pipe stops being the bound.
#define BDIR_PREFETCH_DISTANCE(loads) ((loads) <= 3 ? 8 : ((loads) <= 4 ? 6 : 4))

template <int BN, int NT, int KG, int EPI>
__global__ void __launch_bounds__(256 * KG) conv_bdir_kernel(MfmaArgs a)
{
    fetch_arguments(a);
    constexpr int MT = BN / 16;       // weight fragments (16 features each) per wave and K-step
    constexpr int SPANS = BN / 64;
    constexpr int WP = NT * 16;       // pixels per wave
    constexpr int BM = 4 * WP;        // pixels per workgroup
    constexpr int A_LOADS = BN / 64;  // 16-byte weight chunks per thread per K-step
    // 64 pixels x 128 features per wave: 128 accumulators.  It is the smallest wave tile that leaves both operand paths
    // half empty at full matrix rate (LDS delivers 4096 / pixels bytes per clock, the vector memory path 4096 / features),
    // but only with two waves per SIMD: one wave's own instruction stream does not hide its LDS reads.  To stay under 256
    // registers the look-ahead is three steps and the weight fragments of a step are read when the step starts instead
    // of one step early (the other wave covers the wait).
    constexpr bool LEAN = BN == 128 && NT == 4 && KG == 1;

    // KG groups of four waves split the K-steps of the tile between them and add their partial sums through
    // LDS at the end: long-K layers with few pixels get KG times as many waves per tile to hide latencies with.
    const int t = threadIdx.x & 255;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane((threadIdx.x >> 6) & 3);
    const int grp = KG == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 8);
    const int kq = lane >> 4;
    const int l16 = lane & 15;

    // same workgroup order as the LDS-staged kernel: a die takes every eighth tile of one kind
    const int xcd = blockIdx.x & 7;
    const int j = blockIdx.x >> 3;
    const int j_by_m = (int)a.div_mtiles.div((uint32_t)j), j_by_f = (int)a.div_ofm_tiles.div((uint32_t)j);
    const int ptile = a.by_features ? j - j_by_m * a.mtiles : j_by_f * 8 + xcd;
    const int ntile = a.by_features ? j_by_m * 8 + xcd : j - j_by_f * a.ofm_tiles;
    if (ptile >= a.mtiles || ntile >= a.ofm_tiles) return;
    const uint32_t m0 = (uint32_t)ptile * BM + (uint32_t)wave * WP;

    v4i acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int f = ntile * BN + (mt >> 2) * 64 + kq * 16 + (mt & 3) * 4;
        v4i init = *reinterpret_cast<const v4i*>(a.acc_init + f);
        if (grp != 0) init = v4i{0, 0, 0, 0};
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = init;
    }
    const v4i xm = {(int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask};
    const EarlyTouch early = touch_scales<BN, EPI>(a, ntile * BN, lane);

    extern __shared__ __align__(16) unsigned char smem[];
    v4i* ldsA = reinterpret_cast<v4i*>(smem) + grp * (3 * 4 * BN);  // per group: [3][4 * BN]

    // byte offset of (pixel, slice kq) of each of the lane's pixels; pixels past the end read pixel 0
    uint32_t boff[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const uint32_t m = m0 + nt * 16 + l16;
        const PixelPos pp = pixel_pos(a, m < a.M ? m : 0);
        boff[nt] = (uint32_t)(a.in_off + (int)pp.b * a.in_pb + ((int)pp.oy * a.sy - a.py) * a.in_py
                              + ((int)pp.ox * a.sx - a.px) * 16 + kq * a.in_pf);
    }
    const int steps = a.ksteps / KG;  // the host pads the K-steps to a multiple of KG
    const int step0 = grp * steps;
    const v4i* wsrc = a.wpk + ((size_t)ntile * a.ksteps + step0) * (4 * BN) + t;

    // look-ahead in K-steps for both operands
    // 32 pixels x 128 features per wave with a look-ahead of six steps needs 250-262 registers depending on what the
    // register allocator makes of the prologue, and above 256 the kernel loses its second wave per SIMD (25 % slower):
    // five steps keep it clear of the limit
    constexpr int D = LEAN ? 3 : (BN == 128 && NT == 2 && KG == 1 ? 5 : BDIR_PREFETCH_DISTANCE(A_LOADS + NT));
    constexpr int DA = D;
    v4i ra[DA][A_LOADS], rb[D][NT];
    auto load_a = [&](int ks, v4i (&xa)[A_LOADS]) {
#pragma unroll
        for (int q = 0; q < A_LOADS; ++q) xa[q] = wsrc[(size_t)ks * (4 * BN) + q * 256];
    };
    auto load_b = [&](int ks, v4i (&xb)[NT]) {
        // the four k-chunks of a step are one tap and four consecutive slices: one uniform offset per step
        const int8_t* base = a.in + scalar_table_load(a.ktab, (step0 + ks) * 4);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) xb[nt] = *reinterpret_cast<const v4i*>(base + boff[nt]);
    };
    auto store_a = [&](int buf, const v4i (&xa)[A_LOADS]) {
#pragma unroll
        for (int q = 0; q < A_LOADS; ++q) ldsA[buf * 4 * BN + t + q * 256] = xa[q];
    };
    auto read_a = [&](int buf, v4i (&fa)[MT]) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) fa[mt] = ldsA[buf * 4 * BN + kq * BN + mt * 16 + l16];
    };
    // u8 activations become s8 by flipping the top bit (the accumulators start at 128 * sum of the weights); the flip
    // of step k+1's fragments is done during step k, so a step starts with its matrix instructions
    auto flip = [&](const v4i (&xb)[NT], v4i (&fb)[NT]) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) fb[nt] = xb[nt] ^ xm;
    };
    auto mma = [&](const v4i (&fa)[MT], const v4i (&fb)[NT]) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                acc[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[mt], fb[nt], acc[mt][nt], 0, 0, 0);
    };

    // Set d holds the operands of K-steps d, d+D, ...: activations stay in registers until multiplied; weights
    // pass through a ring of three LDS buffers, written two steps ahead of their use, so that the fragments of
    // step k+1 are read from LDS while the matrix instructions of step k run (one barrier per step).  The loop
    // is branch-free; the weight stream and the tap table carry zero slack for the steps requested past the end.
    if constexpr (LEAN) {
        // The requests go out in the order the loop issues them (weights of step k + 2, activations of step k), each
        // group pinned: the wait at the head of the loop is computed over this path too, and if the scheduler moves one
        // fragment of step 0 to the end of the queue that wait becomes "everything but one", once per trip of the loop.
        load_a(0, ra[0]);
        load_a(1, ra[1]);
        step_fence();
        load_a(2, ra[2]);
        load_b(0, rb[0]);
        step_fence();
        store_a(0, ra[0]);
        store_a(1, ra[1]);
        load_a(3, ra[0]);
        load_b(1, rb[1]);
        step_fence();
        load_a(4, ra[1]);
        load_b(2, rb[2]);
        step_fence();
    } else {
#pragma unroll
        for (int u = 0; u < DA; ++u) load_a(u, ra[u]);
#pragma unroll
        for (int d = 0; d < D; ++d) load_b(d, rb[d]);
        store_a(0, ra[0]);
        store_a(1, ra[1]);
        load_a(DA, ra[0]);
        load_a(DA + 1, ra[1]);
    }
    lds_barrier();
    int b1 = 1, b2 = 2, b0 = 0;  // ring positions of steps k+1, k+2, k
    const int main_steps = (steps / DA) * DA;
    if constexpr (LEAN) {
        v4i fa[MT], fb[NT];
        const int lean_main = (steps / D) * D;
        for (int ks0 = 0; ks0 < lean_main; ks0 += D) {
#pragma unroll
            for (int u = 0; u < D; ++u) {
                const int ks = ks0 + u;
                read_a(b0, fa);
                flip(rb[u], fb);
                mma(fa, fb);
                store_a(b2, ra[(u + 2) % DA]);
                load_a(ks + 2 + DA, ra[(u + 2) % DA]);
                load_b(ks + D, rb[u]);
                lds_barrier();
                step_fence();
                const int tmp = b0;
                b0 = b1, b1 = b2, b2 = tmp;
            }
        }
        const int rest = steps - lean_main;
#pragma unroll
        for (int u = 0; u < D - 1; ++u) {
            if (u < rest) {
                read_a(b0, fa);
                flip(rb[u], fb);
                mma(fa, fb);
                store_a(b2, ra[(u + 2) % DA]);
                lds_barrier();
                step_fence();
                const int tmp = b0;
                b0 = b1, b1 = b2, b2 = tmp;
            }
        }
    } else {
    v4i fa_cur[MT], fa_nxt[MT], fb_cur[NT], fb_nxt[NT];
    read_a(0, fa_cur);
    flip(rb[0], fb_cur);
    for (int ks0 = 0; ks0 < main_steps; ks0 += DA) {
#pragma unroll
        for (int u = 0; u < DA; ++u) {
            const int ks = ks0 + u;
            read_a(b1, fa_nxt);
            mma(fa_cur, fb_cur);
            flip(rb[(u + 1) % D], fb_nxt);
            store_a(b2, ra[(u + 2) % DA]);
            load_a(ks + 2 + DA, ra[(u + 2) % DA]);
            load_b(ks + D, rb[u % D]);
            interleave_step<0, MT * NT, MT, A_LOADS, A_LOADS + NT, NT * 6 + 4>();
            lds_barrier();
            step_fence();
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) fa_cur[mt] = fa_nxt[mt];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) fb_cur[nt] = fb_nxt[nt];
            const int tmp = b0;
            b0 = b1, b1 = b2, b2 = tmp;
        }
    }
    const int rest = steps - main_steps;
#pragma unroll
    for (int u = 0; u < DA - 1; ++u) {
        if (u < rest) {
            read_a(b1, fa_nxt);
            mma(fa_cur, fb_cur);
            flip(rb[(u + 1) % D], fb_nxt);
            store_a(b2, ra[(u + 2) % DA]);
            load_b(main_steps + u + D, rb[u % D]);
            interleave_step<0, MT * NT, MT, A_LOADS, NT, NT * 6 + 4>();
            lds_barrier();
            step_fence();
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) fa_cur[mt] = fa_nxt[mt];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) fb_cur[nt] = fb_nxt[nt];
            const int tmp = b0;
            b0 = b1, b1 = b2, b2 = tmp;
        }
    }
    }

    keep_until_here(early);
    if constexpr (KG > 1) {
        // partial sums of groups 1.. go to LDS as [group - 1][wave][register][lane]; group 0 adds them up
        constexpr int REGS = MT * NT * 4;
        int* part = reinterpret_cast<int*>(smem);
        __syncthreads();  // every group is done with its weight buffers
        if (grp != 0) {
            int* dst = part + ((grp - 1) * 4 + wave) * REGS * 64 + lane;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) dst[((mt * NT + nt) * 4 + i) * 64] = acc[mt][nt][i];
        }
        __syncthreads();
        if (grp != 0) return;
#pragma unroll
        for (int g = 1; g < KG; ++g) {
            const int* src = part + ((g - 1) * 4 + wave) * REGS * 64 + lane;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) acc[mt][nt][i] += src[((mt * NT + nt) * 4 + i) * 64];
        }
    }

    // ---- epilogue: per span of 64 features, lane (kq, l16) holds features f0 .. f0+15 of its pixels
#pragma unroll
    for (int sp = 0; sp < SPANS; ++sp) {
        const int f0 = ntile * BN + sp * 64 + kq * 16;
        if (f0 >= a.OFM) continue;
        const int fs = f0 >> 4;
        const int valid = a.OFM - f0;
        LaneScales sc;
        load_scales<EPI>(a, f0, sc);
        const v4i(&acc_sp)[4][NT] = *reinterpret_cast<const v4i(*)[4][NT]>(&acc[sp * 4]);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const uint32_t m = m0 + nt * 16 + l16;
            if (m < a.M) {
                const PixelPos pp = pixel_pos(a, m);
                const int obase = a.out_off + (int)pp.b * a.out_pb + fs * a.out_pf + (int)pp.oy * a.out_py + (int)pp.ox * 16;
                const int ebase = a.el_off + (int)pp.b * a.el_pb + fs * a.el_pf + (int)(pp.oy * a.esy) * a.el_py
                                  + (int)(pp.ox * a.esx) * 16;
                v4i ev4 = {0, 0, 0, 0};
                if constexpr (EPI == EPI_KIND_FUSED) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
                else if constexpr (EPI == EPI_KIND_FAST)
                    if (a.fe.fused) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
                finish_pixel<NT, EPI>(a, acc_sp, nt, f0, valid, obase, ebase, sc, ev4, pp.b, pp.oy, pp.ox);
            }
        }
    }
}

// =====================================================================================================
// Weights-stationary kernel (input with a zero border, feature slices a multiple of 4, BN * K <= LDS)
// =====================================================================================================
// A persistent workgroup owns ONE tile of 64 output features and a contiguous range of pixel tiles.  It
// copies its whole weight tile (64 x K bytes, already in fragment order) into LDS once; after that the K
// loop has no barrier, no LDS store and no weight traffic from global memory: per K-step a wave reads its
// four weight fragments from LDS (one step ahead of their use), multiplies them with activation fragments
// that come straight from global memory D steps ahead of their use, and the look-ahead runs across pixel
// tiles, so the activations (and the residual) of the next tile are in flight while the current tile is
// requantised and stored.  Requantisation factors, accumulator start values and all pointers stay in
// registers for the lifetime of the wave.  Tap offsets are walked with scalar counters (no table loads).
// K-steps are padded by the host to a multiple of D with zero weights.
struct TapWalk {
    int sg, fx, fy, off;
};
__device__ __forceinline__ void tap_reset(TapWalk& w) { w.sg = 0, w.fx = 0, w.fy = 0, w.off = 0; }
__device__ __forceinline__ void tap_advance(const MfmaArgs& a, TapWalk& w, int cb4)
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

template <int NT, int D, int EPI>
__global__ void __launch_bounds__(256) conv_wsl_kernel(MfmaArgs a)
{
    fetch_arguments(a);
    constexpr int WP = NT * 16;  // pixels per wave and tile
    const int t = threadIdx.x;
    const int lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int kq = lane >> 4;
    const int l16 = lane & 15;

    // partitions of one pixel range that differ in the feature tile get ids congruent modulo 8 and adjacent
    // in time: they run on the same accelerator die and share the activations through its L2
    const int xcd = blockIdx.x & 7;
    const int j = blockIdx.x >> 3;
    const int j_by_f = (int)a.div_ofm_tiles.div((uint32_t)j);
    const int part = j_by_f * 8 + xcd;
    const int ntile = j - j_by_f * a.ofm_tiles;
    const int t_begin = part * a.wsl_tpp;
    const int t_end = min(t_begin + a.wsl_tpp, a.mtiles);
    if (t_begin >= t_end) return;

    extern __shared__ __align__(16) unsigned char smem[];
    v4i* ldsA = reinterpret_cast<v4i*>(smem);  // [ksteps][4][64]
    {
        const v4i* src = a.wpk + (size_t)ntile * a.ksteps * 256;
        const int total = a.ksteps * 256;
        for (int i = t; i < total; i += 8 * 256) {  // eight requests in flight per thread
            v4i r[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) r[u] = src[min(i + u * 256, total - 1)];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (i + u * 256 < total) ldsA[i + u * 256] = r[u];
        }
    }

    const int f0 = ntile * 64 + kq * 16;
    const bool live = f0 < a.OFM;
    const int fs = f0 >> 4;
    const int valid = a.OFM - f0;
    v4i init[4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) init[mt] = *reinterpret_cast<const v4i*>(a.acc_init + f0 + mt * 4);
    LaneScales sc;
    if (live) load_scales<EPI>(a, f0, sc);
    const v4i xm = {(int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask};
    const int cb4 = a.CB >> 2;

    struct TileRefs {
        uint32_t boff[NT];
        int ob[NT], eb[NT];
        PixelPos pos[NT];
    };
    auto setup = [&](int tile, TileRefs& r) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const uint32_t m = ((uint32_t)tile * 4 + (uint32_t)wave) * WP + nt * 16 + l16;
            const bool ok = tile < t_end && m < a.M;
            const PixelPos pp = pixel_pos(a, ok ? m : 0);
            r.boff[nt] = (uint32_t)(a.in_off + (int)pp.b * a.in_pb + ((int)pp.oy * a.sy - a.py) * a.in_py
                                    + ((int)pp.ox * a.sx - a.px) * 16 + kq * a.in_pf);
            const int o = a.out_off + (int)pp.b * a.out_pb + fs * a.out_pf + (int)pp.oy * a.out_py + (int)pp.ox * 16;
            r.ob[nt] = ok && live ? o : -1;
            r.eb[nt] = a.el_off + (int)pp.b * a.el_pb + fs * a.el_pf + (int)(pp.oy * a.esy) * a.el_py
                       + (int)(pp.ox * a.esx) * 16;
            if constexpr (EPI == EPI_KIND_GENERIC) r.pos[nt] = pp;
        }
    };
    auto load_residual = [&](const TileRefs& r, v4i (&ev)[NT]) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            ev[nt] = v4i{0, 0, 0, 0};
            if constexpr (EPI == EPI_KIND_FUSED) {
                if (live) ev[nt] = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + r.eb[nt]);
            } else if constexpr (EPI == EPI_KIND_FAST) {
                if (a.fe.fused && live) ev[nt] = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + r.eb[nt]);
            }
        }
    };
    auto load_b = [&](const TileRefs& r, const TapWalk& w, v4i (&xb)[NT]) {
        const int8_t* base = a.in + (w.fy < a.FY ? w.off : 0);  // padded K-steps read tap 0 (their weights are zero)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) xb[nt] = *reinterpret_cast<const v4i*>(base + r.boff[nt]);
    };
    auto load_a = [&](int ks, v4i (&fa)[4]) {
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) fa[mt] = ldsA[(ks * 4 + kq) * 64 + mt * 16 + l16];
    };

    TileRefs cur, nxt;
    v4i rb[D][NT], ev_cur[NT], ev_nxt[NT], fa_cur[4], fa_nxt[4];
    v4i acc[4][NT];
    TapWalk walk;  // tap of the next activation request
    setup(t_begin, cur);
    tap_reset(walk);
#pragma unroll
    for (int d = 0; d < D; ++d) {
        load_b(cur, walk, rb[d]);
        tap_advance(a, walk, cb4);
    }
    load_residual(cur, ev_cur);
    __syncthreads();  // the weight tile is in LDS
    load_a(0, fa_cur);

    auto step = [&](int ks, int d, const TileRefs& refill_from) {
        load_a(ks + 1 < a.ksteps ? ks + 1 : 0, fa_nxt);
        v4i fb[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) fb[nt] = rb[d][nt] ^ xm;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                acc[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa_cur[mt], fb[nt], acc[mt][nt], 0, 0, 0);
        load_b(refill_from, walk, rb[d]);
        tap_advance(a, walk, cb4);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) fa_cur[mt] = fa_nxt[mt];
        step_fence();
    };

    for (int tile = t_begin; tile < t_end; ++tile) {
        setup(tile + 1, nxt);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = init[mt];
        // chunks whose requests stay inside this tile
        for (int ks0 = 0; ks0 + D < a.ksteps; ks0 += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) step(ks0 + d, d, cur);
        }
        // last chunk: its requests are the first D steps of the next tile
        tap_reset(walk);
#pragma unroll
        for (int d = 0; d < D; ++d) step(a.ksteps - D + d, d, nxt);
        load_residual(nxt, ev_nxt);

#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            if (cur.ob[nt] >= 0) {
                PixelPos pp = PixelPos{0, 0, 0};
                if constexpr (EPI == EPI_KIND_GENERIC) pp = cur.pos[nt];
                finish_pixel<NT, EPI>(a, acc, nt, f0, valid, cur.ob[nt], cur.eb[nt], sc, ev_cur[nt], pp.b, pp.oy, pp.ox);
            }
        }
        cur = nxt;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) ev_cur[nt] = ev_nxt[nt];
    }
}

// =====================================================================================================
// Streaming kernel (short K, bandwidth-bound layers): no LDS, no barriers, no tables.
// A wave owns ONE span of 64 output features of ONE pixel tile (16*NT pixels).  Its MFMA fragments come
// straight from global memory (a fragment of lane l IS a contiguous 16-byte piece of fs_b_yx_fsv16
// memory).  Everything the tile needs - activations of all K-steps, weights, residual, requantisation
// factors - is requested before anything is waited for, so a wave pays one memory round trip; it uses
// few registers, so many waves per SIMD overlap their round trips and keep HBM busy.  The four waves
// of a workgroup take the same pixels and neighbouring spans: the activations reach three of them
// through L1.  KS = number of K-steps, fixed at compile time (the host pads the weight stream with
// zero K-chunks).  Needs constant tap offsets (input with a sufficient zero border, or no padding).
// =====================================================================================================
template <int NT, int KS, int EPI>
__global__ void __launch_bounds__(256) conv_stream_kernel(MfmaArgs a)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kq = lane >> 4;
    const int l16 = lane & 15;
    fetch_arguments(a);
    const uint32_t gw = blockIdx.x * 4u + (uint32_t)wave;
    const int nspans = a.ofm_tiles;
    const uint32_t pt = a.div_ofm_tiles.div(gw);
    const int span = (int)(gw - pt * (uint32_t)nspans);
    if (pt >= (uint32_t)a.mtiles) return;  // no barriers below: a wave may leave on its own

    const int f0 = span * 64 + kq * 16;
    const int fs = f0 >> 4;
    const bool live = f0 < a.OFM;
    const int valid = a.OFM - f0;

    // tap offsets of this lane's K-chunks, computed instead of looked up (a table load would put a second
    // memory round trip in front of the activation loads)
    int koff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const uint32_t kc = ks * 4 + kq;
        const uint32_t tap = a.div_cb.div(kc);
        const uint32_t cb = kc - tap * a.CB;
        const uint32_t fy = a.div_fx.div(tap);
        const uint32_t fx = tap - fy * a.FX;
        koff[ks] = kc < (uint32_t)a.kchunks ? (int)(cb * a.in_pf + fy * a.tap_dy + fx * a.tap_dx) : 0;
    }

    // ---- requests
    v4i fb[KS][NT], ev[NT], fa[KS][4], init[4];
    int ob[NT], eb[NT];
    PixelPos pos[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const uint32_t m = pt * (16u * NT) + nt * 16 + l16;
        const uint32_t mm = m < a.M ? m : a.M - 1;
        int pix, o, e;
        if (a.linear) {  // dense tensors, 1x1 / stride 1: pixel m sits at m * 16, no division needed
            pix = a.in_off + (int)mm * 16;
            o = a.out_off + fs * a.out_pf + (int)mm * 16;
            e = a.el_off + fs * a.el_pf + (int)mm * 16;
            pos[nt] = PixelPos{0, 0, 0};
        } else {
            const PixelPos pp = pixel_pos(a, mm);
            pos[nt] = pp;
            pix = a.in_off + (int)pp.b * a.in_pb + ((int)pp.oy * a.sy - a.py) * a.in_py + ((int)pp.ox * a.sx - a.px) * a.px_bytes;
            o = a.out_off + (int)pp.b * a.out_pb + fs * a.out_pf + (int)pp.oy * a.out_py + (int)pp.ox * 16;
            e = a.el_off + (int)pp.b * a.el_pb + fs * a.el_pf + (int)(pp.oy * a.esy) * a.el_py + (int)(pp.ox * a.esx) * 16;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) fb[ks][nt] = *reinterpret_cast<const v4i*>(a.in + (pix + koff[ks]));
        ob[nt] = m < a.M ? o : -1;
        eb[nt] = e;
        ev[nt] = v4i{0, 0, 0, 0};
        if constexpr (EPI == EPI_KIND_FUSED) {
            if (live) ev[nt] = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + e);
        } else if constexpr (EPI == EPI_KIND_FAST) {
            if (a.fe.fused && live) ev[nt] = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + e);
        }
    }
    const v4i* wsrc = a.wpk + (size_t)span * KS * 256 + kq * 64 + l16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) fa[ks][mt] = wsrc[ks * 256 + mt * 16];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) init[mt] = *reinterpret_cast<const v4i*>(a.acc_init + f0 + mt * 4);
    LaneScales sc;
    if (live) load_scales<EPI>(a, f0, sc);

    // ---- multiply
    const v4i xm = {(int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask};
    v4i acc[4][NT];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = init[mt];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) fb[ks][nt] = fb[ks][nt] ^ xm;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                acc[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fa[ks][mt], fb[ks][nt], acc[mt][nt], 0, 0, 0);
    }

    // ---- requantise and store
    if (live) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            if (ob[nt] >= 0) {
                PixelPos pp = pos[nt];
                if constexpr (EPI == EPI_KIND_GENERIC)
                    if (a.linear) pp = pixel_pos(a, pt * (16u * NT) + nt * 16 + l16);
                finish_pixel<NT, EPI>(a, acc, nt, f0, valid, ob[nt], eb[nt], sc, ev[nt], pp.b, pp.oy, pp.ox);
            }
        }
    }
}

template <int BM, int BN, int WP, bool CHECKED>
void launch_mfma_instance(hipStream_t s, const MfmaArgs& a, int grid, int lds, int epi)
{
    const dim3 g(grid), b(256);
    switch (epi) {
    case EPI_KIND_RELU: hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WP, CHECKED, EPI_KIND_RELU>), g, b, lds, s, a); break;
    case EPI_KIND_FUSED: hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WP, CHECKED, EPI_KIND_FUSED>), g, b, lds, s, a); break;
    case EPI_KIND_LINEAR: hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WP, CHECKED, EPI_KIND_LINEAR>), g, b, lds, s, a); break;
    case EPI_KIND_FAST: hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WP, CHECKED, EPI_KIND_FAST>), g, b, lds, s, a); break;
    default: hipLaunchKernelGGL((conv_mfma_kernel<BM, BN, WP, CHECKED, EPI_KIND_GENERIC>), g, b, lds, s, a); break;
    }
}

template <int BN, int NT, int KG>
void launch_bdir_instance(hipStream_t s, const MfmaArgs& a, int grid, int lds, int epi)
{
    const dim3 g(grid), b(256 * KG);
    // more than 64 KiB of dynamic LDS has to be allowed per kernel, once (any host thread may be the first to launch)
#define BDIR_LAUNCH(KIND)                                                                                       \
    {                                                                                                           \
        static std::once_flag allowed;                                                                          \
        std::call_once(allowed, [] {                                                                            \
            CHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_bdir_kernel<BN, NT, KG, KIND>),  \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));            \
        });                                                                                                     \
        hipLaunchKernelGGL((conv_bdir_kernel<BN, NT, KG, KIND>), g, b, lds, s, a);                              \
    }
    switch (epi) {
    case EPI_KIND_RELU: BDIR_LAUNCH(EPI_KIND_RELU) break;
    case EPI_KIND_FUSED: BDIR_LAUNCH(EPI_KIND_FUSED) break;
    case EPI_KIND_LINEAR: BDIR_LAUNCH(EPI_KIND_LINEAR) break;
    case EPI_KIND_FAST: BDIR_LAUNCH(EPI_KIND_FAST) break;
    default: BDIR_LAUNCH(EPI_KIND_GENERIC) break;
    }
#undef BDIR_LAUNCH
}

template <int NT, int D>
void launch_wsl_instance(hipStream_t s, const MfmaArgs& a, int grid, int lds, int epi)
{
    const dim3 g(grid), b(256);
    // more than 64 KiB of dynamic LDS has to be allowed per kernel, once (any host thread may be the first to launch)
#define WSL_LAUNCH(KIND)                                                                                       \
    {                                                                                                          \
        static std::once_flag allowed;                                                                         \
        std::call_once(allowed, [] {                                                                           \
            CHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&conv_wsl_kernel<NT, D, KIND>),       \
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));           \
        });                                                                                                    \
        hipLaunchKernelGGL((conv_wsl_kernel<NT, D, KIND>), g, b, lds, s, a);                                   \
    }
    switch (epi) {
    case EPI_KIND_RELU: WSL_LAUNCH(EPI_KIND_RELU) break;
    case EPI_KIND_FUSED: WSL_LAUNCH(EPI_KIND_FUSED) break;
    case EPI_KIND_LINEAR: WSL_LAUNCH(EPI_KIND_LINEAR) break;
    case EPI_KIND_FAST: WSL_LAUNCH(EPI_KIND_FAST) break;
    default: WSL_LAUNCH(EPI_KIND_GENERIC) break;
    }
#undef WSL_LAUNCH
}

template <int NT, int KS>
void launch_stream_instance(hipStream_t s, const MfmaArgs& a, int grid, int epi)
{
    const dim3 g(grid), b(256);
    switch (epi) {
    case EPI_KIND_RELU: hipLaunchKernelGGL((conv_stream_kernel<NT, KS, EPI_KIND_RELU>), g, b, 0, s, a); break;
    case EPI_KIND_FUSED: hipLaunchKernelGGL((conv_stream_kernel<NT, KS, EPI_KIND_FUSED>), g, b, 0, s, a); break;
    case EPI_KIND_LINEAR: hipLaunchKernelGGL((conv_stream_kernel<NT, KS, EPI_KIND_LINEAR>), g, b, 0, s, a); break;
    case EPI_KIND_FAST: hipLaunchKernelGGL((conv_stream_kernel<NT, KS, EPI_KIND_FAST>), g, b, 0, s, a); break;
    default: hipLaunchKernelGGL((conv_stream_kernel<NT, KS, EPI_KIND_GENERIC>), g, b, 0, s, a); break;
    }
}

}  // namespace chip
