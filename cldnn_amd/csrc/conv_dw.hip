// Depthwise quantized convolution (groups == input features == output features) on
// fs_b_yx_fsv16.  Not a contraction over features, so no matrix cores: the kernel is a
// stencil bound by HBM bandwidth.  One lane owns the 16 features of one output pixel:
// every tap is one coalesced 128-bit load (a wave covers 64 consecutive pixels = 1 KiB),
// the per-slice weights [tap][16] sit in LDS, and the int8 result leaves as one 128-bit store.
//
// Two kernels: conv_dw3x3_kernel for the case every MobileNet layer is (3x3 filter, input with a zero border,
// int8 output through the short requantisation epilogue), and conv_dw_kernel for everything else.
#include "conv_mfma_kernel.h"

#include <cstring>

namespace chip {

struct DwArgs {
    const int8_t* in;
    const int8_t* wpk;        // [fs][tap][16]
    const int32_t* wmask;     // [fs][tap][16] dwords: weight of feature c alone in byte c % 4 (3x3 kernel)
    const int32_t* acc_init;  // [fs*16]
    void* out;
    const void* eltw;
    int32_t* raw;
    Pitch in_p, out_p, eltw_p;
    int B, IH, IW, OH, OW, C, OHW;
    int FY, FX, sy, sx, dy, dx, py, px, esy, esx;
    int64_t M;
    int in_u8;
    uint32_t xor_mask;
    FastDiv div_ohw, div_ow;
    FastEpi fe;
    Epilogue epi;
};

template <bool IN_U8>
__device__ __forceinline__ void mac16(int* acc, const v4i& x, const v4i& w)
{
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const unsigned xv = (unsigned)x[d], wv = (unsigned)w[d];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int xi = IN_U8 ? (int)((xv >> (8 * i)) & 255u) : (int)(int8_t)(xv >> (8 * i));
            const int wi = (int)(int8_t)(wv >> (8 * i));
            acc[d * 4 + i] += xi * wi;
        }
    }
}

template <bool IN_U8>
__global__ void __launch_bounds__(256) conv_dw_kernel(DwArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    v4i* wl = reinterpret_cast<v4i*>(smem);  // [taps]
    const int fs = blockIdx.y;
    const int taps = a.FY * a.FX;
    for (int i = threadIdx.x; i < taps; i += blockDim.x)
        wl[i] = reinterpret_cast<const v4i*>(a.wpk)[(int64_t)fs * taps + i];
    __syncthreads();

    const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= a.M) return;
    const int b = (int)(m / a.OHW);
    const int r = (int)(m % a.OHW);
    const int oy = r / a.OW, ox = r % a.OW;
    const int iy0 = oy * a.sy - a.py, ix0 = ox * a.sx - a.px;
    const int64_t ibase = a.in_p.off + (int64_t)b * a.in_p.pb + (int64_t)fs * a.in_p.pf;

    int acc[16];
    {
        const v4i* ai = reinterpret_cast<const v4i*>(a.acc_init + fs * 16);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const v4i v = ai[d];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[d * 4 + i] = v[i];
        }
    }
    for (int j = 0; j < a.FY; ++j) {
        const int iy = iy0 + j * a.dy;
        if (iy < 0 || iy >= a.IH) continue;
        for (int i = 0; i < a.FX; ++i) {
            const int ix = ix0 + i * a.dx;
            if (ix < 0 || ix >= a.IW) continue;
            const v4i x = *reinterpret_cast<const v4i*>(a.in + ibase + (int64_t)iy * a.in_p.py + (int64_t)ix * 16);
            mac16<IN_U8>(acc, x, wl[j * a.FX + i]);
        }
    }

    const Epilogue& e = a.epi;
    const int f0 = fs * 16;
    if (a.raw) {
#pragma unroll
        for (int c = 0; c < 16; ++c)
            if (f0 + c < a.C) a.raw[(((int64_t)b * a.C + f0 + c) * a.OH + oy) * a.OW + ox] = acc[c];
        return;
    }
    const int64_t obase = a.out_p.off + (int64_t)b * a.out_p.pb + (int64_t)fs * a.out_p.pf + (int64_t)oy * a.out_p.py
                          + (int64_t)ox * a.out_p.px;
    int64_t ebase = 0;
    if (e.fused)
        ebase = a.eltw_p.off + (int64_t)b * a.eltw_p.pb + (int64_t)fs * a.eltw_p.pf
                + (int64_t)(oy * a.esy) * a.eltw_p.py + (int64_t)(ox * a.esx) * a.eltw_p.px;
    const bool out8 = e.out_dt == CLDNN_HIP_S8 || e.out_dt == CLDNN_HIP_U8;
    v4i packed = {0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const int f = f0 + c;
        EpiOut o;
        o.f = 0.f, o.i = 0;
        if (f < a.C) {
            float ev = 0.f;
            if (e.fused) ev = load_as_float(a.eltw, e.eltw_dt, ebase + c);
            o = epilogue_generic(e, acc[c], f, ev);
        }
        if (out8) packed[c >> 2] |= (int)(((unsigned)o.i & 255u) << (8 * (c & 3)));
        else store_out(a.out, e.out_dt, obase + c, o);
    }
    if (out8) *reinterpret_cast<v4i*>((int8_t*)a.out + obase) = packed;
}

// 3x3 depthwise, constant tap offsets (zero border), short epilogue.  A lane owns the 16 features of one output
// pixel.  The multiply uses the packed dot-product instruction with one weight byte unmasked per call:
// sdot4(x_dword, {0,..,w_c,..,0}, acc_c) adds x_c * w_c to the accumulator of feature c without unpacking a single
// byte; the masked weights of a feature slice are the same for every lane and come through the scalar data path.
// u8 activations are fed as x ^ 0x80 = x - 128, the accumulators start from 128 * sum(w) (+ bias).
template <int EPI>
__global__ void __launch_bounds__(256) conv_dw3x3_kernel(DwArgs a)
{
    const int fs = blockIdx.y;
    const uint32_t m = blockIdx.x * 256u + threadIdx.x;
    const bool ok = m < (uint32_t)a.M;
    const uint32_t mm = ok ? m : 0;
    const uint32_t b = a.div_ohw.div(mm);
    const uint32_t r = mm - b * (uint32_t)a.OHW;
    const uint32_t oy = a.div_ow.div(r);
    const uint32_t ox = r - oy * (uint32_t)a.OW;
    const int32_t in_py = (int32_t)a.in_p.py;
    const int8_t* src = a.in + (a.in_p.off + (int64_t)fs * a.in_p.pf)
                        + ((int32_t)b * (int32_t)a.in_p.pb + ((int32_t)oy * a.sy - a.py) * in_py + ((int32_t)ox * a.sx - a.px) * 16);
    v4i x[9];
#pragma unroll
    for (int j = 0; j < 3; ++j)
#pragma unroll
        for (int i = 0; i < 3; ++i) x[j * 3 + i] = *reinterpret_cast<const v4i*>(src + (j * a.dy * in_py + i * a.dx * 16));

    v4i ev4 = {0, 0, 0, 0};
    const int f0 = fs * 16;
    const int obase = (int)(a.out_p.off + (int64_t)fs * a.out_p.pf) + (int)b * (int)a.out_p.pb + (int)oy * (int)a.out_p.py + (int)ox * 16;
    const int ebase = (int)(a.eltw_p.off + (int64_t)fs * a.eltw_p.pf) + (int)b * (int)a.eltw_p.pb
                      + (int)(oy * a.esy) * (int)a.eltw_p.py + (int)(ox * a.esx) * 16;
    if (a.fe.fused) ev4 = *reinterpret_cast<const v4i*>((const int8_t*)a.eltw + ebase);
    LaneScales sc;
    load_scales<EPI>(a, f0, sc);

    v4i acc[4][1];
#pragma unroll
    for (int d = 0; d < 4; ++d) acc[d][0] = *reinterpret_cast<const v4i*>(a.acc_init + f0 + d * 4);
    const const_i32_ptr wm = (const_i32_ptr)(uintptr_t)(a.wmask + (size_t)fs * 9 * 16);
#pragma unroll
    for (int t = 0; t < 9; ++t) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            const int xd = x[t][d] ^ (int)a.xor_mask;
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[d][0][i] = __builtin_amdgcn_sdot4(xd, wm[t * 16 + d * 4 + i], acc[d][0][i], false);
        }
    }
    if (!ok) return;
    const int valid = a.C - f0;
    const v4i packed = epilogue_fast16<1, EPI>(a, acc, 0, sc.wq, sc.cal, sc.ecal, ev4, valid);
    *reinterpret_cast<v4i*>((int8_t*)a.out + obase) = packed;
}

DwPlan dw_plan(const ConvProblem& p)
{
    DwPlan pl{};
    pl.block = 256;
    const int64_t m = (int64_t)p.B * p.OH * p.OW;
    const int64_t gx = (m + pl.block - 1) / pl.block;
    CHIP_REQUIRE(gx < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "convolution too large for one launch");
    pl.grid = (int)gx;
    pl.packed_bytes = (size_t)((p.OFM + 15) / 16) * p.FY * p.FX * 16;
    pl.mask_bytes = pl.packed_bytes * 4;
    return pl;
}

// weights [C][1][FY][FX] -> [fs][tap][16]
void dw_pack_weights(const ConvProblem& p, const int8_t* w, int8_t* packed)
{
    const int taps = p.FY * p.FX;
    std::memset(packed, 0, (size_t)((p.OFM + 15) / 16) * taps * 16);
    for (int c = 0; c < p.OFM; ++c)
        for (int t = 0; t < taps; ++t) packed[((size_t)(c / 16) * taps + t) * 16 + (c % 16)] = w[(size_t)c * taps + t];
}

// masked weights for the 3x3 kernel: dword (fs, tap, c) holds weight c of the slice in byte c % 4, zeros elsewhere
void dw_mask_weights(const ConvProblem& p, const int8_t* w, int32_t* masked)
{
    const int taps = p.FY * p.FX;
    std::memset(masked, 0, (size_t)((p.OFM + 15) / 16) * taps * 16 * 4);
    for (int c = 0; c < p.OFM; ++c)
        for (int t = 0; t < taps; ++t)
            masked[((size_t)(c / 16) * taps + t) * 16 + (c % 16)] =
                (int32_t)((uint32_t)(uint8_t)w[(size_t)c * taps + t] << (8 * (c % 4)));
}

// the 3x3 kernel applies when: 3x3 filter, zero border covering the padding, short epilogue, 32-bit offsets
bool dw_fast_applies(const ConvProblem& p, bool fast_epilogue)
{
    return fast_epilogue && p.FY == 3 && p.FX == 3 && conv_border_covers(p) && tensor_elems(p.in_t) < (1ull << 31)
           && tensor_elems(p.out_t) < (1ull << 31) && (int64_t)p.B * p.OH * p.OW < (1ll << 31);
}

void launch_conv_dw(hipStream_t s, const ConvProblem& p, const DwPlan& pl, const int8_t* packed, const int32_t* masked,
                    const int32_t* acc_init, const Epilogue& epi, const FastEpi* fast, const void* in, const void* eltw,
                    void* out, int32_t* raw)
{
    DwArgs a{};
    a.wmask = masked;
    a.in = (const int8_t*)in, a.wpk = packed, a.acc_init = acc_init, a.out = out, a.eltw = eltw, a.raw = raw;
    a.in_p = p.in_p, a.out_p = p.out_p, a.eltw_p = p.eltw_p;
    a.B = p.B, a.IH = p.IH, a.IW = p.IW, a.OH = p.OH, a.OW = p.OW, a.C = p.OFM, a.OHW = p.OH * p.OW;
    a.FY = p.FY, a.FX = p.FX, a.sy = p.sy, a.sx = p.sx, a.dy = p.dy, a.dx = p.dx, a.py = p.py, a.px = p.px;
    a.esy = p.esy, a.esx = p.esx;
    a.M = (int64_t)p.B * p.OH * p.OW;
    a.epi = epi;
    const dim3 grid(pl.grid, (p.OFM + 15) / 16);
    if (fast && masked && !raw) {
        a.fe = *fast;
        a.xor_mask = p.in_dt == CLDNN_HIP_U8 ? 0x80808080u : 0u;
        a.div_ohw = make_fast_div((uint32_t)a.OHW), a.div_ow = make_fast_div((uint32_t)a.OW);
        const bool plain = !fast->has_wqf && epi.calib && !fast->fused;
        if (plain && fast->relu_folded) hipLaunchKernelGGL(conv_dw3x3_kernel<EPI_KIND_RELU>, grid, dim3(256), 0, s, a);
        else if (plain && fast->act == CLDNN_HIP_ACT_NONE) hipLaunchKernelGGL(conv_dw3x3_kernel<EPI_KIND_LINEAR>, grid, dim3(256), 0, s, a);
        else hipLaunchKernelGGL(conv_dw3x3_kernel<EPI_KIND_FAST>, grid, dim3(256), 0, s, a);
        CHIP_CHECK(hipGetLastError());
        return;
    }
    const int lds = p.FY * p.FX * 16;
    if (p.in_dt == CLDNN_HIP_U8) hipLaunchKernelGGL(conv_dw_kernel<true>, grid, dim3(pl.block), lds, s, a);
    else hipLaunchKernelGGL(conv_dw_kernel<false>, grid, dim3(pl.block), lds, s, a);
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
