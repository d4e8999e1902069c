// Depthwise quantized convolution (groups == input features == output features) on
// fs_b_yx_fsv16.  Not a contraction over features, so no matrix cores: the kernel is a
// stencil bound by HBM bandwidth.  One lane owns the 16 features of one output pixel:
// every tap is one coalesced 128-bit load (a wave covers 64 consecutive pixels = 1 KiB),
// the per-slice weights [tap][16] sit in LDS, and the int8 result leaves as one 128-bit store.
#include "epilogue.h"
#include "kernels.h"

#include <cstring>

namespace chip {

typedef int v4i __attribute__((ext_vector_type(4)));

struct DwArgs {
    const int8_t* in;
    const int8_t* wpk;        // [fs][tap][16]
    const int32_t* acc_init;  // [fs*16]
    void* out;
    const void* eltw;
    int32_t* raw;
    Pitch in_p, out_p, eltw_p;
    int B, IH, IW, OH, OW, C, OHW;
    int FY, FX, sy, sx, dy, dx, py, px, esy, esx;
    int64_t M;
    int in_u8;
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

DwPlan dw_plan(const ConvProblem& p)
{
    DwPlan pl{};
    pl.block = 256;
    const int64_t m = (int64_t)p.B * p.OH * p.OW;
    const int64_t gx = (m + pl.block - 1) / pl.block;
    CHIP_REQUIRE(gx < (1ll << 31), CLDNN_HIP_UNSUPPORTED_SIZE, "convolution too large for one launch");
    pl.grid = (int)gx;
    pl.packed_bytes = (size_t)((p.OFM + 15) / 16) * p.FY * p.FX * 16;
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

void launch_conv_dw(hipStream_t s, const ConvProblem& p, const DwPlan& pl, const int8_t* packed, const int32_t* acc_init,
                    const Epilogue& epi, const void* in, const void* eltw, void* out, int32_t* raw)
{
    DwArgs a{};
    a.in = (const int8_t*)in, a.wpk = packed, a.acc_init = acc_init, a.out = out, a.eltw = eltw, a.raw = raw;
    a.in_p = p.in_p, a.out_p = p.out_p, a.eltw_p = p.eltw_p;
    a.B = p.B, a.IH = p.IH, a.IW = p.IW, a.OH = p.OH, a.OW = p.OW, a.C = p.OFM, a.OHW = p.OH * p.OW;
    a.FY = p.FY, a.FX = p.FX, a.sy = p.sy, a.sx = p.sx, a.dy = p.dy, a.dx = p.dx, a.py = p.py, a.px = p.px;
    a.esy = p.esy, a.esx = p.esx;
    a.M = (int64_t)p.B * p.OH * p.OW;
    a.epi = epi;
    const dim3 grid(pl.grid, (p.OFM + 15) / 16);
    const int lds = p.FY * p.FX * 16;
    if (p.in_dt == CLDNN_HIP_U8) hipLaunchKernelGGL(conv_dw_kernel<true>, grid, dim3(pl.block), lds, s, a);
    else hipLaunchKernelGGL(conv_dw_kernel<false>, grid, dim3(pl.block), lds, s, a);
    CHIP_CHECK(hipGetLastError());
}

}  // namespace chip
