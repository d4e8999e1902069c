// Few output pixels, long K: fully_connected at small batch, convolutions whose output plane is a handful of pixels.
// The weights are the traffic (a layer of VGG-16's classifier streams 103 MB for 16 x 4096 outputs) and one
// 16-pixel fragment holds every output pixel, so the tile kernels, which give one workgroup 64 features, leave most
// of the chip idle.  Here a workgroup owns 16 features x 16 pixels -- one matrix-instruction fragment -- and its
// waves (4, 8 or 16) split the K range between them: every wave streams its weight fragments and its activation
// fragments straight from global memory into the registers the MFMA reads, eight K-steps ahead of their use, no
// LDS and no barrier in the loop.  The partial sums meet in LDS at the end; wave 0 adds them (integer addition:
// any order gives the same bits) and runs the element-wise epilogue.  Weights and tap table are the tile kernels'
// packed stream for 64-feature tiles: workgroup (tile, q) takes fragment q of every K-step of its tile.
// When the filter is wider than one tap (a fully_connected over a 7x7 plane) a lane's 16 activation bytes of a
// K-step lie in 64 different cache lines, and every workgroup would pull all of them through its L1 again; a small
// kernel first gathers the activations into fragment order (1 KB per K-step and pixel fragment, sign flip applied),
// which the main kernel then reads as it reads the weights.
#include <mutex>

#include "conv_mfma_kernel.h"

namespace chip {

enum { GEMV_D = 8 };  // look-ahead in K-steps; the packed stream and the tap table carry more slack than that

// activations in fragment order: bpk[(ptile * (ksteps + GEMV_SLACK) + ks) * 64 + lane]
enum { GEMV_SLACK = 32 };
// size of the gather scratch that lives in the code object (for callers that may not allocate)
enum { GEMV_STATIC_SCRATCH_BYTES = 4 << 20 };
__global__ void __launch_bounds__(256) gemv_gather_kernel(MfmaArgs a)
{
    const int lane = threadIdx.x & 63;
    const int ks = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int ptile = blockIdx.y;
    if (ks >= a.ksteps) return;
    const int kq = lane >> 4;
    const int l16 = lane & 15;
    const uint32_t m = (uint32_t)ptile * 16 + l16;
    const PixelPos pp = pixel_pos(a, m < a.M ? m : 0);
    const uint32_t boff = (uint32_t)(a.in_off + (int)pp.b * a.in_pb + ((int)pp.oy * a.sy - a.py) * a.in_py
                                     + ((int)pp.ox * a.sx - a.px) * 16 + kq * a.in_pf);
    const v4i xm = {(int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask, (int)a.xor_mask};
    const v4i v = *reinterpret_cast<const v4i*>(a.in + a.ktab[ks * 4] + boff);
    const_cast<v4i*>(a.bpk)[((size_t)ptile * (a.ksteps + GEMV_SLACK) + ks) * 64 + lane] = v ^ xm;
}

template <bool GATHERED>
__global__ void __launch_bounds__(1024) conv_gemv_kernel(MfmaArgs a)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int kq = lane >> 4;
    const int l16 = lane & 15;
    const int q = blockIdx.x & 3;  // fragment of the 64-feature tile: features 16 * kq' + 4 * q + i of the tile
    const int tile = blockIdx.x >> 2;
    const int ntile = tile % a.ofm_tiles;
    const int ptile = tile / a.ofm_tiles;

    const uint32_t m = (uint32_t)ptile * 16 + l16;
    const PixelPos pp = pixel_pos(a, m < a.M ? m : 0);  // pixels past the end read pixel 0
    const uint32_t boff = (uint32_t)(a.in_off + (int)pp.b * a.in_pb + ((int)pp.oy * a.sy - a.py) * a.in_py
                                     + ((int)pp.ox * a.sx - a.px) * 16 + kq * a.in_pf);
    const int per = (a.ksteps + waves - 1) / waves;
    const int s0 = wave * per;
    const int s1 = s0 + per < a.ksteps ? s0 + per : a.ksteps;
    const v4i* wsrc = a.wpk + (size_t)ntile * a.ksteps * 256 + kq * 64 + q * 16 + l16;
    const int xor_mask = GATHERED ? 0 : (int)a.xor_mask;  // gathered activations are flipped already
    const v4i xm = {xor_mask, xor_mask, xor_mask, xor_mask};
    const v4i* bsrc = a.bpk + (size_t)ptile * (a.ksteps + GEMV_SLACK) * 64 + lane;

    v4i acc = {0, 0, 0, 0};
    v4i ra[GEMV_D], rb[GEMV_D];
    auto load = [&](int ks, v4i& xa, v4i& xb) {
        xa = wsrc[(size_t)ks * 256];
        if constexpr (GATHERED) xb = bsrc[(size_t)ks * 64];
        else xb = *reinterpret_cast<const v4i*>(a.in + scalar_table_load(a.ktab, ks * 4) + boff);
    };
    // The loop is branch-free (a branch around a matrix instruction makes the compiler wait for every outstanding
    // load at the join, and a skipped load would break the counting of outstanding loads the waits rely on).  Steps
    // past the end of the wave's range load the range's last step again (a hit in the L1) and are multiplied with
    // zeroed activations.
    // (the fences pin the order of the loads: the waits in the loop count on step d's loads being issued before step d+1's)
    const int last = s1 > s0 ? s1 - 1 : s0;  // a wave without steps reads one step of the slack or of its neighbour
#pragma unroll
    for (int d = 0; d < GEMV_D; ++d) {
        load(s0 + d < last ? s0 + d : last, ra[d], rb[d]);
        step_fence();
    }
    for (int ks = s0; ks < s1; ks += GEMV_D) {
#pragma unroll
        for (int u = 0; u < GEMV_D; ++u) {
            const int keep = ks + u < s1 ? -1 : 0;
            const v4i km = {keep, keep, keep, keep};
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ra[u], (rb[u] ^ xm) & km, acc, 0, 0, 0);
            load(ks + u + GEMV_D < last ? ks + u + GEMV_D : last, ra[u], rb[u]);
            step_fence();
        }
    }

    __shared__ v4i part[16 * 64];
    part[wave * 64 + lane] = acc;
    __syncthreads();
    if (wave != 0) return;
    for (int w = 1; w < waves; ++w) {
        const v4i o = part[w * 64 + lane];
        acc[0] += o[0], acc[1] += o[1], acc[2] += o[2], acc[3] += o[3];
    }
    if (m >= a.M) return;
    const int f0 = ntile * 64 + kq * 16 + q * 4;  // the lane's four features, consecutive inside one slice of 16
    const Epilogue& e = a.epi;
    const int obase = a.out_off + (int)pp.b * a.out_pb + (f0 >> 4) * a.out_pf + (int)pp.oy * a.out_py + (int)pp.ox * 16 + (f0 & 15);
    const int ebase = a.el_off + (int)pp.b * a.el_pb + (f0 >> 4) * a.el_pf + (int)(pp.oy * a.esy) * a.el_py
                      + (int)(pp.ox * a.esx) * 16 + (f0 & 15);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int f = f0 + i;
        if (f >= a.OFM) break;
        const int v = (int)((unsigned)acc[i] + (unsigned)a.acc_init[f]);
        if (a.raw) {
            a.raw[(((size_t)pp.b * a.OFM + f) * a.OH + pp.oy) * a.OW + pp.ox] = v;
            continue;
        }
        float ev = 0.f;
        if (e.fused) ev = load_as_float(a.eltw, e.eltw_dt, ebase + i);
        store_out(a.out, e.out_dt, obase + i, epilogue_generic(e, v, f, ev));
    }
}

void launch_gemv(hipStream_t s, const MfmaArgs& a, int grid, int waves, int mtiles)
{
    if (a.bpk) {
        hipLaunchKernelGGL(gemv_gather_kernel, dim3((a.ksteps + 3) / 4, mtiles), dim3(256), 0, s, a);
        hipLaunchKernelGGL(conv_gemv_kernel<true>, dim3(grid), dim3(64 * waves), 0, s, a);
    } else {
        hipLaunchKernelGGL(conv_gemv_kernel<false>, dim3(grid), dim3(64 * waves), 0, s, a);
    }
}

size_t gemv_gather_bytes(int mtiles, int ksteps) { return ((size_t)mtiles * (ksteps + GEMV_SLACK)) * 1024; }

// ---- gather scratch that nobody allocates: one array per device, part of the loaded code object.
// Every device the library runs on holds its own copy at its own address until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress; kernels and copies take the address that call returns.
static __device__ __align__(256) unsigned char scratch[GEMV_STATIC_SCRATCH_BYTES];

size_t gemv_static_scratch_bytes() { return GEMV_STATIC_SCRATCH_BYTES; }

// Device address of `scratch` on `device`, which the caller has made current.  Looked up once per device.
void* gemv_static_scratch(int device)
{
    enum { MAX_DEVICES = 64 };
    static std::mutex guard;
    static void* address[MAX_DEVICES] = {};
    CHIP_REQUIRE(device >= 0 && device < MAX_DEVICES, CLDNN_HIP_INVALID_ARG, "device index beyond the static scratch table");
    std::lock_guard<std::mutex> lock(guard);
    if (!address[device]) {
        int current = -1;
        CHIP_CHECK(hipGetDevice(&current));
        CHIP_REQUIRE(current == device, CLDNN_HIP_ERROR, "the static scratch is looked up with its device current");
        void* ptr = nullptr;
        CHIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        CHIP_REQUIRE(ptr, CLDNN_HIP_DEVICE_ERROR, "hipGetSymbolAddress returned no address for the static scratch");
        address[device] = ptr;
    }
    return address[device];
}

}  // namespace chip
