// Instances of the streaming (LDS-free) int8 MFMA convolution kernel:
// 16, 32 or 64 pixels per tile x 1, 2, 4 or 8 K-steps.
#include "conv_mfma_kernel.h"

namespace chip {

template <int NT>
static void by_ksteps(hipStream_t s, const MfmaArgs& a, int ks, int grid, int epi)
{
    switch (ks) {
    case 1: launch_stream_instance<NT, 1>(s, a, grid, epi); break;
    case 2: launch_stream_instance<NT, 2>(s, a, grid, epi); break;
    case 4: launch_stream_instance<NT, 4>(s, a, grid, epi); break;
    case 8: launch_stream_instance<NT, 8>(s, a, grid, epi); break;
    default: throw error(CLDNN_HIP_INVALID_ARG, "streaming kernel: K-steps must be 1, 2, 4 or 8");
    }
}

void launch_stream(hipStream_t s, const MfmaArgs& a, int nt, int grid, int epi)
{
    if (nt == 1) by_ksteps<1>(s, a, a.ksteps, grid, epi);
    else if (nt == 2) by_ksteps<2>(s, a, a.ksteps, grid, epi);
    else if (nt == 4) by_ksteps<4>(s, a, a.ksteps, grid, epi);
    else throw error(CLDNN_HIP_INVALID_ARG, "streaming kernel: pixels per tile must be 16, 32 or 64");
}

}  // namespace chip
