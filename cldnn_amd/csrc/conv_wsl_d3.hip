// Instances of the weights-stationary kernel with an activation look-ahead of 3 K-step(s):
// 16, 32 or 64 pixels per wave.
#include "conv_mfma_kernel.h"

namespace chip {

void launch_wsl_d3(hipStream_t s, const MfmaArgs& a, int nt, int grid, int lds, int epi)
{
    switch (nt) {
    case 1: launch_wsl_instance<1, 3>(s, a, grid, lds, epi); break;
    case 2: launch_wsl_instance<2, 3>(s, a, grid, lds, epi); break;
    case 4: launch_wsl_instance<4, 3>(s, a, grid, lds, epi); break;
    default: throw error(CLDNN_HIP_INVALID_ARG, "weights-stationary kernel: pixels per wave must be 16, 32 or 64");
    }
}

}  // namespace chip
