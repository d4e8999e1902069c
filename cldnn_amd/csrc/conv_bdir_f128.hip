// Instances of the direct-activation tile kernel with 128 output features per workgroup:
// 64, 128 or 256 pixels per workgroup (16, 32 or 64 per wave).
#include "conv_mfma_kernel.h"

namespace chip {

void launch_bdir_f128(hipStream_t s, const MfmaArgs& a, int nt, int grid, int lds, int epi)
{
    switch (nt) {
    case 1: launch_bdir_instance<128, 1, 1>(s, a, grid, lds, epi); break;
    case 2: launch_bdir_instance<128, 2, 1>(s, a, grid, lds, epi); break;
    case 4: launch_bdir_instance<128, 4, 1>(s, a, grid, lds, epi); break;
    default: throw error(CLDNN_HIP_INVALID_ARG, "direct-activation kernel: pixels per wave must be 16, 32 or 64");
    }
}

}  // namespace chip
