// Instances of the direct-activation tile kernel with 2 groups of four waves that split the K-steps of a
// 64-feature tile between them (16 or 32 pixels per wave).
#include "conv_mfma_kernel.h"

namespace chip {

void launch_bdir_k2(hipStream_t s, const MfmaArgs& a, int nt, int grid, int lds, int epi)
{
    switch (nt) {
    case 1: launch_bdir_instance<64, 1, 2>(s, a, grid, lds, epi); break;
    case 2: launch_bdir_instance<64, 2, 2>(s, a, grid, lds, epi); break;
    default: throw error(CLDNN_HIP_INVALID_ARG, "split-K direct-activation kernel: pixels per wave must be 16 or 32");
    }
}

}  // namespace chip
