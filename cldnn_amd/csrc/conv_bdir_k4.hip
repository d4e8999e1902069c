// Instances of the direct-activation tile kernel with 4 groups of four waves that split the K-steps of a
// 64-feature tile between them (16 pixels per wave; 32 with two groups).
#include "conv_mfma_kernel.h"

namespace chip {

void launch_bdir_k4(hipStream_t s, const MfmaArgs& a, int nt, int grid, int lds, int epi)
{
    switch (nt) {
    case 1: launch_bdir_instance<64, 1, 4>(s, a, grid, lds, epi); break;
    default: throw error(CLDNN_HIP_INVALID_ARG, "split-K direct-activation kernel: this instance takes 16 pixels per wave");
    }
}

}  // namespace chip
