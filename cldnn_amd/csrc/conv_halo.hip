// Instances of the staged-patch kernel (nine-tap stride-1 convolutions, both operands in LDS): rows of the tile table
// by workgroup shape, each with one or two patch requests per wave and step.
#include "conv_halo_kernel.h"

namespace chip {

template <int WP, int WF>
static void launch_shape(hipStream_t s, const HaloArgs& h, int pl, int grid, int lds, int epi)
{
    if (pl == 1) launch_halo_instance<4, 2, WP, WF, 4, 1>(s, h, grid, lds, epi);
    else launch_halo_instance<4, 2, WP, WF, 4, 2>(s, h, grid, lds, epi);
}

void launch_halo(hipStream_t s, const HaloArgs& h, int row, int pl, int grid, int lds, int epi)
{
    switch (row) {
    case 0: launch_shape<4, 1>(s, h, pl, grid, lds, epi); break;
    case 1: launch_shape<8, 1>(s, h, pl, grid, lds, epi); break;
    default: throw error(CLDNN_HIP_INVALID_ARG, "staged-patch kernel: unknown row");
    }
}

}  // namespace chip
