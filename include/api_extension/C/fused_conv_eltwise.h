/* fused_conv_eltwise descriptor: see api/C/primitives.h (reference api_extension/C/fused_conv_eltwise.h). */
#include "../../api/C/primitives.h"
