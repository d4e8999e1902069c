// Forwards to api/CPP/cldnn.hpp, which declares cldnn::fused_conv_eltwise.
#pragma once
#include "../../api/CPP/cldnn.hpp"
