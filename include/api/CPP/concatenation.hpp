// Forwards to cldnn.hpp, which holds the C++ API of the convolution path in one header.
#pragma once
#include "cldnn.hpp"
