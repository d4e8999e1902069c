/* convolution descriptor: see primitives.h (the reference keeps one header per primitive, api/C/convolution.h). */
#include "primitives.h"
