/* activation descriptor: see primitives.h (the reference keeps one header per primitive, api/C/activation.h). */
#include "primitives.h"
