/* input_layout descriptor: see primitives.h (the reference keeps one header per primitive, api/C/input_layout.h). */
#include "primitives.h"
