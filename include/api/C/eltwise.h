/* eltwise descriptor: see primitives.h (the reference keeps one header per primitive, api/C/eltwise.h). */
#include "primitives.h"
