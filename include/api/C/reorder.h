/* reorder descriptor: see primitives.h (the reference keeps one header per primitive, api/C/reorder.h). */
#include "primitives.h"
