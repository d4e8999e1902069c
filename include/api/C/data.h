/* data descriptor: see primitives.h (the reference keeps one header per primitive, api/C/data.h). */
#include "primitives.h"
