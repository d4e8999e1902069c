/* concatenation primitive of the clDNN C API (declared in primitives.h; this header keeps the reference's file name) */
#ifndef CONCATENATION_H
#define CONCATENATION_H
#include "primitives.h"
#endif /* CONCATENATION_H */
