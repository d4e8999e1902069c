/* fully_connected primitive of the clDNN C API (declared in primitives.h; this header keeps the reference's file name) */
#ifndef FULLY_CONNECTED_H
#define FULLY_CONNECTED_H
#include "primitives.h"
#endif /* FULLY_CONNECTED_H */
