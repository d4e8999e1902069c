/* pooling primitive of the clDNN C API (declared in primitives.h; this header keeps the reference's file name) */
#ifndef POOLING_H
#define POOLING_H
#include "primitives.h"
#endif /* POOLING_H */
