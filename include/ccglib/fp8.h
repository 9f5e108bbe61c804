// fp8_e4m3 / fp8_e5m2: the OCP 8-bit float types, which are the ones gfx950
// computes with (reference: include/ccglib/fp8.h:35-37).
#ifndef CCGLIB_FP8_H_
#define CCGLIB_FP8_H_
#include <hip/hip_fp8.h>
using fp8_e4m3 = __hip_fp8_e4m3;
using fp8_e5m2 = __hip_fp8_e5m2;
#endif
