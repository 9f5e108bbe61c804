// half: the 16-bit IEEE type of the HIP headers, as in the reference's fp16.h.
#ifndef CCGLIB_FP16_H_
#define CCGLIB_FP16_H_
#include <hip/hip_fp16.h>
#endif
