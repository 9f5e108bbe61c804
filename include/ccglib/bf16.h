// bf16: bfloat16 storage type (reference: include/ccglib/bf16.h). One type on
// host and device here.
#ifndef CCGLIB_BF16_H_
#define CCGLIB_BF16_H_
#include <hip/hip_bf16.h>
using bf16 = __hip_bfloat16;
#endif
