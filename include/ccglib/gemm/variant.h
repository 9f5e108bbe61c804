// Part of the ccglib-compatible header tree: the definitions live in common/types.h.
#ifndef CCGLIB_GEMM_VARIANT_H_
#define CCGLIB_GEMM_VARIANT_H_
#include <ccglib/common/types.h>
#endif
