// Part of the ccglib-compatible header tree: the definitions live in common/types.h.
#ifndef CCGLIB_GEMM_MEM_ORDER_H_
#define CCGLIB_GEMM_MEM_ORDER_H_
#include <ccglib/common/types.h>
#endif
