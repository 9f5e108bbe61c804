// Part of the ccglib-compatible header tree: the definitions live in common/types.h.
#ifndef CCGLIB_COMMON_COMPLEX_ORDER_H_
#define CCGLIB_COMMON_COMPLEX_ORDER_H_
#include <ccglib/common/types.h>
#endif
