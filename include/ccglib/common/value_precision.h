// Part of the ccglib-compatible header tree: the definitions live in common/types.h.
#ifndef CCGLIB_COMMON_VALUE_PRECISION_H_
#define CCGLIB_COMMON_VALUE_PRECISION_H_
#include <ccglib/common/types.h>
#endif
