// Umbrella header of the ccglib-compatible C++ API for gfx950.
#ifndef CCGLIB_CCGLIB_HPP_
#define CCGLIB_CCGLIB_HPP_
#include <ccglib/gemm/mma.h>
#include <ccglib/gemm/reference.h>
#include <ccglib/packing/packing.h>
#include <ccglib/pipeline/pipeline.h>
#include <ccglib/transpose/transpose.h>
#endif
