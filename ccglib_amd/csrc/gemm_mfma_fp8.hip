// One part of the MFMA GEMM's instantiations (see the end of gemm_mfma.hip).
#define CCGLIB_GEMM_MFMA_PART 4
#include "gemm_mfma.hip"
