// MFMA GEMM kernels for i8 inputs (see gemm_mfma.h).
#define ACC950_IN IN_I8
#define ACC950_TABLE_FN mfma_variants_i8
#include "gemm_mfma_inst.h"
