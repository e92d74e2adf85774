// MFMA GEMM kernels for f16 inputs (see gemm_mfma.h).
#define ACC950_IN IN_F16
#define ACC950_TABLE_FN mfma_variants_f16
#include "gemm_mfma_inst.h"
