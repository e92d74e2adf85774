// MFMA GEMM kernels for bf16 inputs (see gemm_mfma.h).
#define ACC950_IN IN_BF16
#define ACC950_TABLE_FN mfma_variants_bf16
#include "gemm_mfma_inst.h"
