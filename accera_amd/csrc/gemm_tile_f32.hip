// LDS-tiled MFMA GEMM kernels for fp32 inputs: the 32x32-shape kernels of gemm_mfma.h on v_mfma_f32_32x32x2_f32
// (large fp32 problems; the small ones stay with gemm_f32.hip, whose workgroups take 32x32 blocks straight from global memory).
#define ACC950_IN IN_F32
#define ACC950_TABLE_FN mfma_variants_f32
#define ACC950_NO_MI16
#include "gemm_mfma_inst.h"
