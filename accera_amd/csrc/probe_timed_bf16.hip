// Timed build of the 256x256 MFMA kernels for bf16 inputs (probes library).
#define ACC950_IN IN_BF16
#define ACC950_TIMED_FN launch_mfma_timed_bf16
#include "gemm_mfma_timed.h"
