// Timed build of the 256x256 MFMA kernels for f16 inputs (probes library).
#define ACC950_IN IN_F16
#define ACC950_TIMED_FN launch_mfma_timed_f16
#include "gemm_mfma_timed.h"
