// Timed build of the 256x256 MFMA kernels for i8 inputs (probes library).
#define ACC950_IN IN_I8
#define ACC950_TIMED_FN launch_mfma_timed_i8
#include "gemm_mfma_timed.h"
