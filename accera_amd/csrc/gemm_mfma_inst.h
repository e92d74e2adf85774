// Instantiation list of the MFMA GEMM kernel for one input type.  Each translation
// unit (gemm_mfma_f16.hip, _bf16.hip, _i8.hip) defines ACC950_IN and includes this.
//
// A "variant" is the counterpart of one point of the reference's tuning space
// (outer tile sizes x cache/double-buffer choices,
//  /root/reference/tools/benchmarkers/accera_gemm.py:187-348): block tile BMxBN, the
// K tile fixed at 128 bytes, waves laid out WAVES_M x WAVES_N, the tile fill either
// direct-to-LDS or register-staged, and whether partial edge tiles are handled.
#include "gemm_mfma.h"
#include "variants.h"

namespace acc950 {

#define V(BM, BN, WM, WN, BKC, DIRECT, EDGE)                                                           \
    { BM, BN, WM, WN, /*a_kc=*/true, BKC, DIRECT, EDGE,                                                \
      &launch_mfma<ACC950_IN, BM, BN, WM, WN, true, BKC, DIRECT, EDGE> }

static const MfmaVariant kVariants[] = {
    // B row-major (N contiguous): transpose reads
    V(256, 256, 2, 2, false, true, false),
    V(256, 256, 2, 4, false, true, false),
    V(256, 256, 2, 2, false, false, false),
    V(256, 256, 2, 4, false, false, false),
    V(256, 128, 2, 2, false, true, false),
    V(128, 128, 2, 2, false, true, false),
    V(128, 128, 2, 2, false, false, false),
    V(128, 128, 2, 2, false, false, true),
    // B column-major (K contiguous)
    V(256, 256, 2, 2, true, true, false),
    V(256, 256, 2, 4, true, true, false),
    V(256, 256, 2, 2, true, false, false),
    V(256, 256, 2, 4, true, false, false),
    V(256, 128, 2, 2, true, true, false),
    V(128, 128, 2, 2, true, true, false),
    V(128, 128, 2, 2, true, false, false),
    V(128, 128, 2, 2, true, false, true),
};
#undef V

const MfmaVariant* ACC950_TABLE_FN(int* count)
{
    *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
    return kVariants;
}

} // namespace acc950
