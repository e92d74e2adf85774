// Instantiation list of the MFMA GEMM kernel for one input type.  Each translation
// unit (gemm_mfma_f16.hip, _bf16.hip, _i8.hip) defines ACC950_IN and includes this.
//
// A "variant" is the counterpart of one point of the reference's tuning space
// (outer tile sizes x k split x cache / double-buffer choices,
//  /root/reference/tools/benchmarkers/accera_gemm.py:187-348): block tile BMxBN, K tile
// of KB bytes, waves laid out WAVES_M x WAVES_N, the tile fill either direct-to-LDS
// (STAGES buffers deep) or register-staged, and whether partial edge tiles are handled.
#include "gemm_mfma16w4.h"
#include "variants.h"

namespace acc950 {

#define VA(AKC, BM, BN, WM, WN, BKC, DIRECT, EDGE, KB, STAGES)                                         \
    { BM, BN, WM, WN, AKC, BKC, DIRECT, EDGE, KB, STAGES, false, false, false, false, false,           \
      &launch_mfma<MfmaConfig<ACC950_IN, BM, BN, WM, WN, AKC, BKC, DIRECT, EDGE, KB, STAGES>>, nullptr }
#define VPA(AKC, BM, BN, WM, WN, BKC, KB, STAGES)                                                       \
    { BM, BN, WM, WN, AKC, BKC, true, false, KB, STAGES, true, false, false, false, false,             \
      &launch_mfma<MfmaConfig<ACC950_IN, BM, BN, WM, WN, AKC, BKC, true, false, KB, STAGES, true>>, nullptr }
// (the fp32 unit has the 32x32 instruction shape only: its table keeps the places of the other kernels, so that a variant
// number means the same kernel geometry for every input type, with no launcher behind them)
#ifdef ACC950_NO_MI16
#define V16(AKC, BM, BN, WM, WN, BKC, KB, STAGES) { BM, BN, WM, WN, AKC, BKC, true, false, KB, STAGES, true, true, false, false, false, nullptr, nullptr }
#define V16W4(BKC) { 256, 256, 2, 2, true, BKC, true, false, 64, 4, false, true, true, false, false, nullptr, nullptr }
#define V16W4_192 { 256, 192, 2, 2, true, true, true, false, 64, 4, false, true, true, false, false, nullptr, nullptr }
#define V16W4P(BKC) { 256, 256, 2, 2, true, BKC, true, false, 64, 4, false, true, true, true, false, nullptr, nullptr }
#define V16W4A(BKC) { 256, 256, 2, 2, false, BKC, true, false, 64, 4, false, true, true, false, false, nullptr, nullptr }
#define V16W4PA(BKC) { 256, 256, 2, 2, false, BKC, true, false, 64, 4, false, true, true, true, false, nullptr, nullptr }
#else
// ping-pong on the 16x16 MFMA shapes
#define V16(AKC, BM, BN, WM, WN, BKC, KB, STAGES)                                                       \
    { BM, BN, WM, WN, AKC, BKC, true, false, KB, STAGES, true, true, false, false, false,              \
      &launch_mfma16<Mfma16Config<ACC950_IN, BM, BN, WM, WN, AKC, BKC, KB, STAGES, false>>,           \
      &launch_mfma16<Mfma16Config<ACC950_IN, BM, BN, WM, WN, AKC, BKC, KB, STAGES, true>> }
// four waves, 128x128 wave tiles, hand-laid K loop
#define V16W4(BKC) \
    { 256, 256, 2, 2, true, BKC, true, false, 64, 4, false, true, true, false, false, &launch_mfma16w4<Mfma16W4Config<ACC950_IN, BKC>>, nullptr }
#define V16W4_192 \
    { 256, 192, 2, 2, true, true, true, false, 64, 4, false, true, true, false, false, &launch_mfma16w4<Mfma16W4Config<ACC950_IN, true, false, 192>>, nullptr }
// the same, one workgroup per CU walking several output tiles
#define V16W4P(BKC) \
    { 256, 256, 2, 2, true, BKC, true, false, 64, 4, false, true, true, true, false, &launch_mfma16w4<Mfma16W4Config<ACC950_IN, BKC, false, 256, true>>, nullptr }
// the same kernel for a column-major A (one tile per workgroup)
#define V16W4A(BKC) \
    { 256, 256, 2, 2, false, BKC, true, false, 64, 4, false, true, true, false, false, &launch_mfma16w4<Mfma16W4Config<ACC950_IN, BKC, false, 256, false, false>>, nullptr }
// ... walking several output tiles
#define V16W4PA(BKC) \
    { 256, 256, 2, 2, false, BKC, true, false, 64, 4, false, true, true, true, false, &launch_mfma16w4<Mfma16W4Config<ACC950_IN, BKC, false, 256, true, false>>, nullptr }
#endif
// any sizes, leading dimensions and alignments (the odd shapes of the reference's sweep lists, e.g.
// /root/reference/tools/benchmarkers/gemm_resnet_inception.csv): register-staged 128x128 tiles whose fill takes unaligned chunks
#define VANY(AKC, BKC)                                                                                  \
    { 128, 128, 2, 2, AKC, BKC, false, true, 128, 2, false, false, false, false, true,                 \
      &launch_mfma<MfmaConfig<ACC950_IN, 128, 128, 2, 2, AKC, BKC, false, true, 128, 2, false, false, true>>, nullptr }
#define VANY64(AKC, BKC)                                                                                \
    { 64, 64, 2, 2, AKC, BKC, false, true, 128, 2, false, false, false, false, true,                   \
      &launch_mfma<MfmaConfig<ACC950_IN, 64, 64, 2, 2, AKC, BKC, false, true, 128, 2, false, false, true>>, nullptr }
// the same on 256x256 tiles, eight waves: large problems of odd sizes (half the fill work per MFMA of the 128x128 form)
#define VANY256(AKC, BKC)                                                                               \
    { 256, 256, 2, 4, AKC, BKC, false, true, 128, 2, false, false, false, false, true,                 \
      &launch_mfma<MfmaConfig<ACC950_IN, 256, 256, 2, 4, AKC, BKC, false, true, 128, 2, false, false, true>>, nullptr }
#define V(BM, BN, WM, WN, BKC, DIRECT, EDGE, KB, STAGES) VA(true, BM, BN, WM, WN, BKC, DIRECT, EDGE, KB, STAGES)
#define VP(BM, BN, WM, WN, BKC, KB, STAGES) VPA(true, BM, BN, WM, WN, BKC, KB, STAGES)
// column-major A (M contiguous; the "transA" shapes of the reference's sweep lists,
// /root/reference/tools/benchmarkers/gemm_*.csv): staged as it lies in memory and read with the
// transposing LDS loads, like a row-major B
#define LAYOUT_AT(BKC)                                    \
    VPA(false, 256, 256, 2, 4, BKC, 64, 4),               \
    VA(false, 128, 128, 2, 2, BKC, true, false, 128, 2),  \
    VA(false, 128, 128, 2, 2, BKC, false, true, 128, 2)

#define LAYOUT(BKC)                                 \
    V(256, 256, 2, 4, BKC, true, false, 128, 2),    \
    V(256, 256, 2, 4, BKC, true, false, 64, 4),     \
    V(256, 256, 2, 4, BKC, true, false, 64, 3),     \
    V(256, 128, 2, 2, BKC, true, false, 128, 3),    \
    V(256, 128, 2, 2, BKC, true, false, 64, 3),     \
    V(128, 256, 2, 2, BKC, true, false, 64, 3),     \
    V(128, 128, 2, 2, BKC, true, false, 128, 2),    \
    V(128, 128, 2, 2, BKC, true, false, 64, 4),     \
    V(128, 128, 2, 2, BKC, false, false, 128, 2),   \
    V(128, 128, 2, 2, BKC, false, true, 128, 2),    \
    VP(256, 256, 2, 4, BKC, 64, 4),                 \
    VP(256, 256, 2, 4, BKC, 128, 2),                \
    VP(256, 256, 2, 4, BKC, 64, 3)

static const MfmaVariant kVariants[] = {
    LAYOUT(false), // B row-major (N contiguous): transpose reads
    LAYOUT(true),  // B column-major (K contiguous)
    // 192-wide tiles (N = 3072 = 16 x 192 gives one tile per CU); K-contiguous B only
    VP(256, 192, 4, 2, true, 64, 4),
    V(256, 192, 4, 2, true, true, false, 128, 2),
    LAYOUT_AT(false),
    LAYOUT_AT(true),
    // 16x16 MFMA shapes: A row-major x B row- / column-major, A column-major, 192-wide tiles
    V16(true, 256, 256, 2, 4, false, 64, 4),
    V16(true, 256, 256, 2, 4, false, 128, 2),
    V16(true, 256, 256, 2, 4, true, 64, 4),
    V16(true, 256, 256, 2, 4, true, 128, 2),
    V16(false, 256, 256, 2, 4, false, 64, 4),
    V16(false, 256, 256, 2, 4, true, 64, 4),
    V16(true, 256, 192, 4, 2, true, 64, 4),
    V16W4(false),
    V16W4(true),
    V16W4_192,
    V16W4P(false),
    V16W4P(true),
    V16W4A(false),
    V16W4A(true),
    VANY(true, false),
    VANY(true, true),
    VANY(false, false),
    VANY(false, true),
    // 128x128 tiles with four stages of 128 bytes of K: 96 KB on their way to a CU at a time (medium-sized problems of one
    // tile per CU are bound by the latency of their fills, not by the matrix cores)
    V(128, 128, 2, 2, false, true, false, 128, 4),
    V(128, 128, 2, 2, true, true, false, 128, 4),
    VA(false, 128, 128, 2, 2, false, true, false, 128, 4),
    VA(false, 128, 128, 2, 2, true, true, false, 128, 4),
    // small tiles for problems whose 128x128 tiles would leave most of the chip idle and whose K is too short to split:
    // 64x64 (a wave has one 32x32 block) and 128x64, deep prefetch, two or more workgroups per CU
    V(64, 64, 2, 2, false, true, false, 128, 4),
    V(64, 64, 2, 2, true, true, false, 128, 4),
    VA(false, 64, 64, 2, 2, false, true, false, 128, 4),
    VA(false, 64, 64, 2, 2, true, true, false, 128, 4),
    V(128, 64, 2, 2, false, true, false, 128, 3),
    V(128, 64, 2, 2, true, true, false, 128, 3),
    VA(false, 128, 64, 2, 2, false, true, false, 128, 3),
    VA(false, 128, 64, 2, 2, true, true, false, 128, 3),
    // and the any-alignment form on 64x64 tiles (the odd shapes of the reference's lists are mostly small)
    VANY64(true, false),
    VANY64(true, true),
    VANY64(false, false),
    VANY64(false, true),
    // four-wave kernel for a column-major A, one workgroup per CU walking several output tiles
    V16W4PA(false),
    V16W4PA(true),
    // any sizes, leading dimensions and alignments on 256x256 tiles
    VANY256(true, false),
    VANY256(true, true),
};
#undef LAYOUT_AT
#undef VA
#undef VPA
#undef V16
#undef V16W4
#undef V16W4_192
#undef V16W4P
#undef V16W4A
#undef V16W4PA
#undef VANY
#undef VANY64
#undef VANY256
#undef LAYOUT
#undef V
#undef VP

const MfmaVariant* ACC950_TABLE_FN(int* count)
{
    *count = (int)(sizeof(kVariants) / sizeof(kVariants[0]));
    return kVariants;
}

} // namespace acc950
