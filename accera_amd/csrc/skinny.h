// Host-visible interface of the skinny (few rows of A) streaming GEMM kernels.
#pragma once
#include "common.h"
#include <stddef.h>

namespace acc950 {

struct SkinnyArgs {
    const void* A;  // M x K, row-major (K contiguous), 16-bit elements (8-bit: MFMA family)
    const void* B;  // K x N, row-major (N contiguous)
    void* C;        // M x N, row-major
    int M, N, K;
    int64_t a_rs, b_rs, c_rs; // row strides in elements
    int in_type, out_type;
    int prologue, epilogue;
    float prologue_arg, epilogue_arg;
    int splits;         // K split over grid.y
    int extra_phase;    // MFMA family, splits == 1: column blocks with index % 4 == extra_phase are split in two
                        // (second halves run as extra workgroups behind the regular grid); -1: none
    int batch;                       // independent problems, one per blockIdx.z
    int64_t a_bs, b_bs, c_bs;        // element distance between consecutive problems
    int64_t scratch_bs, counter_bs;  // same for the K-split workspace (floats, counters)
    float* scratch;     // splits > 1: [split][column block][floats per block] partial sums
    unsigned* counters; // splits > 1: one arrival counter per column block, zero between launches
};

// What a skinny kernel needs before its first load, as arguments of their own in front of the struct: the first 14 dwords
// of a kernel's arguments are preloaded into scalar registers at dispatch (see ACC950_HEAD_PARAMS in common.h).
#define ACC950_SKINNY_HEAD_PARAMS const void* head_A, const void* head_B, int head_M, int head_N, int head_K, int head_splits, \
                                  int head_extra_phase, int head_batch, int64_t head_a_rs, int64_t head_b_rs
#define ACC950_SKINNY_HEAD_OF(a) (a).A, (a).B, (a).M, (a).N, (a).K, (a).splits, (a).extra_phase, (a).batch, (a).a_rs, (a).b_rs
#define ACC950_SKINNY_TAKE_HEAD(p)                                                                               \
    do {                                                                                                          \
        (p).A = head_A; (p).B = head_B; (p).M = head_M; (p).N = head_N; (p).K = head_K; (p).splits = head_splits; \
        (p).extra_phase = head_extra_phase; (p).batch = head_batch; (p).a_rs = head_a_rs; (p).b_rs = head_b_rs;   \
    } while (0)

typedef hipError_t (*SkinnyLaunchFn)(const SkinnyArgs&, hipStream_t, LaunchGeom*, bool);

// One kernel instantiation.  Two families: "dot2" (packed dot products on the vector
// ALU, M <= 8, K even) and "mfma" (B transposed out of LDS into MFMA operands, M <= 32,
// K a multiple of 16 per split).
struct SkinnyVariant {
    int cols;          // columns per workgroup
    int waves, depth;  // waves per workgroup, ring slots (steps in flight) per wave
    bool mfma;
    int max_m;         // rows of A the kernel can take
    int k_step;        // K rows per wave step for 16-bit inputs (int8: twice as many); every K split is a whole number of steps
    int block_floats;  // scratch sums (32 bits each) per column block and split
    SkinnyLaunchFn f16, bf16;
    SkinnyLaunchFn i8; // int8 inputs, int32 sums (MFMA family only; null otherwise)
};

// k rows per wave step of variant v for this input type
inline int skinny_k_step(const SkinnyVariant& v, int in_type) { return in_type == T_I8 ? 2 * v.k_step : v.k_step; }

// tables of the two families (gemm_skinny.hip, gemm_skinny_mfma.hip)
const SkinnyVariant* skinny_dot2_table(int* count);
const SkinnyVariant* skinny_mfma_table(int* count);

// place of the MFMA family's 256-column form (four waves, four ring slots) in the table: skinny_variant(kSkinnyWide)
constexpr int kSkinnyWide = 4;

int skinny_num_variants();
const SkinnyVariant& skinny_variant(int v); // MFMA family first, then dot2
void skinny_variant_info(int v, int* lanes_per_row, int* waves, int* depth);
int skinny_column_blocks(int v, int N);
size_t skinny_scratch_floats(int v, int N, int splits);
hipError_t launch_skinny(int v, const SkinnyArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run);

} // namespace acc950
