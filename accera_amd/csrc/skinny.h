// Host-visible interface of the skinny (M <= 8) streaming GEMM kernels.
#pragma once
#include "common.h"
#include <stddef.h>

namespace acc950 {

struct SkinnyArgs {
    const void* A;  // M x K, row-major (K contiguous), 16-bit elements
    const void* B;  // K x N, row-major (N contiguous)
    void* C;        // M x N, row-major
    int M, N, K;
    int64_t a_rs, b_rs, c_rs; // row strides in elements
    int in_type, out_type;
    int prologue, epilogue;
    int splits;         // K split over grid.y
    float* scratch;     // splits > 1: [split][column block][64*LPR] partial sums
    unsigned* counters; // splits > 1: one arrival counter per column block, zero between launches
};

int skinny_num_variants();
void skinny_variant_info(int v, int* lanes_per_row, int* waves, int* depth);
int skinny_column_blocks(int v, int N);
size_t skinny_scratch_floats(int v, int N, int splits);
hipError_t launch_skinny(int v, const SkinnyArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run);

} // namespace acc950
