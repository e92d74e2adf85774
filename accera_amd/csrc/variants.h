// Table entry describing one compiled MFMA GEMM kernel.
#pragma once
#include "common.h"

namespace acc950 {

struct MfmaVariant {
    int bm, bn;          // block tile
    int waves_m, waves_n;
    bool a_kc, b_kc;     // operand has K contiguous in memory (else M/N contiguous)
    bool direct;         // tile fill with global_load_lds (else through registers)
    bool edge;           // handles M/N/K that are not tile multiples
    int kb;              // bytes of K per tile (64 or 128)
    int stages;          // LDS buffers
    bool pingpong;       // sibling waves alternate memory and compute clusters
    bool mi16;           // 16x16 MFMA shapes (else 32x32)
    bool w4;             // four waves with 128x128 wave tiles and the hand-laid K loop: at least four K tiles, an int8 C only written
    bool persist;        // w4 only: one workgroup per CU walks several output tiles, the next tile's first fills overlap this tile's end
    bool any;            // edge only: operands of any size, leading dimension and alignment (unaligned loads, row ends put together from elements)
    LaunchFn launch;
    LaunchFn launch_general; // build that carries every prologue / epilogue op, when `launch` is a lean build (else null)
};

const MfmaVariant* mfma_variants_f16(int* count);
const MfmaVariant* mfma_variants_bf16(int* count);
const MfmaVariant* mfma_variants_i8(int* count);
const MfmaVariant* mfma_variants_f32(int* count); // (32x32-shape entries only; the others have no launcher)

// second step of a K split of the MFMA kernels (gemm_splitk.hip)
hipError_t launch_splitk_reduce(const GemmArgs& g, const void* ws, int splits, hipStream_t stream);

bool f32_can_take(const GemmArgs& g);
hipError_t launch_f32(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run);
hipError_t launch_generic(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run);

} // namespace acc950
