// Thread-bound (non-tensorized) GEMM with fused epilogue: any element type, any
// strides, any M/N/K.  It is the gfx950 counterpart of the reference's plain
// `plan.bind` GPU plan with thread coarsening and a shared-memory cache
// (/root/reference/accera/python/accera/test/mfma_tests.py:250-278,309-356;
//  kernel text /root/reference/docs/Tutorials/GPU/Hello_MatMul_GPU.md:161-192)
// and serves every shape the MFMA kernels do not take (unaligned or tiny problems).
// Inputs are widened before the multiply, the sum is kept in float / int32.
#include "common.h"
#include <type_traits>

namespace acc950 {

namespace {

constexpr int GT = 64;  // output tile edge per workgroup
constexpr int GK = 16;  // K slab
constexpr int GC = 4;   // each of the 16x16 threads owns a 4x4 patch

template <typename AccT>
__device__ __forceinline__ AccT load_in(const void* p, int type, int64_t idx)
{
    switch (type) {
    case T_F32: return (AccT)((const float*)p)[idx];
    case T_F16: return (AccT)f16_bits_to_float(((const uint16_t*)p)[idx]);
    case T_BF16: return (AccT)bf16_bits_to_float(((const uint16_t*)p)[idx]);
    default: return (AccT)((const int8_t*)p)[idx];
    }
}

template <typename AccT>
__global__ void __launch_bounds__(256) gemm_generic_kernel(ACC950_HEAD_PARAMS, GemmArgs p)
{
    __shared__ AccT sA[GK][GT + 1]; // [k][m]
    __shared__ AccT sB[GK][GT + 1]; // [k][n]
    ACC950_TAKE_HEAD(p);
    select_batch(p);
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;

    AccT acc[GC][GC];
#pragma unroll
    for (int i = 0; i < GC; ++i)
#pragma unroll
        for (int j = 0; j < GC; ++j) acc[i][j] = 0;

    for (int k0 = 0; k0 < p.K; k0 += GK) {
        for (int e = threadIdx.x; e < GT * GK; e += 256) {
            int kk = e % GK, r = e / GK;
            int m = m0 + r, n = n0 + r, k = k0 + kk;
            sA[kk][r] = (m < p.M && k < p.K) ? load_in<AccT>(p.A, p.in_type, m * p.a_rs + k * p.a_cs) : AccT(0);
            sB[kk][r] = (n < p.N && k < p.K) ? load_in<AccT>(p.B, p.in_type, k * p.b_rs + n * p.b_cs) : AccT(0);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            AccT a[GC], b[GC];
#pragma unroll
            for (int i = 0; i < GC; ++i) a[i] = sA[kk][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < GC; ++j) b[j] = sB[kk][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < GC; ++i)
#pragma unroll
                for (int j = 0; j < GC; ++j) {
                    if constexpr (std::is_same<AccT, int>::value) // int32: wrap-around sum
                        acc[i][j] = (AccT)((unsigned)acc[i][j] + (unsigned)(a[i] * b[j]));
                    else
                        acc[i][j] += a[i] * b[j];
                }
        }
        __syncthreads();
    }

    // Passes over the thread's elements: old C first (only when the prologue keeps it), then the ops, then the stores.  A
    // load inside the loop over the elements, behind the test of the prologue op, would put every store behind the memory
    // counter of that possible load: one store round trip after the other.
    const bool keeps_c = p.prologue != PRO_SET;
    AccT old[GC][GC];
#pragma unroll
    for (int i = 0; i < GC; ++i)
#pragma unroll
        for (int j = 0; j < GC; ++j) {
            old[i][j] = AccT(0);
            const int m = m0 + ty + 16 * i, n = n0 + tx + 16 * j;
            if (keeps_c && m < p.M && n < p.N) {
                const int64_t idx = m * p.c_rs + n * p.c_cs;
                if constexpr (std::is_same<AccT, int>::value) old[i][j] = load_out_int(p.C, p.out_type, idx);
                else old[i][j] = load_out(p.C, p.out_type, idx);
            }
        }
#pragma unroll
    for (int i = 0; i < GC; ++i)
#pragma unroll
        for (int j = 0; j < GC; ++j) {
            const int m = m0 + ty + 16 * i, n = n0 + tx + 16 * j;
            if (m >= p.M || n >= p.N) continue;
            const int64_t idx = m * p.c_rs + n * p.c_cs;
            const AccT c_old = old[i][j];
            if constexpr (std::is_same<AccT, int>::value) {
                const int v = apply_prologue<int>(acc[i][j], p.prologue, p.prologue_arg, [&]() { return c_old; });
                store_out_int(p.C, p.out_type, idx, apply_epilogue<int>(v, p.epilogue, p.epilogue_arg));
            } else {
                const float v = apply_prologue<float>(acc[i][j], p.prologue, p.prologue_arg, [&]() { return c_old; });
                store_out(p.C, p.out_type, idx, apply_epilogue<float>(v, p.epilogue, p.epilogue_arg));
            }
        }
}

} // namespace

hipError_t launch_generic(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    dim3 grid((a.N + GT - 1) / GT, (a.M + GT - 1) / GT, a.batch > 1 ? a.batch : 1), block(256, 1, 1);
    if (geom) {
        geom->grid[0] = grid.x; geom->grid[1] = grid.y; geom->grid[2] = grid.z;
        geom->block[0] = 256; geom->block[1] = geom->block[2] = 1;
        geom->dyn_lds = 0;
    }
    if (dry_run) return hipSuccess;
    if (a.in_type == T_I8)
        hipLaunchKernelGGL(gemm_generic_kernel<int>, grid, block, 0, stream, ACC950_HEAD_OF(a), a);
    else
        hipLaunchKernelGGL(gemm_generic_kernel<float>, grid, block, 0, stream, ACC950_HEAD_OF(a), a);
    return hipGetLastError();
}

} // namespace acc950
