// Second step of a K split of the MFMA kernels: C = epilogue(prologue(C) + slice 0 + slice 1 + ...).
//
// The first step is the GEMM kernel itself, launched as a batch of `splits` partial products over consecutive ranges of
// K (blockIdx.z picks the range) that writes 32-bit sums into a workspace, slice after slice, each an M x N row-major
// matrix.  This kernel adds the slices of every element in slice order -- a fixed order, so the result does not depend
// on which workgroup finished first -- and then does what the GEMM kernel's write-back does for an unsplit problem: the
// prologue op on the old C, the epilogue op (the fused ReLU comes after the whole sum), the narrowing store.
//
// The reference has no counterpart (its `k_split` is the K depth of the block tile); shapes of its sweep lists with a
// small output and a long K (/root/reference/tools/benchmarkers/gemm_bert_assorted.csv: 768 x 320 x 30522,
// gemm_resnet_inception.csv: 288 x 64 x 21609) are the ones that leave most compute units idle without it.
#include "common.h"
#include "variants.h"

namespace acc950 {

struct SplitReduceArgs {
    const void* ws;       // [splits][M][N] float or int
    int splits, M, N;
    void* C;
    int64_t c_rs, c_cs;
    int out_type, is_int;
    int prologue, epilogue;
    float prologue_arg, epilogue_arg;
};

// one thread per four consecutive columns of a row (N is padded up to a multiple of four by the test below)
// (ws, C, splits, M, N, c_rs, c_cs come as arguments of their own as well: the first 14 dwords of a kernel's arguments are
// preloaded into scalar registers at dispatch, and the loads of the slices need nothing else)
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const void* head_ws, void* head_C, int head_splits, int head_M, int head_N,
                                                            int64_t head_c_rs, int64_t head_c_cs, SplitReduceArgs p)
{
    p.ws = head_ws; p.C = head_C; p.splits = head_splits; p.M = head_M; p.N = head_N; p.c_rs = head_c_rs; p.c_cs = head_c_cs;
    const int groups_n = (p.N + 3) / 4;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= (int64_t)p.M * groups_n) return;
    const int row = (int)(id / groups_n), col0 = (int)(id % groups_n) * 4;
    const int64_t slice = (int64_t)p.M * p.N;
    const int64_t at = (int64_t)row * p.N + col0;
    const int cols = p.N - col0 < 4 ? p.N - col0 : 4;
    // The loads of eight slices are issued together (one trip through memory per batch instead of one per slice); the adds
    // stay in slice order.
    // (a slice starts M * N elements after the one before: every slice's piece is 16 bytes aligned only when that is a multiple of four too)
    const bool vec = cols == 4 && (at & 3) == 0 && (slice & 3) == 0;
    auto add_slices = [&](auto zero, auto&& add) {
        using T = decltype(zero);
        typedef T T4 __attribute__((ext_vector_type(4)));
        T4 sum = {zero, zero, zero, zero};
        const T* w = (const T*)p.ws + at;
        for (int s0 = 0; s0 < p.splits; s0 += 8) {
            T4 x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                x[u] = T4{zero, zero, zero, zero};
                if (s0 + u < p.splits) {
                    const T* src = w + (int64_t)(s0 + u) * slice;
                    if (vec) x[u] = *(const T4*)src;
                    else
                        for (int e = 0; e < cols; ++e) x[u][e] = src[e];
                }
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (s0 + u < p.splits)
                    for (int e = 0; e < 4; ++e) sum[e] = add(sum[e], x[u][e]);
        }
        return sum;
    };
    // Four finished outputs that lie side by side, aligned, in a C that is only written leave as one store.
    const int os = p.out_type == T_I8 ? 1 : (p.out_type == T_F32 || p.out_type == T_I32) ? 4 : 2;
    const int64_t idx0 = (int64_t)row * p.c_rs + col0;
    const bool vec_out = cols == 4 && p.c_cs == 1 && p.prologue == PRO_SET && (((size_t)p.C + (size_t)idx0 * os) & (size_t)(4 * os - 1)) == 0;
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    if (p.is_int) {
        const auto sum = add_slices(0, [](int a, int b) { return wrap_add(a, b); });
        if (vec_out) {
            int r[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = apply_epilogue<int>(wrap_add(sum[e], (int)p.prologue_arg), p.epilogue, p.epilogue_arg);
            if (p.out_type == T_I32) *(i32x4*)((int*)p.C + idx0) = i32x4{r[0], r[1], r[2], r[3]};
            else if (p.out_type == T_I16)
                *(u32x2*)((int16_t*)p.C + idx0) = u32x2{((unsigned)r[0] & 0xffffu) | ((unsigned)r[1] << 16), ((unsigned)r[2] & 0xffffu) | ((unsigned)r[3] << 16)};
            else
                *(unsigned*)((int8_t*)p.C + idx0) = ((unsigned)r[0] & 0xffu) | (((unsigned)r[1] & 0xffu) << 8) | (((unsigned)r[2] & 0xffu) << 16) | ((unsigned)r[3] << 24);
            return;
        }
        for (int e = 0; e < cols; ++e) {
            const int64_t idx = (int64_t)row * p.c_rs + (int64_t)(col0 + e) * p.c_cs;
            const int v = apply_prologue<int>(sum[e], p.prologue, p.prologue_arg, [&]() { return load_out_int(p.C, p.out_type, idx); });
            store_out_int(p.C, p.out_type, idx, apply_epilogue<int>(v, p.epilogue, p.epilogue_arg));
        }
    } else {
        const auto sum = add_slices(0.f, [](float a, float b) { return a + b; });
        if (vec_out) {
            float r[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = apply_epilogue<float>(sum[e] + p.prologue_arg, p.epilogue, p.epilogue_arg);
            if (p.out_type == T_F32) *(f32x4*)((float*)p.C + idx0) = f32x4{r[0], r[1], r[2], r[3]};
            else if (p.out_type == T_F16)
                *(u32x2*)((uint16_t*)p.C + idx0) = u32x2{(unsigned)float_to_f16_bits(r[0]) | ((unsigned)float_to_f16_bits(r[1]) << 16),
                                                         (unsigned)float_to_f16_bits(r[2]) | ((unsigned)float_to_f16_bits(r[3]) << 16)};
            else
                *(u32x2*)((uint16_t*)p.C + idx0) = u32x2{(unsigned)float_to_bf16_bits(r[0]) | ((unsigned)float_to_bf16_bits(r[1]) << 16),
                                                         (unsigned)float_to_bf16_bits(r[2]) | ((unsigned)float_to_bf16_bits(r[3]) << 16)};
            return;
        }
        for (int e = 0; e < cols; ++e) {
            const int64_t idx = (int64_t)row * p.c_rs + (int64_t)(col0 + e) * p.c_cs;
            const float v = apply_prologue<float>(sum[e], p.prologue, p.prologue_arg, [&]() { return load_out(p.C, p.out_type, idx); });
            store_out(p.C, p.out_type, idx, apply_epilogue<float>(v, p.epilogue, p.epilogue_arg));
        }
    }
}

// g: the caller's problem (its C, strides, output type and ops); ws: the slices the first step wrote
hipError_t launch_splitk_reduce(const GemmArgs& g, const void* ws, int splits, hipStream_t stream)
{
    SplitReduceArgs a{};
    a.ws = ws; a.splits = splits; a.M = g.M; a.N = g.N;
    a.C = g.C; a.c_rs = g.c_rs; a.c_cs = g.c_cs;
    a.out_type = g.out_type; a.is_int = g.in_type == T_I8;
    a.prologue = g.prologue; a.epilogue = g.epilogue; a.prologue_arg = g.prologue_arg; a.epilogue_arg = g.epilogue_arg;
    const int64_t threads = (int64_t)g.M * ((g.N + 3) / 4);
    const int64_t blocks = (threads + 255) / 256;
    if (blocks <= 0 || blocks > 0x7fffffffll) return hipErrorInvalidValue;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a.ws, a.C, a.splits, a.M, a.N, a.c_rs, a.c_cs, a);
    return hipGetLastError();
}

} // namespace acc950
