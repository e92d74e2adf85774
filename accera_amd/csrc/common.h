// Shared declarations for the gfx950 GEMM+ReLU kernels and their host launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <mutex>

namespace acc950 {

// Element types (values match include/accera_mi355x_gemm.h).
enum : int { T_F32 = 0, T_F16 = 1, T_BF16 = 2, T_I8 = 3, T_I32 = 4, T_I16 = 5 };
// Prologue / epilogue ops of the tensorized plan
// (/root/reference/accera/python/accera/lang/Plan.py:208-379, fragment ops
//  /root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:630-655).
// Prologue acts on the C fragment before the products are added (NONE: keep C, SET: C = arg,
// SCALE: C *= arg); epilogue acts on the finished sum.  Arguments are cast to the
// accumulator type (float or int), as the reference's fragment helpers do.
enum : int { PRO_NONE = 0, PRO_SET = 1, PRO_SET0 = 1, PRO_SCALE = 2 };
enum : int { EPI_NONE = 0, EPI_RELU = 1, EPI_RELU_NOCOND = 2, EPI_SCALE = 3, EPI_SET = 4 };

// Arguments of one GEMM launch.  Strides are in elements.
struct GemmArgs {
    const void* A;
    const void* B;
    void* C;
    int M, N, K;
    int64_t a_rs, a_cs; // A[i,k] at i*a_rs + k*a_cs
    int64_t b_rs, b_cs; // B[k,j] at k*b_rs + j*b_cs
    int64_t c_rs, c_cs; // C[i,j] at i*c_rs + j*c_cs
    int in_type, out_type;
    int prologue, epilogue;
    float prologue_arg, epilogue_arg; // SET / SCALE operand (0 for the other ops)
    int tiles_m, tiles_n; // workgroup grid in tiles (MFMA kernels)
    int batch;                  // independent problems, one per blockIdx.z (1 for a plain GEMM)
    int64_t a_bs, b_bs, c_bs;   // element distance between consecutive problems of a batch
    int k_last;                 // > 0: K of the last problem of the batch (a K split run as a batch of partial products: the last slice is what is left)
    int stagger_groups, stagger_ticks; // multi-tile kernels: workgroup group g of stagger_groups starts g * stagger_ticks * 10 ns late (0: no stagger)
    unsigned long long* stamps; // timed MFMA instantiation only: [workgroup][4 points][shader clock, 100 MHz clock]
};

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

#define ACC950_LDS __attribute__((address_space(3)))
#define ACC950_GLOBAL __attribute__((address_space(1)))

// ---- scalar conversions --------------------------------------------------------

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }

// float -> bfloat16 bits, round to nearest even, NaN kept quiet.  (The reference's
// GPU store truncates, CppPrinterUtils.h:107-117; nearest-even is what its LLVM
// host path and this library's oracle do.)
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f)
{
    return __builtin_bit_cast(uint16_t, (__bf16)f); // v_cvt_pk_bf16_f32
}

__device__ __forceinline__ uint16_t float_to_f16_bits(float f)
{
    _Float16 h = (_Float16)f; // v_cvt_f16_f32: round to nearest even
    return __builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ float f16_bits_to_float(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }

// ---- fragment ops (CppPrinterUtils.h:630-655) ------------------------------------
// relu:                v > 0 ? v : 0     (NaN -> 0, -0 -> +0)
// relu_no_conditional: v *= (v > 0)      (NaN stays NaN, negatives -> -0)
// scale:               v *= arg          set: v = arg
__device__ __forceinline__ int wrap_mul(int a, int b) { return (int)((unsigned)a * (unsigned)b); }
__device__ __forceinline__ float wrap_mul(float a, float b) { return a * b; }
__device__ __forceinline__ int wrap_add(int a, int b) { return (int)((unsigned)a + (unsigned)b); }
__device__ __forceinline__ float wrap_add(float a, float b) { return a + b; }

template <typename T>
__device__ __forceinline__ T apply_epilogue(T v, int epi, float arg = 0.f)
{
    if (epi == EPI_RELU) return v > T(0) ? v : T(0);
    if (epi == EPI_RELU_NOCOND) return v * T(v > T(0) ? 1 : 0);
    if (epi == EPI_SCALE) return wrap_mul(v, (T)arg);
    if (epi == EPI_SET) return (T)arg;
    return v;
}

// Sum of products + the prologue'd C element (c_old is only read when the op keeps C).
template <typename T, typename LoadC>
__device__ __forceinline__ T apply_prologue(T sum, int pro, float arg, LoadC&& load_c)
{
    if (pro == PRO_SET) return wrap_add(sum, (T)arg);
    if (pro == PRO_SCALE) return wrap_add(sum, wrap_mul(load_c(), (T)arg));
    return wrap_add(sum, load_c());
}

// Cache policy of the stores to C in the LDS-tiled MFMA kernels of the 32x32 shapes and the eight-wave 16x16 ones:
// `sc1 nt` (bit 4 and bit 1 of a buffer instruction's aux operand).  A store whose line is already in the L2 -- a C
// that the same launch has read for its prologue -- otherwise leaves a dirty line there, and all of them are written
// back only when the kernel ends, after the last wave, at about 1 us per MB: 2048^3 fp16 with beta = 1 took 27.1 us
// against 20.8 with beta = 0 on every kernel of the library, the thread-bound one included.  With `sc1` the store goes
// through to memory while the kernel still runs (22.1 us); `nt` keeps the line from taking room that the operand
// panels use (worth 0.5 - 1 us by itself on problems of 20 us that only write C).  Not for everything: the small fp32
// kernel, whose stores are the last thing a 9 us launch does, loses 2.6 us waiting for them to reach memory, and the
// four-wave kernels (a C far larger than the L2, lines gone before the kernel ends) keep `nt` alone: with `sc1` they
// measured 1 % slower when C is only written and 0 - 1 % faster when it is read.
constexpr int C_STORE_AUX = 16 | 2;

// Store one float accumulator as the output element type.
__device__ __forceinline__ void store_out(void* C, int out_type, int64_t idx, float v)
{
    if (out_type == T_F32) ((float*)C)[idx] = v;
    else if (out_type == T_F16) ((uint16_t*)C)[idx] = float_to_f16_bits(v);
    else ((uint16_t*)C)[idx] = float_to_bf16_bits(v);
}
__device__ __forceinline__ float load_out(const void* C, int out_type, int64_t idx)
{
    if (out_type == T_F32) return ((const float*)C)[idx];
    if (out_type == T_F16) return f16_bits_to_float(((const uint16_t*)C)[idx]);
    return bf16_bits_to_float(((const uint16_t*)C)[idx]);
}

// Integer outputs: int8 / int16 elements widen with their sign on the way in and keep the
// low bits of the int32 sum on the way out, as the reference's accumulator fragment load / store
// does with plain C conversions (/root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:277-293).
__device__ __forceinline__ void store_out_int(void* C, int out_type, int64_t idx, int v)
{
    if (out_type == T_I32) ((int*)C)[idx] = v;
    else if (out_type == T_I16) ((int16_t*)C)[idx] = (int16_t)v;
    else ((int8_t*)C)[idx] = (int8_t)v;
}
__device__ __forceinline__ int load_out_int(const void* C, int out_type, int64_t idx)
{
    if (out_type == T_I32) return ((const int*)C)[idx];
    if (out_type == T_I16) return ((const int16_t*)C)[idx];
    return ((const int8_t*)C)[idx];
}

// The first 16 dwords of a kernel's arguments are preloaded into scalar registers when the kernel is dispatched (the
// translation units are built with -amdgpu-kernarg-preload-count=16); what lies behind them is fetched by the kernel itself,
// a trip through memory of about 0.4 us before its first address can be formed (an empty kernel: 2.5 us from launch to
// launch; one that loads and stores a few bytes: 3.0 us with its arguments fetched, 2.6 with them preloaded).  Only scalar
// and pointer arguments are preloaded, not a struct, so the kernels take the fields they need first -- operand pointers,
// sizes, strides -- as arguments of their own in front of the struct and put them back into their copy of it.
// (14 dwords fit beside the registers the dispatch itself needs: two pointers, three sizes, the element strides of A and B
// along K -- 32 bits: the entry points refuse larger ones --, the stagger switch of the multi-tile kernels, which they test
// first thing, and the two row strides.  The MFMA kernels work out their tile counts from M and N themselves.)
#define ACC950_HEAD_PARAMS const void* head_A, const void* head_B, int head_M, int head_N, int head_K, int head_a_cs, int head_b_cs, \
                           int head_stagger_groups, int64_t head_a_rs, int64_t head_b_rs
#define ACC950_HEAD_OF(g) (g).A, (g).B, (g).M, (g).N, (g).K, (int)(g).a_cs, (int)(g).b_cs, (g).stagger_groups, (g).a_rs, (g).b_rs
#define ACC950_TAKE_HEAD(p)                                                                                                      \
    do {                                                                                                                          \
        (p).A = head_A; (p).B = head_B; (p).M = head_M; (p).N = head_N; (p).K = head_K; (p).stagger_groups = head_stagger_groups; \
        (p).a_rs = head_a_rs; (p).b_rs = head_b_rs; (p).a_cs = head_a_cs; (p).b_cs = head_b_cs;                                   \
    } while (0)
// (the MFMA kernels: tile counts as their launchers set them)
#define ACC950_TAKE_HEAD_TILES(p, BM_, BN_)                                                   \
    do {                                                                                      \
        ACC950_TAKE_HEAD(p);                                                                  \
        (p).tiles_m = ((p).M + (BM_) - 1) / (BM_); (p).tiles_n = ((p).N + (BN_) - 1) / (BN_); \
    } while (0)

// Batched launch: blockIdx.z picks the problem; the kernel then sees one plain GEMM.
__device__ __forceinline__ int elem_bytes(int type) { return type == T_I8 ? 1 : (type == T_F16 || type == T_BF16 || type == T_I16) ? 2 : 4; }
// (Problem 0 needs none of this -- a K split has at least two slices, so its last slice is never slice 0 -- and a plain
// GEMM is all problem 0: its workgroups do not wait for the batch fields, which are not among the preloaded arguments.)
__device__ __forceinline__ void select_batch(GemmArgs& p)
{
    const int64_t z = blockIdx.z;
    if (z == 0) return;
    p.A = (const char*)p.A + z * p.a_bs * elem_bytes(p.in_type);
    p.B = (const char*)p.B + z * p.b_bs * elem_bytes(p.in_type);
    p.C = (char*)p.C + z * p.c_bs * elem_bytes(p.out_type);
    if (p.k_last > 0 && (int)z == p.batch - 1) p.K = p.k_last;
}

// MI355X: 256 compute units in 8 XCDs (the library runs on gfx950 only; the launch geometry of the kernels that keep
// one workgroup per CU is part of a package's metadata, so it is a constant and not a device query).
constexpr int kComputeUnits = 256;

// ---- host-side launch record -------------------------------------------------------
struct LaunchGeom {
    unsigned grid[3];
    unsigned block[3];
    unsigned dyn_lds;
};

typedef hipError_t (*LaunchFn)(const GemmArgs&, hipStream_t, LaunchGeom*, bool dry_run);

// Raises a kernel's dynamic LDS limit once per device, whichever host thread launches it first
// (one object per kernel instantiation, as a function-local static of its launcher).
class LdsLimitOnce {
public:
    hipError_t ensure(const void* kernel, int bytes)
    {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        const uint64_t bit = 1ull << (dev & 63);
        std::lock_guard<std::mutex> lock(mutex_);
        if (done_ & bit) return hipSuccess;
        e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        if (e == hipSuccess) done_ |= bit;
        return e;
    }

private:
    std::mutex mutex_;
    uint64_t done_ = 0;
};

} // namespace acc950
