/*
 * CPU oracle for the matmul + fused-ReLU hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the HIP kernels are compared against and the
 * "port" CPU baseline that the benchmark times beside them.  Nothing in the
 * shipped library links, loads or calls it.
 *
 * It restates, in plain C, the loop nests of the reference:
 *
 *   matmul nest   C[i,j] += A[i,k] * B[k,j]
 *                 /root/reference/README.md:59-65
 *                 /root/reference/accera/python/accera/test/mfma_tests.py:58-66
 *   relu nest     C[i,j] = max(C[i,j], 0)
 *                 /root/reference/README.md:67-71
 *   fusion        fuse(matmul, relu, partial=2): for every (i,j) all k of the
 *                 matmul run before the relu of that (i,j)
 *                 /root/reference/README.md:75-77
 *                 /root/reference/docs/Manual/04 Fusing.md:179-239
 *   schedules     "naive"        order i, j, {k..., relu}      README.md:76-77
 *                 "transformed"  i,j tiled 16x16, order j,i,f,k,jj,ii
 *                                                               README.md:79-88
 *   prologue/epilogue ops of the tensorized GPU plan
 *                 SET (C tile := 0 before accumulating), ReLU,
 *                 ReLU_NoConditional
 *                 /root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:630-655
 *                 /root/reference/accera/python/accera/test/mfma_tests.py:380-432
 *
 * Type rule.  Inputs are widened to the accumulator type before the multiply
 * (float for f32/f16/bf16 inputs, int32 for int8 inputs) and the sum is kept in
 * the accumulator type for the whole k range; this is what the tensorized GPU
 * path does (MFMA semantics: the matcher skips casts between mul and add,
 * /root/reference/accera/transforms/src/exec/ExecutionPlanToAffineLoweringPass.cpp:6149-6167)
 * and what the exact-integer host tests spell out with explicit casts
 * (/root/reference/accera/python/accera/test/int_matmul_tests.py:55).
 * The epilogue runs once, after the full-k sum; narrowing to f16/bf16 output
 * rounds to nearest even (the reference's GPU bf16 store truncates,
 * CppPrinterUtils.h:107-117; the difference is below the 1e-2 tolerance).
 *
 * What pins this file (tests/test_oracle.py):
 *   - the reference's known answers A=2,B=3,C=0.42 -> 6K+0.42
 *     (docs/Tutorials/Hello_MatMul.md:165-237, Optimized_MatMul.md:204-280)
 *   - brute-force int64 / float64 NumPy matmul on small shapes, signed data
 *   - identity / permutation B (C == A bit-exactly), power-of-two entries
 *   - exhaustive half <-> float and bf16 <-> float conversion tables against
 *     NumPy float16 and torch bfloat16
 *   - ReLU on -0, NaN, +-inf, INT32_MIN for both epilogue flavours
 *   - both schedules give bit-identical results (same per-element k order)
 *
 * Parity unpinned (nothing in the reference tree fixes it and the reference cannot be
 * built or imported here): the exact float summation order / fast-math result of an
 * Accera-generated HOST package.  It is irrelevant at the tolerances the reference's own
 * tests use (rtol 1e-5 ... 1e-2); integer results are exact and therefore pinned.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { ORA_F32 = 0, ORA_F16 = 1, ORA_BF16 = 2, ORA_I8 = 3, ORA_I32 = 4, ORA_I16 = 5 };
enum { ORA_PRO_NONE = 0, ORA_PRO_SET0 = 1 };
enum { ORA_EPI_NONE = 0, ORA_EPI_RELU = 1, ORA_EPI_RELU_NOCOND = 2 };
enum { ORA_SCHED_NAIVE = 0, ORA_SCHED_TRANSFORMED = 1 };

/* ---- scalar type conversions ------------------------------------------- */

static inline float bits_to_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t float_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* IEEE binary16 -> binary32, exact. */
float oracle_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_to_float(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * (1.0f / 16777216.0f);
        return bits_to_float(sign | float_to_bits(v));
    }
    if (exp == 31) return bits_to_float(sign | 0x7f800000u | (man << 13));
    return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

/* binary32 -> binary16, round to nearest even. */
uint16_t oracle_float_to_half(float f)
{
    uint32_t u = float_to_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) /* inf or nan */
        return (uint16_t)(sign | 0x7c00u | (a > 0x7f800000u ? (0x200u | ((a >> 13) & 0x3ffu)) : 0));
    if (a >= 0x477ff000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    if (a < 0x38800000u) { /* below the smallest normal half: result is subnormal or zero */
        if (a < 0x33000000u) return sign; /* < 2^-25 -> 0 (2^-25 itself ties to even = 0) */
        uint32_t e = a >> 23;                        /* 102..112 */
        uint32_t m = (a & 0x7fffffu) | 0x800000u;    /* 24-bit significand */
        uint32_t shift = 126u - e;                   /* 14..24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t q = (a - 0x38000000u) >> 13; /* rebias exponent, drop 13 mantissa bits */
    uint32_t rem = a & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

/* bfloat16 -> binary32: exact shift (reference: CppPrinterUtils.h:95-104). */
float oracle_bf16_to_float(uint16_t b) { return bits_to_float((uint32_t)b << 16); }

/* binary32 -> bfloat16, round to nearest even, NaN kept quiet. */
uint16_t oracle_float_to_bf16(float f)
{
    uint32_t u = float_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* ---- epilogue ----------------------------------------------------------- */

/* relu: v > 0 ? v : 0 (NaN -> 0, -0 -> +0);  relu_no_conditional: v *= (v > 0)
 * (NaN stays NaN, -x -> -0).  CppPrinterUtils.h:630-643. */
static inline float epi_f(float v, int epi)
{
    if (epi == ORA_EPI_RELU) return v > 0.0f ? v : 0.0f;
    if (epi == ORA_EPI_RELU_NOCOND) return v * (float)(v > 0.0f);
    return v;
}
static inline int32_t epi_i(int32_t v, int epi)
{
    if (epi == ORA_EPI_RELU) return v > 0 ? v : 0;
    if (epi == ORA_EPI_RELU_NOCOND) return v * (int32_t)(v > 0);
    return v;
}

/* ---- element access ------------------------------------------------------ */

static inline float load_f(const void* p, int type, int64_t idx)
{
    switch (type) {
    case ORA_F32: return ((const float*)p)[idx];
    case ORA_F16: return oracle_half_to_float(((const uint16_t*)p)[idx]);
    default: return oracle_bf16_to_float(((const uint16_t*)p)[idx]);
    }
}
static inline void store_f(void* p, int type, int64_t idx, float v)
{
    switch (type) {
    case ORA_F32: ((float*)p)[idx] = v; break;
    case ORA_F16: ((uint16_t*)p)[idx] = oracle_float_to_half(v); break;
    default: ((uint16_t*)p)[idx] = oracle_float_to_bf16(v); break;
    }
}

/* Widen a strided float-family matrix into a dense row-major float copy (exact). */
static float* widen_f(const void* p, int type, int rows, int cols, int64_t rs, int64_t cs)
{
    float* w = (float*)malloc((size_t)rows * (size_t)cols * sizeof(float));
    if (!w) return NULL;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c)
            w[(size_t)r * cols + c] = load_f(p, type, r * rs + c * cs);
    return w;
}

#define TILE 16 /* README.md:81-84 */

/* ---- float family -------------------------------------------------------- */

static int gemm_f(int in_type, int out_type, int M, int N, int K,
                  const void* A, int64_t a_rs, int64_t a_cs,
                  const void* B, int64_t b_rs, int64_t b_cs,
                  void* C, int64_t c_rs, int64_t c_cs,
                  int prologue, int epilogue, int schedule)
{
    /* dense row-major float copies: Aw[M][K], Bw[K][N]; values are unchanged */
    float* Aw = widen_f(A, in_type, M, K, a_rs, a_cs);
    float* Bw = widen_f(B, in_type, K, N, b_rs, b_cs);
    if (!Aw || !Bw) { free(Aw); free(Bw); return -2; }

    if (schedule == ORA_SCHED_NAIVE) {
        /* order i, j, {k..., relu} */
#pragma omp parallel for schedule(static)
        for (int i = 0; i < M; ++i)
            for (int j = 0; j < N; ++j) {
                float acc = prologue == ORA_PRO_SET0 ? 0.0f : load_f(C, out_type, i * c_rs + j * c_cs);
                for (int k = 0; k < K; ++k)
                    acc += Aw[(size_t)i * K + k] * Bw[(size_t)k * N + j];
                store_f(C, out_type, i * c_rs + j * c_cs, epi_f(acc, epilogue));
            }
    } else {
        /* i,j split by 16; order j, i, f, k, jj, ii; f=0 matmul, f=1 relu */
        int nj = (N + TILE - 1) / TILE;
#pragma omp parallel for schedule(static)
        for (int jt = 0; jt < nj; ++jt) {
            int j0 = jt * TILE, jn = N - j0 < TILE ? N - j0 : TILE;
            for (int i0 = 0; i0 < M; i0 += TILE) {
                int in = M - i0 < TILE ? M - i0 : TILE;
                float acc[TILE][TILE];
                for (int jj = 0; jj < jn; ++jj)
                    for (int ii = 0; ii < in; ++ii)
                        acc[ii][jj] = prologue == ORA_PRO_SET0
                                          ? 0.0f
                                          : load_f(C, out_type, (i0 + ii) * c_rs + (j0 + jj) * c_cs);
                for (int k = 0; k < K; ++k)
                    for (int ii = 0; ii < in; ++ii) {
                        float a = Aw[(size_t)(i0 + ii) * K + k];
                        const float* brow = Bw + (size_t)k * N + j0;
                        for (int jj = 0; jj < jn; ++jj)
                            acc[ii][jj] += a * brow[jj];
                    }
                for (int jj = 0; jj < jn; ++jj)
                    for (int ii = 0; ii < in; ++ii)
                        store_f(C, out_type, (i0 + ii) * c_rs + (j0 + jj) * c_cs, epi_f(acc[ii][jj], epilogue));
            }
        }
    }
    free(Aw);
    free(Bw);
    return 0;
}

/* ---- int8 -> int32 ------------------------------------------------------- */

static int gemm_i(int M, int N, int K,
                  const int8_t* A, int64_t a_rs, int64_t a_cs,
                  const int8_t* B, int64_t b_rs, int64_t b_cs,
                  int32_t* C, int64_t c_rs, int64_t c_cs,
                  int prologue, int epilogue, int schedule)
{
    if (schedule == ORA_SCHED_NAIVE) {
#pragma omp parallel for schedule(static)
        for (int i = 0; i < M; ++i)
            for (int j = 0; j < N; ++j) {
                /* unsigned arithmetic: wrap-around on overflow is defined */
                uint32_t acc = prologue == ORA_PRO_SET0 ? 0u : (uint32_t)C[i * c_rs + j * c_cs];
                for (int k = 0; k < K; ++k)
                    acc += (uint32_t)((int32_t)A[i * a_rs + k * a_cs] * (int32_t)B[k * b_rs + j * b_cs]);
                C[i * c_rs + j * c_cs] = epi_i((int32_t)acc, epilogue);
            }
        return 0;
    }
    int nj = (N + TILE - 1) / TILE;
#pragma omp parallel for schedule(static)
    for (int jt = 0; jt < nj; ++jt) {
        int j0 = jt * TILE, jn = N - j0 < TILE ? N - j0 : TILE;
        for (int i0 = 0; i0 < M; i0 += TILE) {
            int in = M - i0 < TILE ? M - i0 : TILE;
            uint32_t acc[TILE][TILE];
            for (int jj = 0; jj < jn; ++jj)
                for (int ii = 0; ii < in; ++ii)
                    acc[ii][jj] = prologue == ORA_PRO_SET0 ? 0u : (uint32_t)C[(i0 + ii) * c_rs + (j0 + jj) * c_cs];
            for (int k = 0; k < K; ++k)
                for (int ii = 0; ii < in; ++ii) {
                    int32_t a = A[(i0 + ii) * a_rs + k * a_cs];
                    const int8_t* brow = B + k * b_rs + j0 * b_cs;
                    if (b_cs == 1)
                        for (int jj = 0; jj < jn; ++jj) acc[ii][jj] += (uint32_t)(a * (int32_t)brow[jj]);
                    else
                        for (int jj = 0; jj < jn; ++jj) acc[ii][jj] += (uint32_t)(a * (int32_t)brow[jj * b_cs]);
                }
            for (int jj = 0; jj < jn; ++jj)
                for (int ii = 0; ii < in; ++ii)
                    C[(i0 + ii) * c_rs + (j0 + jj) * c_cs] = epi_i((int32_t)acc[ii][jj], epilogue);
        }
    }
    return 0;
}

/*
 * C = epilogue( (prologue == SET0 ? 0 : C) + A * B )
 *
 * A is M x K, B is K x N, C is M x N; *_rs / *_cs are the row / column strides
 * in elements (row-major: rs = cols, cs = 1; column-major: rs = 1, cs = rows),
 * the same numbers a .hat file carries as affine_map
 * (/root/reference/accera/ir/src/TranslateToHeader.cpp:726-753).
 * in_type: ORA_F32 | ORA_F16 | ORA_BF16 (out_type any float type), or ORA_I8
 * (out_type ORA_I32, or ORA_I16 / ORA_I8: C widens with its sign on the way in and
 * keeps the low bits of the int32 result on the way out, the plain C conversions of
 * /root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:277-293).  Returns 0, -1 on a bad type combination, -2 on
 * allocation failure.  Threads are set by the caller through OMP_NUM_THREADS /
 * oracle_set_threads().
 */
int oracle_gemm_relu(int in_type, int out_type, int M, int N, int K,
                     const void* A, int64_t a_rs, int64_t a_cs,
                     const void* B, int64_t b_rs, int64_t b_cs,
                     void* C, int64_t c_rs, int64_t c_cs,
                     int prologue, int epilogue, int schedule)
{
    if (M < 0 || N < 0 || K < 0) return -1;
    if (in_type == ORA_I8) {
        if (out_type == ORA_I16 || out_type == ORA_I8) {
            /* through an int32 copy of C */
            int32_t* T = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M > 0 ? M : 1) * (size_t)(N > 0 ? N : 1));
            if (!T) return -2;
            for (int i = 0; i < M; ++i)
                for (int j = 0; j < N; ++j) {
                    const int64_t idx = i * c_rs + j * c_cs;
                    T[(int64_t)i * N + j] = out_type == ORA_I16 ? (int32_t)((const int16_t*)C)[idx] : (int32_t)((const int8_t*)C)[idx];
                }
            int rc = gemm_i(M, N, K, (const int8_t*)A, a_rs, a_cs, (const int8_t*)B, b_rs, b_cs, T, N, 1, prologue, epilogue, schedule);
            for (int i = 0; i < M && rc == 0; ++i)
                for (int j = 0; j < N; ++j) {
                    const int64_t idx = i * c_rs + j * c_cs;
                    const uint32_t u = (uint32_t)T[(int64_t)i * N + j];
                    if (out_type == ORA_I16) ((uint16_t*)C)[idx] = (uint16_t)u; /* same bits as the int16_t conversion */
                    else ((uint8_t*)C)[idx] = (uint8_t)u;
                }
            free(T);
            return rc;
        }
        if (out_type != ORA_I32) return -1;
        return gemm_i(M, N, K, (const int8_t*)A, a_rs, a_cs, (const int8_t*)B, b_rs, b_cs,
                      (int32_t*)C, c_rs, c_cs, prologue, epilogue, schedule);
    }
    if (in_type != ORA_F32 && in_type != ORA_F16 && in_type != ORA_BF16) return -1;
    if (out_type != ORA_F32 && out_type != ORA_F16 && out_type != ORA_BF16) return -1;
    return gemm_f(in_type, out_type, M, N, K, A, a_rs, a_cs, B, b_rs, b_cs, C, c_rs, c_cs,
                  prologue, epilogue, schedule);
}

#ifdef _OPENMP
#include <omp.h>
void oracle_set_threads(int n) { omp_set_num_threads(n > 0 ? n : 1); }
int oracle_max_threads(void) { return omp_get_max_threads(); }
#else
void oracle_set_threads(int n) { (void)n; }
int oracle_max_threads(void) { return 1; }
#endif

/* Vector forms of the scalar conversions, for the exhaustive table tests. */
void oracle_half_to_float_n(const uint16_t* in, float* out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = oracle_half_to_float(in[i]); }
void oracle_float_to_half_n(const float* in, uint16_t* out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = oracle_float_to_half(in[i]); }
void oracle_bf16_to_float_n(const uint16_t* in, float* out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = oracle_bf16_to_float(in[i]); }
void oracle_float_to_bf16_n(const float* in, uint16_t* out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = oracle_float_to_bf16(in[i]); }
