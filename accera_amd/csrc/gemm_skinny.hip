// Bandwidth-bound "skinny" GEMM for decode-shaped problems: M <= 8 rows of A against a
// large row-major B (K x N, N contiguous), fp32 accumulate, fused epilogue, fp16 / bf16
// / fp32 output.  No MFMA: the kernel is a pure stream over B with wavefront-level
// reductions.
//
// In the reference such a shape can only take the non-tensorized thread-bound plan
// (M = 8 is below every MMA shape: /root/reference/accera/python/accera/test/mfma_tests.py:250-278,309-356).
// That plan forms products in the input type; this kernel widens to fp32 first.
//
// Work split
//   * grid.x = column blocks of CB = 8*LPR columns, grid.y = K splits.
//   * inside a wave, lane = kp*LPR + cg: cg picks 8 adjacent columns (one 16-byte load
//     per B row), kp picks a pair of adjacent k rows, so a wave instruction pair
//     covers 2*(64/LPR) rows x CB columns; rows are dealt round-robin to the waves.
//   * two k rows are interleaved with v_perm_b32 into (k, k+1) half pairs and
//     multiplied with the matching A pair by v_dot2_f32_f16 / v_dot2_f32_bf16
//     (2 MACs per lane per instruction, fp32 accumulate): 8x8 accumulators per lane.
//   * A (at most 8 x K) is staged once per workgroup in LDS as [k pair][m] so that a
//     lane fetches its 8 pairs with two ds_read_b128.
//   * at the end the 64/LPR partial sums held by different lanes are combined with a
//     halving butterfly (each step exchanges half of the live values with the lane
//     32, 16, 8 ... away), then across waves through LDS, then -- when the K range is
//     split over workgroups -- through an fp32 scratch buffer where the last
//     workgroup to arrive sums the slices in fixed order (deterministic result).
#include "common.h"
#include "skinny.h"

namespace acc950 {

namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

template <bool BF16>
__device__ __forceinline__ float dot2(unsigned a, unsigned b, float c)
{
    if constexpr (BF16) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
    } else {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
    }
}

// LPR: lanes per B row segment (8 columns each); WAVES: waves per workgroup.
template <bool BF16, int LPR, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) gemm_skinny_kernel(SkinnyArgs p)
{
    constexpr int NT = WAVES * 64;
    constexpr int NKP = 64 / LPR;        // k pairs per wave instruction
    constexpr int CB = LPR * 8;          // columns per workgroup
    constexpr int VPL = 64 / NKP;        // values per lane after the butterfly
    extern __shared__ __attribute__((aligned(16))) char smem[];
    unsigned* sA = (unsigned*)smem;      // [k pair][8] half pairs

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kp = lane / LPR, cg = lane % LPR;
    const int col0 = blockIdx.x * CB + cg * 8;
    const bool col_ok = col0 < p.N; // N is a multiple of 8

    // K range of this workgroup, in k pairs
    const int pairs_total = p.K / 2;
    const int pairs_per_split = (pairs_total + p.splits - 1) / p.splits;
    const int pair_begin = blockIdx.y * pairs_per_split;
    const int pair_end = min(pair_begin + pairs_per_split, pairs_total);
    const int npairs = max(pair_end - pair_begin, 0);

    // stage A[0..8) x [2*pair_begin, 2*pair_end) as [pair][m]; rows >= M are zero
    const unsigned* A32 = (const unsigned*)p.A;
    for (int e = tid; e < npairs * 8; e += NT) {
        int m = e / npairs, pr = e % npairs;
        unsigned v = 0;
        if (m < p.M) v = A32[((int64_t)m * p.a_rs) / 2 + pair_begin + pr];
        sA[pr * 8 + m] = v;
    }
    __syncthreads();

    float acc[8][8];
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
        for (int n = 0; n < 8; ++n) acc[m][n] = 0.f;

    const char* Bb = (const char*)p.B;
    const int64_t row_bytes = p.b_rs * 2;
    constexpr int STEP = WAVES * NKP; // k pairs per workgroup pass
    const int iters = (npairs + STEP - 1) / STEP;
    constexpr int U = 4;
    for (int it0 = 0; it0 < iters; it0 += U) {
        u32x4 b0[U], b1[U];
        int pr[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            pr[u] = (it0 + u) * STEP + wave * NKP + kp;
            const bool ok = col_ok && pr[u] < npairs;
            b0[u] = u32x4{0, 0, 0, 0};
            b1[u] = u32x4{0, 0, 0, 0};
            if (ok) {
                const char* g = Bb + (int64_t)(2 * (pair_begin + pr[u])) * row_bytes + (int64_t)col0 * 2;
                b0[u] = __builtin_nontemporal_load((const u32x4*)g);
                b1[u] = __builtin_nontemporal_load((const u32x4*)(g + row_bytes));
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool in_range = pr[u] < npairs;
            const int prc = in_range ? pr[u] : 0;
            u32x4 a_lo = *(const u32x4*)(sA + prc * 8);
            u32x4 a_hi = *(const u32x4*)(sA + prc * 8 + 4);
            if (!in_range) { // keep 0 * inf out of the sums
                a_lo = u32x4{0, 0, 0, 0};
                a_hi = u32x4{0, 0, 0, 0};
            }
            unsigned bp[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                bp[2 * j] = __builtin_amdgcn_perm(b1[u][j], b0[u][j], 0x05040100u);     // (B[k][n], B[k+1][n]), n even
                bp[2 * j + 1] = __builtin_amdgcn_perm(b1[u][j], b0[u][j], 0x07060302u); // n odd
            }
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                const unsigned am = m < 4 ? a_lo[m & 3] : a_hi[m & 3];
#pragma unroll
                for (int n = 0; n < 8; ++n) acc[m][n] = dot2<BF16>(am, bp[n], acc[m][n]);
            }
        }
    }

    // ---- reduce over the NKP lane groups: halving butterfly ----
    // before: lane holds v[e], e = m*8+n, partial over its own k pairs
    // after : lane holds VPL values, e = j + VPL*kp, summed over all kp of the wave
    float v[64];
#pragma unroll
    for (int e = 0; e < 64; ++e) v[e] = acc[e >> 3][e & 7];
    int live = 64;
#pragma unroll
    for (int dist = 32; dist >= LPR; dist >>= 1) {
        const bool upper = (lane & dist) != 0;
        const int half = live / 2;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            if (j < half) {
                const float send = upper ? v[j] : v[j + half];
                const float keep = upper ? v[j + half] : v[j];
                v[j] = keep + __shfl_xor(send, dist, 64);
            }
        }
        live = half;
    }

    // ---- reduce over waves through LDS (reuses the A staging area) ----
    __syncthreads();
    float* red = (float*)smem; // [wave][VPL][64]
    if (wave > 0) {
#pragma unroll
        for (int j = 0; j < VPL; ++j) red[((wave - 1) * VPL + j) * 64 + lane] = v[j];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int w = 1; w < WAVES; ++w)
#pragma unroll
        for (int j = 0; j < VPL; ++j) v[j] += red[((w - 1) * VPL + j) * 64 + lane];

    // lane (kp, cg) now owns elements e = j + VPL*kp: m = e/8, n = e%8 of columns col0..col0+7
    auto finish = [&](int m, int n, float s) {
        if (!col_ok || m >= p.M) return;
        const int64_t idx = (int64_t)m * p.c_rs + (col0 + n);
        if (p.prologue == PRO_NONE) s += load_out(p.C, p.out_type, idx);
        store_out(p.C, p.out_type, idx, apply_epilogue<float>(s, p.epilogue));
    };

    if (p.splits == 1) {
#pragma unroll
        for (int j = 0; j < VPL; ++j) finish((j + VPL * kp) >> 3, (j + VPL * kp) & 7, v[j]);
        return;
    }

    // ---- K split over workgroups: partial sums to scratch, last arrival finishes ----
    float* part = p.scratch + ((int64_t)blockIdx.y * gridDim.x + blockIdx.x) * (64 * LPR);
#pragma unroll
    for (int j = 0; j < VPL; ++j) part[j * 64 + lane] = v[j];
    __threadfence();
    unsigned ticket = 0;
    if (lane == 0) ticket = atomicAdd(p.counters + blockIdx.x, 1u);
    ticket = __shfl(ticket, 0, 64);
    if (ticket != (unsigned)p.splits - 1) return;
    __threadfence();
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
        float s = 0.f;
        for (int sp = 0; sp < p.splits; ++sp)
            s += __builtin_nontemporal_load(p.scratch + ((int64_t)sp * gridDim.x + blockIdx.x) * (64 * LPR) + j * 64 + lane);
        finish((j + VPL * kp) >> 3, (j + VPL * kp) & 7, s);
    }
    if (lane == 0) p.counters[blockIdx.x] = 0; // ready for the next launch
}

template <bool BF16, int LPR, int WAVES>
hipError_t launch_one(const SkinnyArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    constexpr int CB = LPR * 8;
    auto kern = gemm_skinny_kernel<BF16, LPR, WAVES>;
    const int pairs_per_split = (a.K / 2 + a.splits - 1) / a.splits;
    unsigned lds = (unsigned)pairs_per_split * 32u;
    const unsigned red = (WAVES - 1) * (64 / (64 / LPR)) * 64 * 4;
    if (lds < red) lds = red;
    dim3 grid((a.N + CB - 1) / CB, a.splits, 1), block(WAVES * 64, 1, 1);
    if (geom) {
        geom->grid[0] = grid.x; geom->grid[1] = grid.y; geom->grid[2] = 1;
        geom->block[0] = block.x; geom->block[1] = geom->block[2] = 1;
        geom->dyn_lds = lds;
    }
    if (dry_run) return hipSuccess;
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    static unsigned attr_lds = 0;
    if (lds > 64 * 1024 && lds > attr_lds) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_lds = 160 * 1024;
    }
    hipLaunchKernelGGL(kern, grid, block, lds, stream, a);
    return hipGetLastError();
}

struct SkinnyVariant {
    int lpr, waves;
    hipError_t (*f16)(const SkinnyArgs&, hipStream_t, LaunchGeom*, bool);
    hipError_t (*bf16)(const SkinnyArgs&, hipStream_t, LaunchGeom*, bool);
};
#define SV(LPR, W) { LPR, W, &launch_one<false, LPR, W>, &launch_one<true, LPR, W> }
const SkinnyVariant kSkinny[] = { SV(8, 4), SV(8, 8), SV(8, 16), SV(16, 4), SV(16, 8), SV(4, 8), SV(4, 4) };
#undef SV
constexpr int kNumSkinny = (int)(sizeof(kSkinny) / sizeof(kSkinny[0]));

} // namespace

int skinny_num_variants() { return kNumSkinny; }
void skinny_variant_info(int v, int* lpr, int* waves)
{
    *lpr = kSkinny[v].lpr;
    *waves = kSkinny[v].waves;
}
int skinny_column_blocks(int v, int N) { return (N + kSkinny[v].lpr * 8 - 1) / (kSkinny[v].lpr * 8); }
size_t skinny_scratch_floats(int v, int N, int splits)
{
    return splits <= 1 ? 0 : (size_t)splits * skinny_column_blocks(v, N) * 64 * kSkinny[v].lpr;
}

hipError_t launch_skinny(int v, const SkinnyArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    if (v < 0 || v >= kNumSkinny) return hipErrorInvalidValue;
    return a.in_type == T_BF16 ? kSkinny[v].bf16(a, stream, geom, dry_run) : kSkinny[v].f16(a, stream, geom, dry_run);
}

} // namespace acc950
