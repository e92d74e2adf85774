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
//   * inside a wave, lane = kp*LPR + cg: cg picks 8 adjacent columns (16 bytes of a B
//     row), kp picks a pair of adjacent k rows, so one wave step covers 2*(64/LPR) rows
//     x CB columns; steps are dealt round-robin to the waves of the workgroup.
//   * every wave is an independent streaming engine: it owns a ring of DEPTH slots in
//     LDS and fills them with global_load_lds (no staging registers): per step two
//     16-byte-per-lane loads for the two B rows and one 4-byte-per-lane load for the
//     matching A pairs, laid out [k pair][m].  DEPTH steps are in flight per wave at all
//     times (s_waitcnt vmcnt(3*(DEPTH-1)) admits the oldest), which is what hides the
//     HBM latency; there is no barrier in the streaming phase.
//   * two k rows are interleaved with v_perm_b32 into (k, k+1) half pairs and
//     multiplied with the matching A pair by v_dot2_f32_f16 / v_dot2_f32_bf16
//     (2 MACs per lane per instruction, fp32 accumulate): 8x8 accumulators per lane.
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

// LPR: lanes per B row segment (8 columns each); WAVES: waves per workgroup;
// DEPTH: ring slots (steps in flight) per wave.
template <bool BF16, int LPR, int WAVES, int DEPTH>
__global__ void __launch_bounds__(WAVES * 64) gemm_skinny_kernel(ACC950_SKINNY_HEAD_PARAMS, SkinnyArgs p)
{
    ACC950_SKINNY_TAKE_HEAD(p);
    constexpr int NKP = 64 / LPR;        // k pairs per wave step
    constexpr int CB = LPR * 8;          // columns per workgroup
    constexpr int VPL = 64 / NKP;        // values per lane after the butterfly
    constexpr int SLOT_BYTES = 2048 + 256; // two B rows (64 lanes x 16 B each) + A pairs (64 x 4 B)
    constexpr int RING_BYTES = DEPTH * SLOT_BYTES;
    static_assert(3 * (DEPTH - 1) < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    if (blockIdx.z != 0) { // batched launch: blockIdx.z picks the problem (and its slice of the K-split workspace); problem 0 waits for none of these fields
        const int64_t z = blockIdx.z;
        p.A = (const char*)p.A + z * p.a_bs * 2;
        p.B = (const char*)p.B + z * p.b_bs * 2;
        p.C = (char*)p.C + z * p.c_bs * (p.out_type == T_F32 ? 4 : 2);
        p.scratch += z * p.scratch_bs;
        p.counters += z * p.counter_bs;
    }

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kp = lane / LPR, cg = lane % LPR;
    // Workgroup ids are dealt round-robin to the 8 XCDs; column block = (id % 8) * per + id / 8
    // gives every XCD a contiguous range of blocks, hence all residues of the 128-byte line
    // index and all channels of its L2 (ids mapped 1:1 to blocks would leave an XCD with
    // every 8th line of a row only).
    const int nblocks = (p.N + CB - 1) / CB;
    const int bx = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    if (bx >= nblocks) return;
    const int col0 = bx * CB + cg * 8;
    const bool col_ok = col0 < p.N; // N is a multiple of 8

    // K range of this workgroup, in k pairs
    const int pairs_total = p.K / 2;
    const int pairs_per_split = (pairs_total + p.splits - 1) / p.splits;
    const int pair_begin = blockIdx.y * pairs_per_split;
    const int pair_end = min(pair_begin + pairs_per_split, pairs_total);
    const int npairs = max(pair_end - pair_begin, 0);

    constexpr int STEP = WAVES * NKP; // k pairs per workgroup pass
    const int iters = (npairs + STEP - 1) / STEP;

    // wave-private ring in LDS
    char* ring = smem + wave * RING_BYTES;
    const unsigned ring_addr = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(ACC950_LDS char*)ring);

    // per-lane global byte offsets relative to the (uniform) base of a step; lanes outside
    // the matrix fetch a valid address (column 0 / pair 0) and are masked at the MACs
    const int64_t row_bytes = p.b_rs * 2;
    const char* Bb = (const char*)p.B + (int64_t)(2 * pair_begin) * row_bytes;
    const char* Ab = (const char*)p.A + (int64_t)pair_begin * 4;
    const int am = lane & 7, akp = lane >> 3;            // A fill: lane -> (pair akp of the step, row am)
    auto issue = [&](int it, int slot) {
        const int pr = it * STEP + wave * NKP + kp;      // this lane's pair for B
        const int prc = pr < npairs ? pr : 0;
        const unsigned boff = (unsigned)((int64_t)(2 * prc) * row_bytes + (int64_t)(col_ok ? col0 : 0) * 2);
        const int apr = it * STEP + wave * NKP + (akp < NKP ? akp : 0);
        const int aprc = apr < npairs ? apr : 0;
        const unsigned aoff = (unsigned)((int64_t)(am < p.M ? am : 0) * p.a_rs * 2 + (int64_t)aprc * 4);
        const unsigned dst = ring_addr + slot * SLOT_BYTES;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t"
                     "s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %2\n\t"
                     "s_mov_b32 m0, %5\n\ts_nop 0\n\tglobal_load_lds_dword %6, %7"
                     :
                     : "s"(dst), "v"(boff), "s"(Bb), "s"(dst + 1024), "v"(boff + (unsigned)row_bytes), "s"(dst + 2048),
                       "v"(aoff), "s"(Ab)
                     : "memory");
    };

    float acc[8][8];
#pragma unroll
    for (int m = 0; m < 8; ++m)
#pragma unroll
        for (int n = 0; n < 8; ++n) acc[m][n] = 0.f;

    // prologue: DEPTH steps in flight (steps past the end re-fetch a valid address, unused)
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) issue(d, d);

    for (int it0 = 0; it0 < iters; it0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int it = it0 + d;
            // the 3 loads of step `it` are the oldest outstanding ones
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * (DEPTH - 1)) : "memory");
            const char* slot = ring + d * SLOT_BYTES;
            const u32x4 b0 = *(const u32x4*)(slot + lane * 16);
            const u32x4 b1 = *(const u32x4*)(slot + 1024 + lane * 16);
            const u32x4 a_lo = *(const u32x4*)(slot + 2048 + kp * 32);
            const u32x4 a_hi = *(const u32x4*)(slot + 2048 + kp * 32 + 16);
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // slot is in registers: it may be refilled
            issue(it + DEPTH, d);
            const int pr = it * STEP + wave * NKP + kp;
            if (pr < npairs && it < iters && col_ok) {
                unsigned bp[8];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    bp[2 * j] = __builtin_amdgcn_perm(b1[j], b0[j], 0x05040100u);     // (B[k][n], B[k+1][n]), n even
                    bp[2 * j + 1] = __builtin_amdgcn_perm(b1[j], b0[j], 0x07060302u); // n odd
                }
#pragma unroll
                for (int m = 0; m < 8; ++m) {
                    const unsigned amv = m < 4 ? a_lo[m & 3] : a_hi[m & 3];
#pragma unroll
                    for (int n = 0; n < 8; ++n) acc[m][n] = dot2<BF16>(amv, bp[n], acc[m][n]);
                }
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // drain the look-ahead fills before the LDS is reused

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

    // ---- reduce over waves through LDS (reuses the rings) ----
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
        s = apply_prologue<float>(s, p.prologue, p.prologue_arg, [&]() { return load_out(p.C, p.out_type, idx); });
        store_out(p.C, p.out_type, idx, apply_epilogue<float>(s, p.epilogue, p.epilogue_arg));
    };

    if (p.splits == 1) {
#pragma unroll
        for (int j = 0; j < VPL; ++j) finish((j + VPL * kp) >> 3, (j + VPL * kp) & 7, v[j]);
        return;
    }

    // ---- K split over workgroups: partial sums to scratch, last arrival finishes ----
    // The partial sums are written as agent-scope relaxed atomics (written through to the
    // level of the memory system that all XCDs share), so no cache-wide write-back is
    // needed: the stores only have to be acknowledged (vmcnt = 0) before this workgroup
    // takes its ticket.
    float* part = p.scratch + ((int64_t)blockIdx.y * nblocks + bx) * (64 * LPR);
#pragma unroll
    for (int j = 0; j < VPL; ++j) __hip_atomic_store(part + j * 64 + lane, v[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    unsigned ticket = 0;
    if (lane == 0) ticket = __hip_atomic_fetch_add(p.counters + bx, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ticket = __shfl(ticket, 0, 64);
    if (ticket != (unsigned)p.splits - 1) return;
    // last arrival: drop any stale copies of the scratch lines from this XCD's caches, then
    // read all slices with ordinary pipelined loads and add them in split order
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    float sum[VPL];
#pragma unroll
    for (int j = 0; j < VPL; ++j) sum[j] = 0.f;
    for (int sp = 0; sp < p.splits; ++sp) {
        const float* src = p.scratch + ((int64_t)sp * nblocks + bx) * (64 * LPR) + lane;
#pragma unroll
        for (int j = 0; j < VPL; ++j) sum[j] += src[j * 64];
    }
#pragma unroll
    for (int j = 0; j < VPL; ++j) finish((j + VPL * kp) >> 3, (j + VPL * kp) & 7, sum[j]);
    if (lane == 0) p.counters[bx] = 0; // ready for the next launch
}

template <bool BF16, int LPR, int WAVES, int DEPTH>
hipError_t launch_one(const SkinnyArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    constexpr int CB = LPR * 8;
    auto kern = gemm_skinny_kernel<BF16, LPR, WAVES, DEPTH>;
    unsigned lds = WAVES * DEPTH * (2048 + 256);
    const unsigned red = (WAVES - 1) * LPR * 64 * 4;
    if (lds < red) lds = red;
    dim3 grid(((a.N + CB - 1) / CB + 7) / 8 * 8, a.splits, a.batch > 1 ? a.batch : 1), block(WAVES * 64, 1, 1);
    if (geom) {
        geom->grid[0] = grid.x; geom->grid[1] = grid.y; geom->grid[2] = grid.z;
        geom->block[0] = block.x; geom->block[1] = geom->block[2] = 1;
        geom->dyn_lds = lds;
    }
    if (dry_run) return hipSuccess;
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    // (the LDS need grows with M and the ring depth, never past the instantiation's largest: ask for that once)
    static LdsLimitOnce lds_limit;
    if (lds > 64 * 1024)
        if (hipError_t e = lds_limit.ensure((const void*)kern, 160 * 1024); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, grid, block, lds, stream, ACC950_SKINNY_HEAD_OF(a), a);
    return hipGetLastError();
}

#define SV(LPR, W, D) { LPR * 8, W, D, false, 8, 2, 64 * LPR, &launch_one<false, LPR, W, D>, &launch_one<true, LPR, W, D> }
const SkinnyVariant kSkinny[] = { SV(8, 4, 8), SV(8, 8, 4), SV(16, 4, 8), SV(32, 4, 8) };
#undef SV

} // namespace

const SkinnyVariant* skinny_dot2_table(int* count)
{
    *count = (int)(sizeof(kSkinny) / sizeof(kSkinny[0]));
    return kSkinny;
}

int skinny_num_variants()
{
    int a, b;
    skinny_mfma_table(&a);
    skinny_dot2_table(&b);
    return a + b;
}
const SkinnyVariant& skinny_variant(int v)
{
    int a, b;
    const SkinnyVariant* m = skinny_mfma_table(&a);
    const SkinnyVariant* d = skinny_dot2_table(&b);
    return v < a ? m[v] : d[v - a];
}
void skinny_variant_info(int v, int* lpr, int* waves, int* depth)
{
    const SkinnyVariant& s = skinny_variant(v);
    *lpr = s.cols / 8;
    *waves = s.waves;
    *depth = s.depth;
}
int skinny_column_blocks(int v, int N) { return (N + skinny_variant(v).cols - 1) / skinny_variant(v).cols; }
size_t skinny_scratch_floats(int v, int N, int splits)
{
    return splits <= 1 ? 0 : (size_t)splits * skinny_column_blocks(v, N) * skinny_variant(v).block_floats;
}

hipError_t launch_skinny(int v, const SkinnyArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    if (v < 0 || v >= skinny_num_variants()) return hipErrorInvalidValue;
    const SkinnyVariant& s = skinny_variant(v);
    if (a.in_type == T_I8) return s.i8 ? s.i8(a, stream, geom, dry_run) : hipErrorInvalidValue;
    return a.in_type == T_BF16 ? s.bf16(a, stream, geom, dry_run) : s.f16(a, stream, geom, dry_run);
}

} // namespace acc950
