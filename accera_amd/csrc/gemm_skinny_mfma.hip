// Bandwidth-bound "skinny" GEMM on the matrix cores: up to 32 rows of A against a large
// row-major B (K x N, N contiguous), fp32 accumulate, fused epilogue.
//
// The kernel is a pure stream over B, like the packed-dot-product kernel in
// gemm_skinny.hip, but the multiply-accumulates run on MFMA so that the vector ALU does
// (almost) nothing per byte: the transposed product C^T = B^T * A^T is computed, with a
// 32-column slice of B as the 32-row MFMA operand and A^T (rows of A beyond M are zero)
// as the 32-column operand.  B arrives row-major (k rows); ds_read_b64_tr_b16 transposes
// it on the way out of LDS into the K-contiguous layout the MFMA wants.
//
// Reference counterpart: the non-tensorized thread-bound plan is all the reference can
// emit for M below its smallest MMA shape (/root/reference/accera/python/accera/test/mfma_tests.py:250-278,309-356).
//
// Work split
//   * grid.x = blocks of CB = 64 or 256 columns, grid.y = K splits; inside a workgroup the
//     k steps are dealt round-robin to the waves.
//   * a wave step is 16 k rows x CB columns of B (2 or 8 KB, fetched by 1 KB fill
//     instructions that cover 8 rows x 128 B or 2 rows x 512 B) plus the matching 32 x 16
//     piece of A (1 KB, rows >= M stay zero).
//   * every wave owns a ring of DEPTH slots in LDS, filled by global_load_lds, DEPTH steps
//     in flight, no barrier while streaming.  Fills stop at the end of the wave's K range:
//     the last DEPTH steps are consumed with a shrinking s_waitcnt instead of prefetching
//     past the end.
//   * per step and 32 columns: 2 transposing LDS reads and 1 MFMA 32x32x16.
//   * tail: accumulators go to LDS in [row of A][column] order, every thread sums float4
//     groups over the waves and stores 4 adjacent outputs at once.
//   * K split: the workgroup's partial goes to the scratch buffer and the last workgroup to
//     arrive (ticket) adds the slices in split order with all its threads, applies the
//     epilogue and stores.  Each trip through memory (publish + acknowledge, ticket,
//     slice loads, final stores) costs about 1.7 us on this chip, so a split only pays
//     when the column blocks alone cannot occupy the CUs.  (Unequal splits, where one
//     workgroup per block ends later and finds everything published, were measured and
//     do not pay: a single CU streams at most ~40 GB/s through global_load_lds, so the
//     late workgroups cannot use the bandwidth the early ones leave.)
//   * 256-column blocks make every fill fetch whole 512-byte pieces of B rows.  With
//     64-column blocks and a row stride that is a multiple of 512 bytes, the blocks whose
//     128-byte lines have address bits 8:7 = 11 stream about 25 % slower than the others
//     (measured, cause unknown); the wide form has no such stragglers but needs a K split
//     to occupy the chip unless N is large.
#include "common.h"
#include "skinny.h"
#include <type_traits>

namespace acc950 {

namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// IN: T_F16, T_BF16 (16 k rows per step, v_mfma_f32_32x32x16) or T_I8 (32 k rows per step, v_mfma_i32_32x32x32_i8, sums
// that wrap around like the reference's int32 accumulator: /root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:342-360).
// A step has the same bytes either way: a 64-column block of int8 is 32 k rows x 64 bytes where fp16 has 16 x 128.
template <int IN, int CB, int WAVES, int DEPTH>
__global__ void __launch_bounds__(WAVES * 64) gemm_skinny_mfma_kernel(ACC950_SKINNY_HEAD_PARAMS, SkinnyArgs p)
{
    ACC950_SKINNY_TAKE_HEAD(p);
    static_assert(CB == 64 || CB == 256, "column block of 64 or 256");
    constexpr bool I8 = IN == T_I8, BF16 = IN == T_BF16;
    constexpr int ES = I8 ? 1 : 2;                // bytes per input element
    constexpr int KS = 32 / ES;                   // k rows per step (32 bytes of K per row of A)
    constexpr int RB = CB * ES;                   // bytes of one B row piece
    using sum_t = std::conditional_t<I8, int, float>;
    typedef sum_t sum4 __attribute__((ext_vector_type(4)));
    typedef sum_t sum16 __attribute__((ext_vector_type(16)));
    constexpr int CPR = RB / 16;                  // 16-byte chunks per row piece
    constexpr int RPF = 64 / CPR;                 // rows per fill instruction (1 KB)
    constexpr int BFILLS = KS / RPF;              // B fills per step
    constexpr int JB = CB / 32;                   // 32-column MFMA blocks
    constexpr int B_BYTES = KS * RB;
    constexpr int SLOT_BYTES = B_BYTES + 1024;    // + A: 32 rows x 32 B
    constexpr int RING_BYTES = DEPTH * SLOT_BYTES;
    constexpr int LOADS = BFILLS + 1;             // fills per step
    constexpr int NT = WAVES * 64;
    static_assert(LOADS * (DEPTH - 1) < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    if (blockIdx.z != 0) { // batched launch: blockIdx.z picks the problem (and its slice of the K-split workspace); problem 0 waits for none of these fields
        const int64_t z = blockIdx.z;
        p.A = (const char*)p.A + z * p.a_bs * ES;
        p.B = (const char*)p.B + z * p.b_bs * ES;
        p.C = (char*)p.C + z * p.c_bs * elem_bytes(p.out_type);
        p.scratch += z * p.scratch_bs;
        p.counters += z * p.counter_bs;
    }

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroup ids are dealt round-robin to the 8 XCDs; column block = (id % 8) * per + id / 8
    // gives every XCD a contiguous range of blocks (its L2 then sees whole stretches of each
    // B row instead of every 8th block).  With extra_phase >= 0 the blocks of that phase
    // (the slow-streaming ones, see the file comment) are each shared by two workgroups.
    const int nblocks = (p.N + CB - 1) / CB;
    const int regular = (nblocks + 7) & ~7; // ids below this are dealt to blocks, the rest are second halves
    int bx, split_idx = blockIdx.y, nsplit = p.splits;
    if ((int)blockIdx.x < regular) {
        bx = (blockIdx.x & 7) * (regular >> 3) + (blockIdx.x >> 3);
        if (bx >= nblocks) return;
        if (p.extra_phase >= 0 && (bx & 3) == p.extra_phase) nsplit = 2;
    } else {
        bx = p.extra_phase + 4 * ((int)blockIdx.x - regular);
        if (bx >= nblocks) return;
        split_idx = 1;
        nsplit = 2;
    }
    const int col_base = bx * CB;

    const int steps_total = p.K / KS;
    const int steps_per_split = (steps_total + nsplit - 1) / nsplit;
    const int s_begin = split_idx * steps_per_split;
    const int nsteps = max(min(s_begin + steps_per_split, steps_total) - s_begin, 0);
    const int my_steps = nsteps > wave ? (nsteps - wave + WAVES - 1) / WAVES : 0; // steps wave, wave + WAVES, ...

    char* ring = smem + wave * RING_BYTES;
    const unsigned ring_addr = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(ACC950_LDS char*)ring);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) *(u32x4*)(ring + d * SLOT_BYTES + B_BYTES + lane * 16) = u32x4{0, 0, 0, 0};
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");

    // B fill number f puts rows f*RPF .. of the step at the same LDS rows (RB bytes each):
    // lane l lands at row f*RPF + l/CPR, chunk position l%CPR, and fetches the logical chunk
    // position ^ swz(row): the k rows of one transposing read go to different banks (16-bit: four rows of 128 bytes and
    // more, x 2*(row%4); 8-bit: eight rows, of which rows j and j+4 of a 64-byte pitch share their banks, x 2*(row/4%2)).
    auto swz = [](int row) { return I8 && CB == 64 ? ((row >> 2) & 1) << 1 : I8 ? (row & 7) << 1 : (row & 3) << 1; };
    const int64_t row_bytes = p.b_rs * ES;
    const int fh = lane / CPR, fpos = lane % CPR;
    unsigned boff[BFILLS];
#pragma unroll
    for (int f = 0; f < BFILLS; ++f) {
        const int row = RPF * f + fh;
        const int col = col_base + ((fpos ^ swz(row)) << 4) / ES;
        boff[f] = (unsigned)((int64_t)row * row_bytes + (int64_t)(col < p.N ? col : 0) * ES); // outside N: any valid address
    }
    const int am = lane >> 1;
    const bool a_active = am < p.M;
    // the two 16-byte halves of a row swap places in rows 8-15 and 24-31, so that the 16 lanes of one
    // read phase (32-byte row pitch) spread over all banks
    const unsigned aoff = (unsigned)((int64_t)(a_active ? am : 0) * p.a_rs * ES + ((lane & 1) ^ ((am >> 3) & 1)) * 16);

    auto issue = [&](int it, int slot) { // it < my_steps
        const int s = s_begin + wave + it * WAVES;
        const char* bsrc = (const char*)p.B + (int64_t)s * KS * row_bytes;
        const char* asrc = (const char*)p.A + (int64_t)s * KS * ES;
        const unsigned dst = ring_addr + slot * SLOT_BYTES;
#pragma unroll
        for (int f = 0; f < BFILLS; f += 2)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t"
                         "s_mov_b32 m0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %4, %2"
                         :
                         : "s"(dst + f * 1024), "v"(boff[f]), "s"(bsrc), "s"(dst + (f + 1) * 1024), "v"(boff[f + 1])
                         : "memory");
        if (a_active) // lanes 0 .. 2M-1; every wave issues it (M >= 1), so vmcnt counts LOADS per step
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(dst + B_BYTES), "v"(aoff), "s"(asrc) : "memory");
    };

    // read offsets inside a slot
    const int h = lane >> 5, g = (lane >> 4) & 1, i16 = lane & 15;
    unsigned roff[JB][2];
#pragma unroll
    for (int j = 0; j < JB; ++j)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            if constexpr (I8) {
                // ds_read_b64_tr_b8: lanes 2j, 2j+1 of a group of 16 point at k row j (2 x 8 bytes = 16 columns), lane i gets column i of those 8 rows
                const int k = h * 16 + q * 8 + (i16 >> 1);
                const int chunk = j * 2 + g;
                roff[j][q] = (unsigned)(k * RB + ((chunk ^ swz(k)) << 4) + (i16 & 1) * 8);
            } else {
                const int k = h * 8 + q * 4 + (i16 >> 2);
                const int chunk = j * 4 + g * 2 + ((i16 & 3) >> 1);
                roff[j][q] = (unsigned)(k * RB + ((chunk ^ swz(k)) << 4) + (i16 & 1) * 8);
            }
        }
    const unsigned aread = B_BYTES + (lane & 31) * 32 + (h ^ (((lane & 31) >> 3) & 1)) * 16;

    sum16 acc[JB];
#pragma unroll
    for (int j = 0; j < JB; ++j) acc[j] = sum16{};

    auto consume = [&](int slot_idx, auto refill) {
        const char* slot = ring + slot_idx * SLOT_BYTES;
        i32x4 bfrag[JB];
#pragma unroll
        for (int j = 0; j < JB; ++j)
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                i32x2 w;
                if constexpr (I8) w = __builtin_amdgcn_ds_read_tr8_b64_v2i32((ACC950_LDS i32x2*)(slot + roff[j][q]));
                else w = __builtin_bit_cast(i32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((ACC950_LDS s16x4*)(slot + roff[j][q])));
                bfrag[j][q * 2] = w[0];
                bfrag[j][q * 2 + 1] = w[1];
            }
        const i32x4 afrag = *(const i32x4*)(slot + aread);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // slot is in registers: it may be refilled
        refill();
#pragma unroll
        for (int j = 0; j < JB; ++j) {
            if constexpr (I8)
                acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bfrag[j], afrag, acc[j], 0, 0, 0);
            else if constexpr (BF16)
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, bfrag[j]), __builtin_bit_cast(bf16x8, afrag), acc[j], 0, 0, 0);
            else
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, bfrag[j]), __builtin_bit_cast(f16x8, afrag), acc[j], 0, 0, 0);
        }
    };

    // prologue: up to DEPTH steps in flight
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
        if (d < my_steps) issue(d, d);
    int it = 0, head = 0;
    // steady state: step it + DEPTH exists and takes over the slot that step it leaves
    for (; it + DEPTH < my_steps; ++it) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS * (DEPTH - 1)) : "memory");
        consume(head, [&]() { issue(it + DEPTH, head); });
        head = head + 1 == DEPTH ? 0 : head + 1;
    }
    // drain: my_steps - it (<= DEPTH) steps are outstanding, nothing left to fetch
    const int rem = my_steps - it;
#pragma unroll
    for (int r = DEPTH - 1; r >= 0; --r)
        if (r < rem) {
            asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS * r) : "memory");
            consume(head, [&]() {});
            head = head + 1 == DEPTH ? 0 : head + 1;
        }

    // ---- tail ----
    // accumulator layout (C^T block j): register r of lane l = column j*32 + (r/4)*8 + (l/32)*4 + r%4,
    // row l%32 of A.  Reorder through LDS to [row][256 columns].
    __syncthreads(); // every wave is done with its ring
    sum_t* red = (sum_t*)smem; // [wave][M][CB]
    const int m = lane & 31;
    if (m < p.M) {
        sum_t* mine = red + ((size_t)wave * p.M + m) * CB + h * 4;
#pragma unroll
        for (int j = 0; j < JB; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *(sum4*)(mine + j * 32 + q * 8) = sum4{acc[j][q * 4], acc[j][q * 4 + 1], acc[j][q * 4 + 2], acc[j][q * 4 + 3]};
    }
    __syncthreads();

    const int groups = p.M * (CB / 4); // groups of four sums of the workgroup's block
    // four adjacent columns of one row: one 4-, 8- or 16-byte store when C allows it
    const int os = elem_bytes(p.out_type);
    const bool vec_ok = p.prologue == PRO_SET && p.c_rs % 4 == 0 && ((size_t)p.C & (size_t)(4 * os - 1)) == 0;
    auto finish4 = [&](int grp, sum4 s) {
        const int row = grp / (CB / 4), n = col_base + (grp % (CB / 4)) * 4;
        if (n >= p.N) return; // N is a multiple of 8: a group is entirely inside or outside
        const int64_t idx = (int64_t)row * p.c_rs + n;
        if (vec_ok) {
            sum_t r[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = apply_epilogue<sum_t>(wrap_add(s[e], (sum_t)p.prologue_arg), p.epilogue, p.epilogue_arg);
            if constexpr (I8) {
                if (p.out_type == T_I32) *(i32x4*)((int*)p.C + idx) = i32x4{r[0], r[1], r[2], r[3]};
                else if (p.out_type == T_I16)
                    *(i32x2*)((int16_t*)p.C + idx) = i32x2{(int)(((unsigned)r[0] & 0xffffu) | ((unsigned)r[1] << 16)), (int)(((unsigned)r[2] & 0xffffu) | ((unsigned)r[3] << 16))};
                else
                    *(unsigned*)((int8_t*)p.C + idx) = ((unsigned)r[0] & 0xffu) | (((unsigned)r[1] & 0xffu) << 8) | (((unsigned)r[2] & 0xffu) << 16) | ((unsigned)r[3] << 24);
            } else if (p.out_type == T_F32) {
                *(f32x4*)((float*)p.C + idx) = f32x4{r[0], r[1], r[2], r[3]};
            } else if (p.out_type == T_F16) {
                typedef _Float16 h4 __attribute__((ext_vector_type(4)));
                *(h4*)((uint16_t*)p.C + idx) = h4{(_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3]};
            } else {
                typedef __bf16 b4 __attribute__((ext_vector_type(4)));
                *(b4*)((uint16_t*)p.C + idx) = b4{(__bf16)r[0], (__bf16)r[1], (__bf16)r[2], (__bf16)r[3]};
            }
            return;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (I8) {
                const int v = apply_prologue<int>(s[e], p.prologue, p.prologue_arg, [&]() { return load_out_int(p.C, p.out_type, idx + e); });
                store_out_int(p.C, p.out_type, idx + e, apply_epilogue<int>(v, p.epilogue, p.epilogue_arg));
            } else {
                const float v = apply_prologue<float>(s[e], p.prologue, p.prologue_arg, [&]() { return load_out(p.C, p.out_type, idx + e); });
                store_out(p.C, p.out_type, idx + e, apply_epilogue<float>(v, p.epilogue, p.epilogue_arg));
            }
        }
    };

    if (nsplit == 1) {
        for (int grp = tid; grp < groups; grp += NT) {
            sum4 s = *(const sum4*)(red + (size_t)grp * 4);
            for (int w = 1; w < WAVES; ++w) s += *(const sum4*)(red + (size_t)w * p.M * CB + (size_t)grp * 4);
            finish4(grp, s);
        }
        return;
    }

    // ---- K split ----
    // The partial goes out as agent-scope relaxed atomic stores (written through to the level
    // all XCDs share) and only has to be acknowledged (vmcnt = 0) before the ticket is taken.
    sum_t* part = (sum_t*)p.scratch + ((int64_t)split_idx * nblocks + bx) * (32 * CB);
    for (int grp = tid; grp < groups; grp += NT) {
        sum4 s = *(const sum4*)(red + (size_t)grp * 4);
        for (int w = 1; w < WAVES; ++w) s += *(const sum4*)(red + (size_t)w * p.M * CB + (size_t)grp * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) __hip_atomic_store(part + grp * 4 + e, s[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads(); // all partial stores of the workgroup are acknowledged; the slabs are free again
    unsigned* ticket_slot = (unsigned*)smem;
    if (tid == 0) *ticket_slot = __hip_atomic_fetch_add(p.counters + bx, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*ticket_slot != (unsigned)nsplit - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); // drop stale copies of the scratch lines from this XCD's caches
    const int64_t slice = (int64_t)nblocks * (32 * CB);
    for (int grp = tid; grp < groups; grp += NT) {
        // loads of 8 slices are issued together (one memory latency per batch); the adds stay in split order
        const sum_t* src = (const sum_t*)p.scratch + (int64_t)bx * (32 * CB) + (size_t)grp * 4;
        sum4 s = {0, 0, 0, 0};
        for (int sp0 = 0; sp0 < nsplit; sp0 += 8) {
            sum4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = sp0 + u < nsplit ? *(const sum4*)(src + (sp0 + u) * slice) : sum4{0, 0, 0, 0};
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (sp0 + u < nsplit) s += v[u];
        }
        finish4(grp, s);
    }
    if (tid == 0) p.counters[bx] = 0; // ready for the next launch
}

template <int IN, int CB, int WAVES, int DEPTH>
hipError_t launch_one(const SkinnyArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    auto kern = gemm_skinny_mfma_kernel<IN, CB, WAVES, DEPTH>;
    unsigned lds = WAVES * DEPTH * (32 * CB + 1024); // (a step's piece of B is 32 bytes of K for every column, whatever the type)
    const unsigned red = WAVES * a.M * CB * 4; // [wave][row of A][column] floats of the tail
    if (lds < red) lds = red;
    const int nblocks = (a.N + CB - 1) / CB;
    const int extra = a.extra_phase >= 0 && a.splits == 1 ? (nblocks - a.extra_phase + 3) / 4 : 0;
    dim3 grid((nblocks + 7) / 8 * 8 + extra, a.splits, a.batch > 1 ? a.batch : 1), block(WAVES * 64, 1, 1);
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

// narrow (64 columns, no K split needed from 128 blocks up) first, then wide
#define SM(CB, W, D) { CB, W, D, true, 32, 16, 32 * CB, &launch_one<T_F16, CB, W, D>, &launch_one<T_BF16, CB, W, D>, &launch_one<T_I8, CB, W, D> }
const SkinnyVariant kSkinnyMfma[] = { SM(64, 4, 4), SM(64, 4, 8), SM(64, 2, 8), SM(64, 8, 4), SM(256, 4, 4), SM(256, 2, 4) };
#undef SM

} // namespace

const SkinnyVariant* skinny_mfma_table(int* count)
{
    *count = (int)(sizeof(kSkinnyMfma) / sizeof(kSkinnyMfma[0]));
    return kSkinnyMfma;
}

} // namespace acc950
