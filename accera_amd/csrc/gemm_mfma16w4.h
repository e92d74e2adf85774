// Four-wave MFMA GEMM on the 16x16 instruction shapes: one wave per SIMD, each with a 128x128
// piece of a 256x256 output tile (or 128x96 of a 256x192 one).
//
// Counterpart of the same tensorized plan of the reference as gemm_mfma16.h
// (/root/reference/accera/transforms/src/exec/ExecutionPlanToAffineLoweringPass.cpp:5986-6533),
// with the largest wave tile the register file takes.  A 128x128 wave tile reads 16 fragments
// from LDS per 64 MFMAs; the eight-wave kernel's 128x64 wave tile reads 12 per 32.  LDS traffic
// per unit of arithmetic drops by a third, and on a part that runs large GEMMs at its power
// limit that is clock rate for the matrix cores.
//
// The 256 accumulator registers live in a[0:255] and the K loop is hand-laid assembly
// (gemm_mfma16w4_loop.inc, written by gen_w4_loop.py) -- left to the compiler the same loop
// moves accumulators between the register files and spills.  Tile staging, the LDS layout and
// the stores are those of gemm_mfma16.h.
//
// Takes: A row-major (or column-major, with 256-wide tiles: staged as it lies in memory and
// read with the transposing LDS loads, like a row-major B), any M >= 256 and any 16-byte-aligned N >= the tile width
// (the last row / column of tiles overlaps the one before), K a multiple of one k-step (64 bytes)
// and at least four of them, rows of C 16 bytes aligned;
// every prologue / epilogue op (an int8 C is only written, never read): C = A*B starts from zeros, C += A*B with a
// 32-bit C loads the tile of C straight into the accumulator registers, everything else (a 16-bit C, beta * C,
// a SET constant) is written into them by ordinary code before the loop.
#pragma once
#include "gemm_mfma16.h"
#include "gemm_mfma16w4_loop.inc"

namespace acc950 {

// BN: 256, or 192 (K-contiguous B only; N = 3072 = 16 x 192 gives one tile per CU) with 128x96 wave tiles
// PERSIST: one workgroup per CU walks several output tiles (grid = min(tiles, CUs)); the closing k-steps of a tile
// fetch the first K tiles of the next one, and that tile's loop starts while this tile's stores are still on their way.
template <int IN_, bool B_KC_, bool TIMED_ = false, int BN_ = 256, bool PERSIST_ = false, bool A_KC_ = true>
struct Mfma16W4Config {
    static constexpr bool TIMED = TIMED_, PERSIST = PERSIST_;
    static_assert(!PERSIST_ || BN_ == 256, "the 192-wide tile is for problems of one tile per CU");
    static constexpr int IN = IN_, BM = 256, BN = BN_, WAVES_M = 2, WAVES_N = 2, KB = 64, STAGES = 4, NT = 256;
    static constexpr bool A_KC = A_KC_, B_KC = B_KC_;
    static_assert(A_KC_ || BN_ == 256, "column-major A: 256-wide tiles");
    // (a workgroup that walks several tiles stages its write-back behind the last LDS stage while the others already receive
    // the next tile: it asks for the whole LDS of the CU)
    static constexpr int LDS_BYTES = PERSIST_ ? 160 * 1024 : STAGES * (BM + BN) * KB;
    static_assert(BN == 256 || (BN == 192 && B_KC), "tile widths the loop is written for");
};

// accumulator blocks N and N+1 (eight registers) out of the AGPR file.  The moves go through the matrix
// pipeline and take a while to land; eight in a row, and a whole row of blocks before the first use,
// keep that latency out of the write-back's critical path.
struct W4BlockPair { i32x4 a, b; };
template <int N>
__device__ __forceinline__ W4BlockPair w4_acc_pair()
{
    int x0, x1, x2, x3, y0, y1, y2, y3;
    asm volatile("v_accvgpr_read_b32 %0, a[%8]\n\tv_accvgpr_read_b32 %1, a[%9]\n\tv_accvgpr_read_b32 %2, a[%10]\n\tv_accvgpr_read_b32 %3, a[%11]\n\t"
                 "v_accvgpr_read_b32 %4, a[%12]\n\tv_accvgpr_read_b32 %5, a[%13]\n\tv_accvgpr_read_b32 %6, a[%14]\n\tv_accvgpr_read_b32 %7, a[%15]"
                 : "=v"(x0), "=v"(x1), "=v"(x2), "=v"(x3), "=v"(y0), "=v"(y1), "=v"(y2), "=v"(y3)
                 : "n"(N * 4), "n"(N * 4 + 1), "n"(N * 4 + 2), "n"(N * 4 + 3), "n"(N * 4 + 4), "n"(N * 4 + 5), "n"(N * 4 + 6), "n"(N * 4 + 7));
    return W4BlockPair{i32x4{x0, x1, x2, x3}, i32x4{y0, y1, y2, y3}};
}

template <int B, int E, typename F>
__device__ __forceinline__ void w4_static_for(F&& f)
{
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        w4_static_for<B + 1, E>(f);
    }
}

template <typename Cfg>
__global__ void __launch_bounds__(256, 1) gemm_mfma16w4_kernel(ACC950_HEAD_PARAMS, GemmArgs p)
{
    constexpr int IN = Cfg::IN, BM = 256, BN = Cfg::BN, NT = 256, KB = 64, WAVES_N = 2;
    constexpr bool A_KC = Cfg::A_KC, B_KC = Cfg::B_KC;
    constexpr int ES = InTraits<IN>::ES;
    constexpr int BK = KB / ES;
    constexpr int WTM = 128, WTN = BN / 2, TM = 8, TN = WTN / 16;
    constexpr int FILLS_B = BN * KB / (NT * 16), FILLS = 4 + FILLS_B; // fill instructions per thread and K tile
    // (swizzle and address arithmetic only: these are the tiles of the eight-wave kernel)
    using TA = OperandTile<IN, BM, A_KC, 512, KB, true>;
    using TB = OperandTile<IN, BN, B_KC, 512, KB, true>;
    using acc_t = typename In16Traits<IN>::acc_t;
    using scalar_t = typename In16Traits<IN>::scalar_t;
    constexpr int STAGE_BYTES = TA::TILE_BYTES + TB::TILE_BYTES;
    static_assert(STAGE_BYTES == 16384 + TN * 2048 && TA::TILE_BYTES == 16384, "the loop's offsets are written for these");

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    ACC950_TAKE_HEAD_TILES(p, BM, BN);
    select_batch(p);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wr0 = (wave / WAVES_N) * WTM;
    const int wc0 = (wave % WAVES_N) * WTN;

    unsigned long long stamp_clk[4], stamp_ref[4];
    auto stamp = [&](int i) {
        if constexpr (Cfg::TIMED) {
            __builtin_amdgcn_sched_barrier(0);
            stamp_clk[i] = __builtin_amdgcn_s_memtime();
            stamp_ref[i] = __builtin_amdgcn_s_memrealtime();
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    stamp(0);

    // M and N need not be multiples of the tile: the last row / column of tiles ends at M / N and overlaps its
    // neighbour (the host allows this only for N whose last tile still starts on a 16-byte boundary of B's and C's
    // rows).  What both compute gets the same bits from both; when C is read, the moved tile leaves the rows and
    // columns it shares with its neighbour to the neighbour (see the write-back), so that no element is added to twice.
    auto tile_origin = [&](int id, int& r0, int& c0) __attribute__((always_inline)) {
        int tile_m, tile_n;
        tile_coords(id, p.tiles_m, p.tiles_n, tile_m, tile_n);
        r0 = tile_m * BM + BM <= p.M ? tile_m * BM : p.M - BM;
        c0 = tile_n * BN + BN <= p.N ? tile_n * BN : p.N - BN;
    };
    // (a workgroup that walks several tiles takes ids blockIdx.x, blockIdx.x + gridDim.x, ...: in every round the
    // workgroups of one XCD -- ids equal modulo 8 -- work on one compact rectangle of tiles, as when every tile has its own workgroup)
    const int total_tiles = p.tiles_m * p.tiles_n;
    if constexpr (Cfg::PERSIST) {
        // Tiles take equal time, so workgroups that start together reach every write-back together, and all of C's
        // bytes of a round then queue at the memory at once while the matrix cores wait.  Groups of workgroups (taken
        // across the XCDs: ids / 8) start a little apart instead; the offsets last for the whole launch, and one
        // group's stores drain while the others compute.  (A bounded wait on the constant 100 MHz counter.)
        const unsigned grp = p.stagger_groups > 1 ? (blockIdx.x >> 3) % (unsigned)p.stagger_groups : 0u;
        if (grp) {
            const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
            const unsigned long long wait = (unsigned long long)grp * (unsigned)p.stagger_ticks;
            while (__builtin_amdgcn_s_memrealtime() - t0 < wait) __builtin_amdgcn_s_sleep(16);
        }
    }
    int tile_id = blockIdx.x;
    int m0, n0;
    tile_origin(tile_id, m0, n0);

    const char* Ab = (const char*)p.A;
    const char* Bb = (const char*)p.B;
    const int64_t lda = A_KC ? p.a_rs : p.a_cs;
    const int64_t ldb = B_KC ? p.b_cs : p.b_rs;
    const int KT = p.K / BK;

    // ---- tile fills: 4 + 4 instructions per thread and K tile.  A (and a K-contiguous B): one
    // instruction of the workgroup covers 64 rows.  B with N contiguous: 8 (16-bit) or 16 (8-bit)
    // k rows, half a period of the swizzle, so even and odd instructions have their own lane offset.
    const unsigned smem_addr = (unsigned)(size_t)(ACC950_LDS char*)smem;
    const unsigned ldsb = __builtin_amdgcn_readfirstlane(smem_addr + (unsigned)(wave * 1024));
    constexpr int B_CPR = TB::CPR;
    constexpr int B_RPP = NT / B_CPR; // rows of B's tile one fill instruction of the workgroup covers
    // K-contiguous tiles (64-byte rows): chunk c of row r sits at position c ^ kc_swz(r).  With this map
    // the 16-row ds_read_b128 of a fragment is free of bank conflicts (the row/4 map of the eight-wave
    // kernel costs two passes; there the sibling wave's MFMAs hide it, here nothing does).
    auto kc_swz = [](int row) { return ((row >> 1) & 1) | ((((row >> 1) ^ (row >> 2)) & 1) << 1); };
    constexpr int A_CPR = TA::CPR;
    constexpr int A_RPP = NT / A_CPR;
    unsigned a_off, a_off1;
    if constexpr (A_KC) {
        a_off = a_off1 = (unsigned)TA::global_off(tid / 4, (tid % 4) ^ kc_swz(tid / 4), 0, 0, lda);
    } else {
        a_off = (unsigned)TA::global_off(tid / A_CPR, TA::swizzle(tid / A_CPR, tid % A_CPR), 0, 0, lda);
        a_off1 = (unsigned)TA::global_off(tid / A_CPR, TA::swizzle(tid / A_CPR + A_RPP, tid % A_CPR), 0, 0, lda);
    }
    unsigned b_off0, b_off1;
    if constexpr (B_KC) {
        b_off0 = b_off1 = (unsigned)TB::global_off(tid / 4, (tid % 4) ^ kc_swz(tid / 4), 0, 0, ldb);
    } else {
        b_off0 = (unsigned)TB::global_off(tid / B_CPR, TB::swizzle(tid / B_CPR, tid % B_CPR), 0, 0, ldb);
        b_off1 = (unsigned)TB::global_off(tid / B_CPR, TB::swizzle(tid / B_CPR + B_RPP, tid % B_CPR), 0, 0, ldb);
    }
    const unsigned da = __builtin_amdgcn_readfirstlane((unsigned)((A_KC ? 64 : A_RPP) * lda * ES));
    const unsigned db = __builtin_amdgcn_readfirstlane((unsigned)((B_KC ? 64 : B_RPP) * ldb * ES));
    const unsigned sa = __builtin_amdgcn_readfirstlane(A_KC ? (unsigned)KB : (unsigned)(BK * lda * ES));
    const unsigned sb = __builtin_amdgcn_readfirstlane(B_KC ? (unsigned)KB : (unsigned)(BK * ldb * ES));
    auto a_panel = [&](int r0) __attribute__((always_inline)) { return Ab + (A_KC ? (int64_t)r0 * lda * ES : (int64_t)r0 * ES); };
    auto b_panel = [&](int c0) __attribute__((always_inline)) { return Bb + (B_KC ? (int64_t)c0 * ldb * ES : (int64_t)c0 * ES); };
    const char* a_tile = a_panel(m0);
    const char* b_tile = b_panel(n0);
    // The loop's last k-step runs at position 3 of its four-step pattern, so the first one starts at position
    // p0 = (4 - KT % 4) % 4: tile s goes to LDS stage (s + p0) % 4, and a partial first trip through the body
    // counts as one more trip.
    const unsigned p0 = __builtin_amdgcn_readfirstlane((unsigned)((4 - KT % 4) % 4));
    // With paired fills a K-contiguous B is fetched two K tiles at a time on the even positions of the loop's pattern
    // (both 64-byte halves of a cache line in neighbouring requests), so its third tile is issued here only when the
    // first k-step sits at an odd position; otherwise the loop's first step fetches tiles 2 and 3.
    constexpr bool B_PAIRED = A_KC && B_KC && (BN == 192 || IN == IN_I8); // measured: behind the plain scheme for 16-bit inputs on 256-wide tiles
    const unsigned b_tiles_here = B_PAIRED ? 2u + (p0 & 1u) : 3u;
    // the first three K tiles of an output tile, issued ahead of its loop
    // (always inline: the panel addresses are scalar-register operands of the fill instructions)
    auto first_fills = [&](const char* a_src, const char* b_src) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            const unsigned stage = ldsb + ((s + p0) & 3) * STAGE_BYTES;
#pragma unroll
            for (int f = 0; f < 4; ++f)
                TA::direct_issue_uniform(stage + f * 4096, (f & 1) ? a_off1 : a_off, a_src + (int64_t)s * sa + (int64_t)f * da);
            if ((unsigned)s < b_tiles_here) {
#pragma unroll
                for (int f = 0; f < FILLS_B; ++f)
                    TB::direct_issue_uniform(stage + TA::TILE_BYTES + f * 4096, (f & 1) ? b_off1 : b_off0, b_src + (int64_t)s * sb + (int64_t)f * db);
            }
        }
    };
    first_fills(a_tile, b_tile);
    const unsigned groups = __builtin_amdgcn_readfirstlane((unsigned)(KT / 4 - 1 + (KT % 4 ? 1 : 0)));

    // ---- LDS addresses of the fragment reads (stage 0; the loop adds stage and block offsets)
    const int kg = lane >> 4, li = lane & 15;
    // (a column-major A: the address of the wave's first block of rows; the loop derives the other seven from it, which
    // differ in the bits of the block number only -- the swizzle is an XOR and every k row of the tile starts on a multiple of its length)
    unsigned a_rd;
    if constexpr (A_KC) a_rd = smem_addr + (unsigned)((wr0 + li) * 64 + (kg ^ kc_swz(li)) * 16);
    else if constexpr (ES == 2) {
        const int col_byte = (wr0 + (li & 3) * 4) * 2, k = kg * 8 + (li >> 2);
        a_rd = smem_addr + (unsigned)(k * TA::ROW_BYTES + TA::swizzle(k, col_byte >> 4) * 16 + (col_byte & 15));
    } else {
        const int col_byte = wr0 + (li & 1) * 8, k = kg * 16 + (li >> 1);
        a_rd = smem_addr + (unsigned)(k * TA::ROW_BYTES + TA::swizzle(k, col_byte >> 4) * 16 + (col_byte & 15));
    }
    unsigned b_rd[8];
    if constexpr (B_KC) {
#pragma unroll
        for (int x = 0; x < 8; ++x) b_rd[x] = smem_addr + (unsigned)((wc0 + li) * 64 + (kg ^ kc_swz(li)) * 16);
    } else if constexpr (ES == 2) {
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            const int col_byte = (wc0 + x * 16 + (li & 3) * 4) * 2, k = kg * 8 + (li >> 2);
            b_rd[x] = smem_addr + (unsigned)(k * TB::ROW_BYTES + TB::swizzle(k, col_byte >> 4) * 16 + (col_byte & 15));
        }
    } else {
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            const int col_byte = wc0 + x * 16 + (li & 1) * 8, k = kg * 16 + (li >> 1);
            b_rd[x] = smem_addr + (unsigned)(k * TB::ROW_BYTES + TB::swizzle(k, col_byte >> 4) * 16 + (col_byte & 15));
        }
    }

    // C += A*B: the loop starts from the tile of C instead of zeros (the host sends nothing else with a prologue
    // other than SET 0 here).  A 32-bit C is loaded by the loop's preamble:  Lane l owns row i*16 + l%16, columns j*16 + (l/16)*4 .. +3 of block (i, j).
    // How the accumulators start: 0 zeros (SET 0: C = A*B), 1 the loop's preamble loads a 32-bit C into them (C += A*B),
    // 2 the code below sets them up (a 16-bit C, beta * C, or a SET constant) and the loop leaves them as they are.
    const bool c_is_32bit = p.out_type == T_F32 || p.out_type == T_I32;
    const unsigned accum = __builtin_amdgcn_readfirstlane(
        p.prologue == PRO_SET ? (p.prologue_arg == 0.f ? 0u : 2u) : (p.prologue == PRO_NONE && c_is_32bit) ? 1u : 2u);
    const unsigned c_off = (unsigned)(wr0 + (lane & 15)) * ((unsigned)p.c_rs * 4) + (unsigned)(wc0 + (lane >> 4) * 4) * 4;
    const unsigned c_row16 = __builtin_amdgcn_readfirstlane((unsigned)p.c_rs * 64);
    const unsigned os = p.out_type == T_I8 ? 1 : (p.out_type == T_F32 || p.out_type == T_I32) ? 4 : 2;
    // The closing k-steps of a tile can fetch for the next one when its K tile s belongs in LDS stage s (entry at
    // position 0) and the loop has such closing steps (not the paired-fill loops).
    constexpr bool TAIL_PREFETCH = Cfg::PERSIST && !B_PAIRED;
    bool came_prefetched = false; // this tile's first three K tiles were issued by the previous tile's closing steps (before its stores)

    // ---- one output tile per trip (a single trip unless the workgroup walks several tiles)
    for (;;) {
    const int next_id = tile_id + (int)gridDim.x;
    const bool has_next = Cfg::PERSIST && next_id < total_tiles;
    int m0_next = m0, n0_next = n0;
    if (has_next) tile_origin(next_id, m0_next, n0_next);
    const char* pa_n = a_panel(m0_next);
    const char* pb_n = b_panel(n0_next);
    const char* pa_n_u = nullptr;
    const char* pb_n_u = nullptr;
    const bool prefetch_next = TAIL_PREFETCH && has_next && p0 == 0;
    // bit 0: the closing steps fetch the next tile's K tiles 0..2; bit 1: the first k-steps allow for the previous tile's
    // stores (64 per thread with a 32-bit C) between this tile's fills
    const unsigned flags = __builtin_amdgcn_readfirstlane((prefetch_next ? 1u : 0u) | (came_prefetched && os == 4 && groups >= 1 ? 2u : 0u));
    // (lane 0's copy of each address, explicitly: they are scalar-register operands of the loop, and with scalar registers
    // short around it the compiler may keep a value that is the same in every lane in vector registers)
    auto uniform_ptr = [](const char* q) __attribute__((always_inline)) {
        const unsigned long long a = (unsigned long long)q;
        const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
        return (const char*)(((unsigned long long)hi << 32) | lo);
    };
    const char* pa = uniform_ptr(a_tile + 3 * (int64_t)sa);
    const char* pb = uniform_ptr(b_tile + (int64_t)b_tiles_here * sb);
    pa_n_u = uniform_ptr(pa_n);
    pb_n_u = uniform_ptr(pb_n);
    const CTile c_in = c_tile(p, m0, n0, 4);
    const auto c_rsrc = c_in.rsrc;

    if (accum == 2) {
        // The lane's four elements of every block are written into the accumulator registers here: the SET constant,
        // or C widened (16-bit types) and scaled (SCALE prologue; x 1 is exact otherwise).
        // (All fills are waited for first: the compiler counts only its own loads when it places the waits.)
        auto put = [](auto n_tag, int x0, int x1, int x2, int x3) {
            constexpr int n = decltype(n_tag)::value;
            asm volatile("v_accvgpr_write_b32 a[%4], %0\n\tv_accvgpr_write_b32 a[%5], %1\n\tv_accvgpr_write_b32 a[%6], %2\n\tv_accvgpr_write_b32 a[%7], %3"
                         :
                         : "v"(x0), "v"(x1), "v"(x2), "v"(x3), "n"(n), "n"(n + 1), "n"(n + 2), "n"(n + 3));
        };
        const scalar_t c_mul = p.prologue == PRO_SCALE ? (scalar_t)p.prologue_arg : scalar_t(1);
        auto scaled = [&](scalar_t c) -> int {
            if constexpr (IN == IN_I8) return wrap_mul(c, c_mul);
            else return (int)__float_as_uint(c * c_mul);
        };
        if (p.prologue == PRO_SET) {
            const scalar_t set_v = (scalar_t)p.prologue_arg;
            int x;
            if constexpr (IN == IN_I8) x = set_v;
            else x = (int)__float_as_uint(set_v);
            w4_static_for<0, TM * TN>([&](auto b) { put(std::integral_constant<int, b.value * 4>{}, x, x, x, x); });
        } else if (c_is_32bit) {
            wait_vmcnt<0>();
            // four rows of blocks at a time: their loads are all in flight before the first is used
            w4_static_for<0, TM / 4>([&](auto q) {
                u32x4 w[4][TN];
#pragma unroll
                for (int ii = 0; ii < 4; ++ii)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        w[ii][j] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(c_rsrc, c_off + j * 64,
                                                                                                 (unsigned)((q.value * 4 + ii) * 16) * ((unsigned)p.c_rs * 4), 0));
                w4_static_for<0, 4>([&](auto ii) {
                    w4_static_for<0, TN>([&](auto j) {
                        int x[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const unsigned bits = w[ii.value][j.value][e]; // (a bit cast applied to the element expression itself reads element 0)
                            x[e] = scaled(__builtin_bit_cast(scalar_t, bits));
                        }
                        put(std::integral_constant<int, ((q.value * 4 + ii.value) * TN + j.value) * 4>{}, x[0], x[1], x[2], x[3]);
                    });
                });
            });
        } else {
            wait_vmcnt<0>();
            const CTile c16 = c_tile(p, m0, n0, 2);
            const unsigned rb = (unsigned)p.c_rs * 2;
            const unsigned off16 = (unsigned)(wr0 + (lane & 15)) * rb + (unsigned)(wc0 + (lane >> 4) * 4) * 2;
            const unsigned m_f16 = p.out_type == T_F16 ? ~0u : 0u, m_bf16 = p.out_type == T_BF16 ? ~0u : 0u;
            typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
            w4_static_for<0, TM / 4>([&](auto q) {
                u32x2 w[4][TN];
#pragma unroll
                for (int ii = 0; ii < 4; ++ii)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        w[ii][j] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(c16.rsrc, off16 + j * 32,
                                                                                                 (unsigned)((q.value * 4 + ii) * 16) * rb, 0));
                w4_static_for<0, 4>([&](auto ii) {
                    w4_static_for<0, TN>([&](auto j) {
                        const unsigned w0 = w[ii.value][j.value][0], w1 = w[ii.value][j.value][1];
                        int x[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const unsigned half = (((e & 2) ? w1 : w0) >> ((e & 1) * 16)) & 0xffffu;
                            if constexpr (IN == IN_I8) x[e] = scaled((int)(short)half); // int16 widens with its sign
                            else {
                                const unsigned short h = (unsigned short)half;
                                const unsigned as_f16 = __float_as_uint((float)__builtin_bit_cast(_Float16, h));
                                x[e] = scaled(__uint_as_float((as_f16 & m_f16) | ((half << 16) & m_bf16)));
                            }
                        }
                        put(std::integral_constant<int, ((q.value * 4 + ii.value) * TN + j.value) * 4>{}, x[0], x[1], x[2], x[3]);
                    });
                });
            });
        }
    }

    // K tile 0 has landed (tile 1 and tile 2 -- A's part of it at least -- may be in flight).  Memory operations complete in
    // the order issued, so after closing steps that fetched ahead the previous tile's stores (issued after these fills:
    // 64, 32 or 16 per thread for 4-, 2-, 1-byte elements of C) may be in flight as well.
    if (!came_prefetched) wait_vmcnt<B_PAIRED ? 4 + FILLS : 2 * FILLS>();
    else if (os == 4) wait_vmcnt<63>();
    else if (os == 2) wait_vmcnt<2 * FILLS + 32>();
    else wait_vmcnt<2 * FILLS + 16>();
    // (the bare instruction: a fence would make the compiler wait for the previous tile's stores here)
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    stamp(1);

#define ACC950_W4_OPERANDS                                                                                              \
    : [a_rd] "v"(a_rd), [b_rd0] "v"(b_rd[0]), [b_rd1] "v"(b_rd[1]), [b_rd2] "v"(b_rd[2]), [b_rd3] "v"(b_rd[3]),          \
      [b_rd4] "v"(b_rd[4]), [b_rd5] "v"(b_rd[5]), [b_rd6] "v"(b_rd[6]), [b_rd7] "v"(b_rd[7]), [a_off] "v"(a_off),        \
      [a_off1] "v"(a_off1),                                                                                               \
      [b_off0] "v"(b_off0), [b_off1] "v"(b_off1), [pa] "s"(pa), [pb] "s"(pb), [da] "s"(da), [db] "s"(db), [sa] "s"(sa),   \
      [sb] "s"(sb), [ldsb] "s"(ldsb), [groups] "s"(groups), [accum] "s"(accum), [c_off] "v"(c_off), [p0] "s"(p0),       \
      [c_rsrc] "s"(c_rsrc), [c_row16] "s"(c_row16), [pa_n] "s"(pa_n_u), [pb_n] "s"(pb_n_u), [flags] "s"(flags)               \
    : "memory", "scc", "s72", "s73", "s74", "s75", "s76", "s77", "s78", "s79", "s80", "s81", ACC950_W4_V(10), ACC950_W4_V(11), \
      ACC950_W4_V(12), ACC950_W4_V(13), ACC950_W4_V(14), ACC950_W4_V(15), ACC950_W4_V(16), ACC950_W4_V(17),             \
      ACC950_W4_V(18), ACC950_W4_V(19), ACC950_W4_V(20), ACC950_W4_V(21), ACC950_W4_V(22), ACC950_W4_V(23),             \
      ACC950_W4_V(24), "v250", "v251", "v252", "v253", "v254", "v255", "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7",   \
      "a8", "a9", ACC950_W4_A(1), ACC950_W4_A(2), ACC950_W4_A(3), ACC950_W4_A(4), ACC950_W4_A(5), ACC950_W4_A(6), ACC950_W4_A(7), ACC950_W4_A(8), ACC950_W4_A(9),   \
      ACC950_W4_A(10), ACC950_W4_A(11), ACC950_W4_A(12), ACC950_W4_A(13), ACC950_W4_A(14), ACC950_W4_A(15),             \
      ACC950_W4_A(16), ACC950_W4_A(17), ACC950_W4_A(18), ACC950_W4_A(19), ACC950_W4_A(20), ACC950_W4_A(21),             \
      ACC950_W4_A(22), ACC950_W4_A(23), ACC950_W4_A(24), "a250", "a251", "a252", "a253", "a254", "a255"
// ten registers of a file, by decade
#define ACC950_W4_R(f, d) f #d "0", f #d "1", f #d "2", f #d "3", f #d "4", f #d "5", f #d "6", f #d "7", f #d "8", f #d "9"
#define ACC950_W4_V(d) ACC950_W4_R("v", d)
#define ACC950_W4_A(d) ACC950_W4_R("a", d)
    if constexpr (!A_KC && TAIL_PREFETCH) {
        if constexpr (IN == IN_I8) {
            if constexpr (B_KC) asm volatile(ACC950_W4_LOOP_KC_AMC8_P("v_mfma_i32_16x16x64_i8") : ACC950_W4_OPERANDS);
            else asm volatile(ACC950_W4_LOOP_MC8_AMC8_P("v_mfma_i32_16x16x64_i8") : ACC950_W4_OPERANDS);
        } else if constexpr (B_KC) {
            if constexpr (IN == IN_F16) asm volatile(ACC950_W4_LOOP_KC_AMC16_P("v_mfma_f32_16x16x32_f16") : ACC950_W4_OPERANDS);
            else asm volatile(ACC950_W4_LOOP_KC_AMC16_P("v_mfma_f32_16x16x32_bf16") : ACC950_W4_OPERANDS);
        } else {
            if constexpr (IN == IN_F16) asm volatile(ACC950_W4_LOOP_MC16_AMC16_P("v_mfma_f32_16x16x32_f16") : ACC950_W4_OPERANDS);
            else asm volatile(ACC950_W4_LOOP_MC16_AMC16_P("v_mfma_f32_16x16x32_bf16") : ACC950_W4_OPERANDS);
        }
    } else if constexpr (!A_KC) {
        if constexpr (IN == IN_I8) {
            if constexpr (B_KC) asm volatile(ACC950_W4_LOOP_KC_AMC8("v_mfma_i32_16x16x64_i8") : ACC950_W4_OPERANDS);
            else asm volatile(ACC950_W4_LOOP_MC8_AMC8("v_mfma_i32_16x16x64_i8") : ACC950_W4_OPERANDS);
        } else if constexpr (B_KC) {
            if constexpr (IN == IN_F16) asm volatile(ACC950_W4_LOOP_KC_AMC16("v_mfma_f32_16x16x32_f16") : ACC950_W4_OPERANDS);
            else asm volatile(ACC950_W4_LOOP_KC_AMC16("v_mfma_f32_16x16x32_bf16") : ACC950_W4_OPERANDS);
        } else {
            if constexpr (IN == IN_F16) asm volatile(ACC950_W4_LOOP_MC16_AMC16("v_mfma_f32_16x16x32_f16") : ACC950_W4_OPERANDS);
            else asm volatile(ACC950_W4_LOOP_MC16_AMC16("v_mfma_f32_16x16x32_bf16") : ACC950_W4_OPERANDS);
        }
    } else if constexpr (B_KC && BN == 192) {
        if constexpr (IN == IN_F16) asm volatile(ACC950_W4_LOOP_KCP6("v_mfma_f32_16x16x32_f16") : ACC950_W4_OPERANDS);
        else if constexpr (IN == IN_BF16) asm volatile(ACC950_W4_LOOP_KCP6("v_mfma_f32_16x16x32_bf16") : ACC950_W4_OPERANDS);
        else asm volatile(ACC950_W4_LOOP_KCP6("v_mfma_i32_16x16x64_i8") : ACC950_W4_OPERANDS);
    } else if constexpr (TAIL_PREFETCH && B_KC) {
        if constexpr (IN == IN_F16) asm volatile(ACC950_W4_LOOP_KC_P("v_mfma_f32_16x16x32_f16") : ACC950_W4_OPERANDS);
        else asm volatile(ACC950_W4_LOOP_KC_P("v_mfma_f32_16x16x32_bf16") : ACC950_W4_OPERANDS);
    } else if constexpr (TAIL_PREFETCH) {
        if constexpr (IN == IN_F16) asm volatile(ACC950_W4_LOOP_MC16_P("v_mfma_f32_16x16x32_f16") : ACC950_W4_OPERANDS);
        else if constexpr (IN == IN_BF16) asm volatile(ACC950_W4_LOOP_MC16_P("v_mfma_f32_16x16x32_bf16") : ACC950_W4_OPERANDS);
        else asm volatile(ACC950_W4_LOOP_MC8_P("v_mfma_i32_16x16x64_i8") : ACC950_W4_OPERANDS);
    } else if constexpr (B_KC) {
        if constexpr (IN == IN_F16) asm volatile(ACC950_W4_LOOP_KC("v_mfma_f32_16x16x32_f16") : ACC950_W4_OPERANDS);
        else if constexpr (IN == IN_BF16) asm volatile(ACC950_W4_LOOP_KC("v_mfma_f32_16x16x32_bf16") : ACC950_W4_OPERANDS);
        else asm volatile(ACC950_W4_LOOP_KCP("v_mfma_i32_16x16x64_i8") : ACC950_W4_OPERANDS);
    } else {
        if constexpr (IN == IN_F16) asm volatile(ACC950_W4_LOOP_MC16("v_mfma_f32_16x16x32_f16") : ACC950_W4_OPERANDS);
        else if constexpr (IN == IN_BF16) asm volatile(ACC950_W4_LOOP_MC16("v_mfma_f32_16x16x32_bf16") : ACC950_W4_OPERANDS);
        else asm volatile(ACC950_W4_LOOP_MC8("v_mfma_i32_16x16x64_i8") : ACC950_W4_OPERANDS);
    }
    stamp(2);
#undef ACC950_W4_OPERANDS
#undef ACC950_W4_R
#undef ACC950_W4_V
#undef ACC950_W4_A

    // ---- write-back: block (i, j) leaves the AGPR file just before its store.  Lane l holds row
    // i*16 + l%16 and columns j*16 + (l/16)*4 .. +3 of the wave tile.
    // (In a workgroup that walks several tiles the write-back's addresses do not change from tile to tile; computed from
    // an opaque copy of the lane id they are recomputed per tile instead of being kept in registers across the K loop,
    // where only v0-v99 are free.)
    int lane_wb = lane, wave_wb = wave;
    if constexpr (Cfg::PERSIST) asm volatile("" : "+v"(lane_wb), "+v"(wave_wb));
    const int wave_u = __builtin_amdgcn_readfirstlane(wave_wb);
    // One copy of the stores per epilogue (a uniform branch).
    // (epi_tag: 0 nothing, 1 ReLU, 2 the other epilogue ops, applied element by element from the call's arguments)
    auto write_back = [&](auto epi_tag) __attribute__((always_inline)) {
        constexpr int EPI = decltype(epi_tag)::value;
        constexpr bool RELU = EPI == 1;
        // the epilogue on four finished sums
        auto finish = [&](acc_t v) __attribute__((always_inline)) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if constexpr (RELU) {
                    if constexpr (IN == IN_I8) v[e] = v[e] > 0 ? v[e] : 0;
                    else v[e] = __builtin_fmaxf(v[e], 0.f);
                } else if constexpr (EPI == 2) {
                    v[e] = apply_epilogue<scalar_t>(v[e], p.epilogue, p.epilogue_arg);
                }
            }
            return v;
        };
        {
            // 16 rows of the wave tile (one row of blocks) go from the accumulator registers into a wave-private slab of the
            // (now idle) tile buffers as they are -- LDS stores take their data from the accumulator file directly, which
            // saves the 256 register-file moves per wave that every other way out needs -- and come back as whole stretches of
            // a row: 4 / 8 / 16 neighbouring sums per lane, which get the epilogue, are narrowed to the output type and leave
            // as one 16-byte store.  A store instruction that writes 2 rows x 512 bytes (or whole rows of a narrow type)
            // passes through a CU's memory pipeline more than twice as fast as one that writes the accumulator layout's
            // 16 rows x 64 bytes (measured: 256 KB per CU in 2.4-2.9 us against 6.2-7.0 us).
            __syncthreads();
            // (the lambdas of the write-back are always inlined: left as functions they would take the kernel's state by
            // reference through memory, and everything they capture -- tile origin, descriptors, the call's arguments -- would
            // live in scratch and come back in vector registers)
            auto staged = [&](auto os_tag, auto&& pack) __attribute__((always_inline)) {
                constexpr int OS = decltype(os_tag)::value;
                // Non-temporal stores: C is written once and not read again by this launch.  Measured with the `nt` bit: int8
                // 8192^3 4 % faster, fp16 4096^3 0.8 % (`sc1` alone changes nothing); the K loops that run while other
                // workgroups write back stall less (MFMA pipe busy 0.91 -> 0.95 of the loop's cycles on int8 8192^3), while the
                // L2 hit counts of the panel fetches stay as they were.
                constexpr int AUX = 2;
                constexpr int RAW_ROW = WTN * 4;      // a row of the wave tile as 32-bit sums
                // 16 bytes past a row: the 16 row starts are an odd number of 4-bank steps apart
                constexpr int PITCH = RAW_ROW + 16;
                static_assert(RAW_ROW % 32 == 0, "(RAW_ROW / 16 + 1) must be odd for the 16 row starts to differ mod 64 banks");
                // (a workgroup that walks several tiles keeps the slabs behind stage 2: stage 3 is the stage of the last k-step,
                // the others may already be receiving the next tile)
                static_assert((Cfg::PERSIST ? 3 * STAGE_BYTES : 0) + 4 * 16 * PITCH <= Cfg::LDS_BYTES, "four slabs fit (behind the first three stages)");
                const unsigned slab_off = (Cfg::PERSIST ? 3 * STAGE_BYTES : 0) + wave_u * (16 * PITCH);
                const char* slab = smem + slab_off;
                const unsigned mine = smem_addr + slab_off + (unsigned)((lane_wb & 15) * PITCH + (lane_wb >> 4) * 16);
                const CTile tile = c_tile(p, m0 + (wave_u / WAVES_N) * WTM, n0 + (wave_u % WAVES_N) * WTN, OS);
                const unsigned row_bytes = (unsigned)p.c_rs * OS;
                // A tile that was moved up / left to end at M / N, of a problem that reads C: its first rows / columns belong
                // to the neighbouring tile, which may or may not have written them yet -- they are not stored from here.
                // (first row / column of the wave tile this workgroup owns; 0 wherever nothing is shared)
                int own_row = 0, own_col = 0;
                if (p.prologue != PRO_SET) {
                    int tm, tn;
                    tile_coords(tile_id, p.tiles_m, p.tiles_n, tm, tn);
                    own_row = tm * BM - m0 - (wave_u / WAVES_N) * WTM;
                    own_col = tn * BN - n0 - (wave_u % WAVES_N) * WTN;
                }
                constexpr int VPL = 16 / OS;                 // sums per lane and store
                constexpr int GPR = WTN / VPL;               // 16-byte pieces of the output per row of the wave tile
                constexpr int PIECES = (16 * GPR + 63) / 64; // stores per lane and row of blocks
                w4_static_for<0, TM>([&](auto i) {
                    w4_static_for<0, TN>([&](auto j) {
                        constexpr int n = (i.value * TN + j.value) * 4;
                        const unsigned at = mine; // (asm operands do not capture on their own)
                        asm volatile("ds_write_b128 %0, a[%1:%2] offset:%3" : : "v"(at), "n"(n), "n"(n + 3), "n"(j.value * 64) : "memory");
                    });
#pragma unroll
                    for (int it = 0; it < PIECES; ++it) {
                        const int id = it * 64 + lane_wb;
                        if ((16 * GPR) % 64 != 0 && id >= 16 * GPR) break;
                        const int r = id / GPR, g = id % GPR;
                        acc_t v[VPL / 4];
#pragma unroll
                        for (int q = 0; q < VPL / 4; ++q) v[q] = finish(*(const acc_t*)(slab + r * PITCH + g * (VPL * 4) + q * 16));
                        if (i.value * 16 + r >= own_row && g * VPL >= own_col)
                            __builtin_amdgcn_raw_buffer_store_b128(pack(v), tile.rsrc, (unsigned)r * row_bytes + g * 16,
                                                                   (unsigned)(i.value * 16) * row_bytes, AUX);
                    }
                });
            };
            typedef _Float16 h8 __attribute__((ext_vector_type(8)));
            typedef __bf16 b8 __attribute__((ext_vector_type(8)));
            auto pack_f16 = [](const acc_t (&v)[2]) -> u32x4 {
                return __builtin_bit_cast(u32x4, h8{(_Float16)v[0][0], (_Float16)v[0][1], (_Float16)v[0][2], (_Float16)v[0][3],
                                                    (_Float16)v[1][0], (_Float16)v[1][1], (_Float16)v[1][2], (_Float16)v[1][3]});
            };
            auto pack_bf16 = [](const acc_t (&v)[2]) -> u32x4 {
                return __builtin_bit_cast(u32x4, b8{(__bf16)v[0][0], (__bf16)v[0][1], (__bf16)v[0][2], (__bf16)v[0][3],
                                                    (__bf16)v[1][0], (__bf16)v[1][1], (__bf16)v[1][2], (__bf16)v[1][3]});
            };
            auto pack_i16 = [](const acc_t (&v)[2]) -> u32x4 {
                u32x4 w;
#pragma unroll
                for (int q = 0; q < 2; ++q)
#pragma unroll
                    for (int h = 0; h < 2; ++h) w[q * 2 + h] = ((unsigned)v[q][2 * h] & 0xffffu) | ((unsigned)v[q][2 * h + 1] << 16);
                return w;
            };
            auto pack_i8 = [](const acc_t (&v)[4]) -> u32x4 {
                u32x4 w;
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    w[q] = ((unsigned)v[q][0] & 0xffu) | (((unsigned)v[q][1] & 0xffu) << 8) | (((unsigned)v[q][2] & 0xffu) << 16) | ((unsigned)v[q][3] << 24);
                return w;
            };
            auto pack_32 = [](const acc_t (&v)[1]) -> u32x4 { return __builtin_bit_cast(u32x4, v[0]); };
            if (os == 4) staged(std::integral_constant<int, 4>{}, pack_32);
            else if constexpr (IN == IN_I8) {
                if (os == 2) staged(std::integral_constant<int, 2>{}, pack_i16);
                else staged(std::integral_constant<int, 1>{}, pack_i8);
            } else {
                if (p.out_type == T_F16) staged(std::integral_constant<int, 2>{}, pack_f16);
                else staged(std::integral_constant<int, 2>{}, pack_bf16);
            }
        }
    };
    if (p.epilogue == EPI_RELU) write_back(std::integral_constant<int, 1>{});
    else if (p.epilogue == EPI_NONE) write_back(std::integral_constant<int, 0>{});
    else write_back(std::integral_constant<int, 2>{});

    if constexpr (Cfg::TIMED) {
        // four stamps per output tile: start (the first tile's includes its fills), loop entered, loop left, stores
        // issued -- acknowledged too when the workgroup has one tile; one that walks on does not wait for them
        if constexpr (!Cfg::PERSIST) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        stamp(3);
        if (threadIdx.x == 0 && p.stamps) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                p.stamps[(tile_id * 4 + i) * 2] = stamp_clk[i];
                p.stamps[(tile_id * 4 + i) * 2 + 1] = stamp_ref[i];
            }
        }
        stamp(0);
    }
    if constexpr (!Cfg::PERSIST) break;
    if (tile_id + (int)gridDim.x >= total_tiles) break;
    came_prefetched = TAIL_PREFETCH && p0 == 0; // (what this trip's closing steps did, as there is a next tile)
    tile_id += (int)gridDim.x;
    tile_origin(tile_id, m0, n0); // (computed again rather than carried across the loop and the write-back in scalar registers)
    a_tile = a_panel(m0);
    b_tile = b_panel(n0);
    if (!came_prefetched) {
        __syncthreads(); // every wave has read its last fragments (stage 3) and is done with its slab
        first_fills(a_tile, b_tile);
    }
    } // tiles

}

template <typename Cfg>
hipError_t launch_mfma16w4(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    auto kern = gemm_mfma16w4_kernel<Cfg>;
    // an int8 C is written in 16-byte pieces of 16-byte aligned rows; no kernel here has a path for anything else
    if (a.out_type == T_I8 && (a.c_rs % 16 || ((size_t)a.C & 15) || (a.batch > 1 && a.c_bs % 16))) return hipErrorInvalidValue;
    GemmArgs args = a;
    args.tiles_m = (a.M + Cfg::BM - 1) / Cfg::BM;
    args.tiles_n = (a.N + Cfg::BN - 1) / Cfg::BN;
    // one workgroup per tile, or one per CU that walks the tiles id, id + grid, ... (the LDS of a CU holds one workgroup)
    unsigned grid_x = (unsigned)(args.tiles_m * args.tiles_n);
    if (Cfg::PERSIST && grid_x > (unsigned)kComputeUnits) grid_x = kComputeUnits;
    args.stagger_groups = args.stagger_ticks = 0;
    if (Cfg::PERSIST && args.tiles_m * args.tiles_n > kComputeUnits) {
        // measured on int8 8192^3 (four rounds): four groups 1.5 us apart gain 2 %; eight groups, or more than about
        // 10 us in all, lose several per cent (workgroups of an XCD then no longer share their panels in its L2)
        args.stagger_groups = 4;
        args.stagger_ticks = 150;
    }
    if (geom) {
        geom->grid[0] = grid_x;
        geom->grid[1] = 1;
        geom->grid[2] = a.batch > 1 ? a.batch : 1;
        geom->block[0] = Cfg::NT;
        geom->block[1] = geom->block[2] = 1;
        geom->dyn_lds = Cfg::LDS_BYTES;
    }
    if (dry_run) return hipSuccess;
    static LdsLimitOnce lds_limit; // per instantiation
    if (hipError_t e = lds_limit.ensure((const void*)kern, Cfg::LDS_BYTES); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(grid_x, 1, a.batch > 1 ? a.batch : 1), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, ACC950_HEAD_OF(args), args);
    return hipGetLastError();
}

} // namespace acc950
