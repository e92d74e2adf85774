// Ping-pong MFMA GEMM on the 16x16 instruction shapes of gfx950:
// v_mfma_f32_16x16x32_{f16,bf16} and v_mfma_i32_16x16x64_i8.
//
// Same tiling, staging and schedule as the 8-wave ping-pong form of gemm_mfma.h (the
// replacement for the reference's tensorized plan,
// /root/reference/accera/transforms/src/exec/ExecutionPlanToAffineLoweringPass.cpp:5986-6533);
// what differs is the matrix instruction.  One 16x16 instruction sums 64 bytes of K per output
// element before it touches the accumulator, twice the run of the 32x32 shapes, and the matrix
// cores draw measurably less power for the same arithmetic: with random operands and nothing
// but MFMAs in flight the part sustains about 12 % more throughput on this shape.  Large
// GEMMs run at the power limit, so that difference carries over.
//
// The operands are passed swapped (matrix B's fragment as the instruction's first operand), so
// a lane ends up with one row and four neighbouring columns of C per 16x16 block: outputs leave
// as 16-byte (fp32 / int32), 8-byte (16-bit) or 4-byte (int8) pieces with no lane exchange.
#pragma once
#include "gemm_mfma.h"

namespace acc950 {

template <int IN> struct In16Traits { using acc_t = f32x4; using scalar_t = float; };
template <> struct In16Traits<IN_I8> { using acc_t = i32x4; using scalar_t = int; };

// c (16x16, lane: row l%16 of `rows`, columns (l/16)*4..+3 of `cols`) += rows x cols^T over one k-step
template <int IN>
__device__ __forceinline__ void mfma16(const i32x4& cols, const i32x4& rows, typename In16Traits<IN>::acc_t& c)
{
    if constexpr (IN == IN_F16)
        c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, cols), __builtin_bit_cast(f16x8, rows), c, 0, 0, 0);
    else if constexpr (IN == IN_BF16)
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, cols), __builtin_bit_cast(bf16x8, rows), c, 0, 0, 0);
    else
        c = __builtin_amdgcn_mfma_i32_16x16x64_i8(cols, rows, c, 0, 0, 0);
}

// GENERAL: the build that carries every prologue / epilogue op; the other build takes only C = A*B
// and C = relu(A*B) (SET 0 prologue) and is kept free of scratch use, which costs 4-20 us per dispatch.
template <int IN_, int BM_, int BN_, int WAVES_M_, int WAVES_N_, bool A_KC_, bool B_KC_, int KB_, int STAGES_, bool GENERAL_ = false, bool TIMED_ = false>
struct Mfma16Config {
    static constexpr bool TIMED = TIMED_, GENERAL = GENERAL_;
    static constexpr int IN = IN_, BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, KB = KB_, STAGES = STAGES_;
    static constexpr bool A_KC = A_KC_, B_KC = B_KC_;
    static constexpr int NT = WAVES_M * WAVES_N * 64;
    static constexpr int LDS_BYTES = STAGES * (BM + BN) * KB;
    static_assert(WAVES_M * WAVES_N == 8, "two waves per SIMD take turns");
    static_assert(STAGES >= 2 && STAGES <= 4, "2 to 4 LDS stages (a fifth, 160 KB in all, measured slower)");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
};

template <typename Cfg>
__global__ void __launch_bounds__(Cfg::NT, 1) gemm_mfma16_kernel(ACC950_HEAD_PARAMS, GemmArgs p)
{
    constexpr int IN = Cfg::IN, BM = Cfg::BM, BN = Cfg::BN, WAVES_M = Cfg::WAVES_M, WAVES_N = Cfg::WAVES_N;
    constexpr int KB = Cfg::KB, STAGES = Cfg::STAGES, NT = Cfg::NT;
    constexpr bool A_KC = Cfg::A_KC, B_KC = Cfg::B_KC;
    constexpr int ES = InTraits<IN>::ES;
    constexpr int BK = KB / ES;
    constexpr int KSTEPS = KB / 64;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 16, TN = WTN / 16;
    static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile is made of 16x16 MFMA blocks");
    using TA = OperandTile<IN, BM, A_KC, NT, KB, true>;
    using TB = OperandTile<IN, BN, B_KC, NT, KB, true>;
    using acc_t = typename In16Traits<IN>::acc_t;
    using scalar_t = typename In16Traits<IN>::scalar_t;
    constexpr int STAGE_BYTES = TA::TILE_BYTES + TB::TILE_BYTES;

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

    int tile_m, tile_n;
    tile_coords(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const char* Ab = (const char*)p.A;
    const char* Bb = (const char*)p.B;
    const int64_t lda = A_KC ? p.a_rs : p.a_cs; // KC: stride between rows; MC: stride between k
    const int64_t ldb = B_KC ? p.b_cs : p.b_rs;

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = acc_t{};

    const int KT = (p.K + BK - 1) / BK;

    // ---- tile fills, straight from global memory into LDS
    const unsigned smem_addr = (unsigned)(size_t)(ACC950_LDS char*)smem;
    const unsigned wave_lds = __builtin_amdgcn_readfirstlane((unsigned)(wave * 1024));
    const unsigned a_lane_off = TA::direct_lane_offset(lda, tid), b_lane_off = TB::direct_lane_offset(ldb, tid);
    constexpr int FILLS_A = TA::PER_THREAD, FILLS_B = TB::PER_THREAD, FILLS = FILLS_A + FILLS_B;
    auto fill_one = [&](auto tile_tag, int f, unsigned lds_tile, unsigned lane_off, const char* base, int r0, int k0, int64_t ld) {
        using T = decltype(tile_tag);
        unsigned pos = wave_lds + f * NT * 16; // byte position of this wave's 1 KB inside the tile (wave-uniform)
        const char* src = T::direct_base(base, f, r0, k0, ld);
        if constexpr (!T::EVEN_SPLIT) {
            if (pos >= (unsigned)T::TILE_BYTES) {
                pos -= T::TILE_BYTES;
                src -= T::wrap_bytes(ld);
            }
        }
        T::direct_issue(lds_tile + pos, lane_off, src);
    };
    auto issue_fill = [&](int f, int stage, int k0) {
        if (f < FILLS_A) fill_one(TA{}, f, smem_addr + stage * STAGE_BYTES, a_lane_off, Ab, m0, k0, lda);
        else fill_one(TB{}, f - FILLS_A, smem_addr + stage * STAGE_BYTES + TA::TILE_BYTES, b_lane_off, Bb, n0, k0, ldb);
    };

    // ---- main loop.  Every k-step (64 bytes of K) is a memory cluster (fragment reads, a share
    // of the fills of tile kt+D) and a compute cluster (its TM x TN MFMAs), each closed by a
    // barrier.  Waves 4..7 run one cluster behind waves 0..3, so on every SIMD one wave computes
    // while its sibling reads.
    constexpr int D = STAGES - 1;
    const int group = wave >> 2;
    auto raw_barrier = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
#pragma unroll
    for (int s = 0; s < D; ++s)
        if (s < KT) {
#pragma unroll
            for (int f = 0; f < FILLS; ++f) issue_fill(f, s, s * BK);
        }
    if (KT >= D) wait_vmcnt<(D - 1) * FILLS>();
    else wait_vmcnt<0>();
    __syncthreads();
    stamp(1);
    if (group == 1) raw_barrier(); // one cluster behind
    constexpr int FPC = (FILLS + KSTEPS - 1) / KSTEPS; // fills issued per cluster
    i32x4 af[TM], bf[TN];
    // order_tag: 0 = A's fills first, then B's; 1 / 2 = the K-contiguous operand's fills first / last (see the loop below)
    auto pp_tile = [&](int kt, auto fill_tag, auto order_tag) {
        constexpr bool fill = decltype(fill_tag)::value;
        constexpr int order = decltype(order_tag)::value;
        const char* sa = smem + (kt % STAGES) * STAGE_BYTES;
        const char* sb = sa + TA::TILE_BYTES;
#pragma unroll
        for (int c = 0; c < KSTEPS; ++c) {
            // ---- memory cluster
#pragma unroll
            for (int j = 0; j < TN; ++j) bf[j] = TB::read_frag16(sb, wc0 + j * 16, c, lane);
#pragma unroll
            for (int i = 0; i < TM; ++i) af[i] = TA::read_frag16(sa, wr0 + i * 16, c, lane);
            if constexpr (fill) {
                constexpr int FX = A_KC ? FILLS_A : FILLS_B, FY = FILLS - FX, X0 = A_KC ? 0 : FILLS_A, Y0 = A_KC ? FILLS_A : 0;
#pragma unroll
                for (int u = 0; u < FPC; ++u)
                    if (c * FPC + u < FILLS) {
                        const int n = c * FPC + u; // position in this tile's sequence of fills
                        const int f = order == 0 ? n : order == 1 ? (n < FX ? X0 + n : Y0 + (n - FX)) : (n < FY ? Y0 + n : X0 + (n - FY));
                        issue_fill(f, (kt + D) % STAGES, (kt + D) * BK);
                    }
            }
            if (c + 1 == KSTEPS) { // own fills of tile kt+1 have landed before the barrier publishes them
                if constexpr (fill) wait_vmcnt<(D - 1) * FILLS>();
                else wait_vmcnt<0>();
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // fragments are in registers: the buffer may be refilled
            raw_barrier();
            // ---- compute cluster
            __builtin_amdgcn_s_setprio(2);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) mfma16<IN>(bf[j], af[i], acc[i][j]);
            __builtin_amdgcn_s_setprio(0);
            raw_barrier();
        }
    };
    {
        int kt = 0;
        if constexpr (KSTEPS == 1 && (A_KC || B_KC) && IN != IN_I8) {
            // A 64-byte K tile of a K-contiguous operand is half a cache line per row, and the two halves of a line
            // belong to tiles 2m and 2m+1.  Two tiles per trip, so that the order of the fills is fixed at compile
            // time: the operand's fills go last for the even tile and first for the odd one, the halves are
            // requested back to back, and the second one is still in the CU's vector cache.  Measured +2 % on fp16
            // 4096^3; the int8 kernel ran 9 % slower with it (not understood) and keeps the plain order.
            constexpr int EVEN = ((0 + D) & 1) ? 1 : 2, ODD = ((1 + D) & 1) ? 1 : 2; // tile kt + D odd: its halves come second -> first in line
            for (; kt + D + 1 < KT; kt += 2) {
                pp_tile(kt, std::true_type{}, std::integral_constant<int, EVEN>{});
                pp_tile(kt + 1, std::true_type{}, std::integral_constant<int, ODD>{});
            }
        }
        for (; kt + D < KT; ++kt) pp_tile(kt, std::true_type{}, std::integral_constant<int, 0>{});
        for (; kt < KT; ++kt) pp_tile(kt, std::false_type{}, std::integral_constant<int, 0>{});
    }
    if (group == 0) raw_barrier(); // match the extra barrier of the other group

    stamp(2);
    // ---- write-back.  Two leaves, chosen once: the fused matmul + ReLU (SET 0 prologue: C is not
    // read, one max per element on the way out) and everything else (acc += (beta *) C, SET constant,
    // epilogue op, then the same stores).  No accumulator changes on one side of a branch and is
    // used after it, so the register allocator never has two versions of the tile to merge -- that
    // merging used to push a few registers into scratch, and a kernel that uses scratch at all
    // pays 4 us (256 workgroups) to 20 us (1024) more per dispatch on this device.
    // In block (i, j) lane l holds row i*16 + l%16 and columns j*16 + (l/16)*4 .. +3 of the wave tile.
    const int lrow = wr0 + (lane & 15), lcol = wc0 + (lane >> 4) * 4;
    const unsigned os = p.out_type == T_I8 ? 1 : (p.out_type == T_F32 || p.out_type == T_I32) ? 4 : 2;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    // the four values of a block narrowed to the output type, packed in column order
    auto pack_f16 = [](const acc_t& v) -> i32x2 {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        return __builtin_bit_cast(i32x2, h4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]}); // RNE
    };
    auto pack_bf16 = [](const acc_t& v) -> i32x2 {
        typedef __bf16 b4 __attribute__((ext_vector_type(4)));
        return __builtin_bit_cast(i32x2, b4{(__bf16)v[0], (__bf16)v[1], (__bf16)v[2], (__bf16)v[3]}); // RNE
    };
    auto pack_i16 = [](const acc_t& v) -> i32x2 { // low bits of the int32 sums
        return i32x2{(int)(((unsigned)v[0] & 0xffffu) | ((unsigned)v[1] << 16)), (int)(((unsigned)v[2] & 0xffffu) | ((unsigned)v[3] << 16))};
    };
    auto pack_i8 = [](const acc_t& v) -> int {
        return (int)(((unsigned)v[0] & 0xffu) | (((unsigned)v[1] & 0xffu) << 8) | (((unsigned)v[2] & 0xffu) << 16) | ((unsigned)v[3] << 24));
    };
    // pass C: fin(v) is the last elementwise step (ReLU in the fused leaf, identity otherwise)
    auto store_tile = [&](auto&& fin) {
        auto fin4 = [&](const acc_t& v) { return acc_t{fin(v[0]), fin(v[1]), fin(v[2]), fin(v[3])}; };
    if (os == 4) {
        // one 16-byte store per block and lane
        const CTile tile = c_tile(p, m0, n0, 4);
        const unsigned row_bytes = (unsigned)p.c_rs * 4;
        const unsigned lane_off = (unsigned)lrow * row_bytes + (unsigned)lcol * 4;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, fin4(acc[i][j])), tile.rsrc, lane_off + j * 64,
                                                       (unsigned)(i * 16) * row_bytes, C_STORE_AUX);
    } else if ((p.c_rs * os) % 16 == 0 && ((size_t)p.C & 15) == 0) {
        // narrow outputs: 16 rows of the wave tile are put together in a wave-private slab of the
        // (now idle) tile buffers and leave as 16-byte pieces that cover whole rows
        __syncthreads(); // every wave is done reading the tile buffers
        auto staged = [&](auto os_tag, auto&& pack) {
            constexpr int OS = decltype(os_tag)::value;
            constexpr int ROW = WTN * OS;
            constexpr int PITCH = (ROW / 32) % 2 == 0 ? ROW + 32 : ROW; // an odd number of 32-byte units: rows spread over the banks
            static_assert(NT / 64 * 16 * PITCH <= Cfg::LDS_BYTES, "slabs fit the tile buffers");
            char* slab = smem + wave_u * (16 * PITCH);
            const CTile tile = c_tile(p, m0 + (wave_u / WAVES_N) * WTM, n0 + (wave_u % WAVES_N) * WTN, OS);
            const unsigned row_bytes = (unsigned)p.c_rs * OS;
            constexpr int CPRW = ROW / 16;                    // 16-byte pieces per row of the wave tile
            constexpr int PIECES = (16 * CPRW + 63) / 64;     // per lane and 16-row slab
            char* mine = slab + (lane & 15) * PITCH + ((lane >> 4) * 4) * OS;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    auto w = pack(fin4(acc[i][j]));
                    *(decltype(w)*)(mine + j * 16 * OS) = w;
                }
#pragma unroll
                for (int it = 0; it < PIECES; ++it) {
                    const int id = it * 64 + lane;
                    if ((16 * CPRW) % 64 != 0 && id >= 16 * CPRW) break;
                    const int row = id / CPRW, cc = id % CPRW;
                    const i32x4 v = *(const i32x4*)(slab + row * PITCH + cc * 16);
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), tile.rsrc, (unsigned)row * row_bytes + cc * 16,
                                                           (unsigned)(i * 16) * row_bytes, C_STORE_AUX);
                }
            }
        };
        if constexpr (IN == IN_I8) {
            if (os == 2) staged(std::integral_constant<int, 2>{}, pack_i16);
            else staged(std::integral_constant<int, 1>{}, pack_i8);
        } else {
            if (p.out_type == T_F16) staged(std::integral_constant<int, 2>{}, pack_f16);
            else staged(std::integral_constant<int, 2>{}, pack_bf16);
        }
    } else {
        // rows of C that are not 16-byte aligned: single elements
        const CTile tile = c_tile(p, m0, n0, os);
        const unsigned row_bytes = (unsigned)p.c_rs * os;
        const unsigned lane_off = (unsigned)lrow * row_bytes + (unsigned)lcol * os;
        auto by_element = [&](auto os_tag, auto&& pack) {
            constexpr int OS = decltype(os_tag)::value;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const unsigned so = (unsigned)(i * 16) * row_bytes + (unsigned)(j * 16) * OS;
                    auto w = pack(fin4(acc[i][j]));
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        static_assert(OS == 2, "16-bit elements");
                        __builtin_amdgcn_raw_buffer_store_b16((unsigned short)((unsigned)w[e >> 1] >> ((e & 1) * 16)), tile.rsrc, lane_off + e * 2, so, 0);
                    }
                }
        };
        if constexpr (IN == IN_I8) {
            // int8 outputs with unaligned rows never get here: the host sends them to the thread-bound kernel
            if (os == 2) by_element(std::integral_constant<int, 2>{}, pack_i16);
        } else {
            if (p.out_type == T_F16) by_element(std::integral_constant<int, 2>{}, pack_f16);
            else by_element(std::integral_constant<int, 2>{}, pack_bf16);
        }
    }

    };

    if constexpr (!Cfg::GENERAL) {
        // the host sends only SET 0 + ReLU / no epilogue here
        if (p.epilogue == EPI_RELU) store_tile([](scalar_t v) { return v > scalar_t(0) ? v : scalar_t(0); });
        else store_tile([](scalar_t v) { return v; });
    } else {
        // pass A: the four elements of C a lane owns in a block arrive in one load -- 16 bytes (32-bit
        // elements), or the 12 / 8 bytes from the dword boundary below them (16- / 8-bit elements, rows
        // of C may start at any element), realigned with v_alignbyte.  The loads of a block sit behind
        // one uniform branch per element width; the arithmetic does not (c = 0 when C is not read).
        // The descriptor ends with the last row of C, so the few bytes a realigned load reads past its
        // elements are never fetched from beyond the matrix.
        const bool read_c = p.prologue != PRO_SET;
        const scalar_t c_mul = p.prologue == PRO_SCALE ? (scalar_t)p.prologue_arg : scalar_t(read_c ? 1 : 0); // x1 is exact
        const unsigned sh = (p.out_type == T_I32 || p.out_type == T_F32) ? 2 : (p.out_type == T_I8 ? 0 : 1);
        const unsigned m_f16 = p.out_type == T_F16 ? ~0u : 0u, m_bf16 = p.out_type == T_BF16 ? ~0u : 0u;
        char* tile_base = (char*)p.C + (((int64_t)m0 * p.c_rs + n0) << sh);
        const unsigned base_mis = (unsigned)(size_t)tile_base & 3u; // the descriptor starts at the dword that holds the tile's first element
        // (up to the end of the dword that holds the last element: the range check is per dword)
        const int64_t c_bytes_left = (((((int64_t)(p.M - 1 - m0)) * p.c_rs + (p.N - n0)) << sh) + base_mis + 3) & ~(int64_t)3;
        const CTile tile = CTile{__builtin_amdgcn_make_buffer_rsrc(tile_base - base_mis, 0, (int)(unsigned)(c_bytes_left < 0xffffffffll ? c_bytes_left : 0xffffffffll), 0x00020000)};
        const unsigned row_bytes = (unsigned)p.c_rs << sh;
        const unsigned lane_off = base_mis + (unsigned)lrow * row_bytes + ((unsigned)lcol << sh);
        // pass B operands: SET constant and the epilogue op as wave-uniform selects
        const scalar_t set_value = p.prologue == PRO_SET ? (scalar_t)p.prologue_arg : scalar_t(0);
        const scalar_t epi_arg = (scalar_t)p.epilogue_arg;
        // (blended with masks: a select on a wave-uniform condition comes back as a branch per element)
        const unsigned k_relu = p.epilogue == EPI_RELU ? ~0u : 0u, k_nocond = p.epilogue == EPI_RELU_NOCOND ? ~0u : 0u,
                       k_scale = p.epilogue == EPI_SCALE ? ~0u : 0u, k_set = p.epilogue == EPI_SET ? ~0u : 0u,
                       k_none = p.epilogue == EPI_NONE ? ~0u : 0u;
        auto bits = [](scalar_t x) { return __builtin_bit_cast(unsigned, x); };
        const bool simple = (p.epilogue == EPI_RELU || p.epilogue == EPI_NONE) && set_value == scalar_t(0);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                scalar_t c[4] = {scalar_t(0), scalar_t(0), scalar_t(0), scalar_t(0)};
                if (read_c) {
                    const unsigned off = lane_off + ((unsigned)(i * 16) * row_bytes + ((unsigned)(j * 16) << sh));
                    const unsigned mis = off & 3u; // bytes between the dword boundary and the first element
                    if (sh == 2) {
                        // (the builtins return GCC-style vectors; assigning one to an ext_vector type compiles, to something else)
                        const u32x4 w = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(tile.rsrc, off, 0, 0));
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const unsigned x = w[e]; // (a bit cast applied to the element expression itself reads element 0 with this compiler)
                            c[e] = __builtin_bit_cast(scalar_t, x);
                        }
                    } else if (sh == 1) {
                        typedef unsigned u32x3 __attribute__((ext_vector_type(3)));
                        const u32x3 w = __builtin_bit_cast(u32x3, __builtin_amdgcn_raw_buffer_load_b96(tile.rsrc, off - mis, 0, 0));
                        const unsigned lo = __builtin_amdgcn_alignbyte(w[1], w[0], mis), hi = __builtin_amdgcn_alignbyte(w[2], w[1], mis);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const unsigned half = ((e & 2) ? hi : lo) >> ((e & 1) * 16);
                            if constexpr (IN == IN_I8) c[e] = (int)(short)half; // int16 widens with its sign
                            else {
                                const unsigned as_f16 = __float_as_uint((float)__builtin_bit_cast(_Float16, (unsigned short)half));
                                c[e] = __uint_as_float((as_f16 & m_f16) | ((half << 16) & m_bf16));
                            }
                        }
                    } else {
                        if constexpr (IN == IN_I8) {
                            typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
                            const u32x2 w = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(tile.rsrc, off - mis, 0, 0));
                            const unsigned v4 = __builtin_amdgcn_alignbyte(w[1], w[0], mis);
#pragma unroll
                            for (int e = 0; e < 4; ++e) c[e] = __builtin_amdgcn_sbfe((int)v4, e * 8, 8); // int8 widens with its sign
                        }
                    }
                }
                if (simple) {
                    // C = relu(C + A*B) or C + A*B, beta included: v, then max(v, 0) or max(v, v)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        scalar_t v;
                        if constexpr (IN == IN_I8) v = wrap_add(acc[i][j][e], wrap_mul(c[e], c_mul));
                        else v = acc[i][j][e] + c[e] * c_mul;
                        const scalar_t lo = __builtin_bit_cast(scalar_t, bits(v) & k_none);
                        acc[i][j][e] = v > lo ? v : lo;
                    }
                } else
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    scalar_t v;
                    if constexpr (IN == IN_I8) v = wrap_add(acc[i][j][e], wrap_mul(c[e], c_mul));
                    else v = acc[i][j][e] + c[e] * c_mul;
                    v = wrap_add(v, set_value);
                    const scalar_t r = v > scalar_t(0) ? v : scalar_t(0);
                    const scalar_t n = v * (v > scalar_t(0) ? scalar_t(1) : scalar_t(0));
                    const scalar_t m = wrap_mul(v, epi_arg);
                    acc[i][j][e] = __builtin_bit_cast(scalar_t, (bits(r) & k_relu) | (bits(n) & k_nocond) | (bits(m) & k_scale) |
                                                                    (bits(epi_arg) & k_set) | (bits(v) & k_none));
                }
                __builtin_amdgcn_sched_barrier(0); // block by block: a handful of temporaries next to the 128 accumulators
            }
        store_tile([](scalar_t v) { return v; });
    }

    if constexpr (Cfg::TIMED) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // stores acknowledged
        stamp(3);
        if (threadIdx.x == 0 && p.stamps) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                p.stamps[(blockIdx.x * 4 + i) * 2] = stamp_clk[i]; // (probe runs unbatched)
                p.stamps[(blockIdx.x * 4 + i) * 2 + 1] = stamp_ref[i];
            }
        }
    }
}

// Host launcher for one kernel instantiation.
template <typename Cfg>
hipError_t launch_mfma16(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    auto kern = gemm_mfma16_kernel<Cfg>;
    // an int8 C is written in 16-byte pieces of 16-byte aligned rows; no kernel here has a path for anything else
    if (a.out_type == T_I8 && (a.c_rs % 16 || ((size_t)a.C & 15) || (a.batch > 1 && a.c_bs % 16))) return hipErrorInvalidValue;
    GemmArgs args = a;
    args.tiles_m = (a.M + Cfg::BM - 1) / Cfg::BM;
    args.tiles_n = (a.N + Cfg::BN - 1) / Cfg::BN;
    if (geom) {
        geom->grid[0] = (unsigned)(args.tiles_m * args.tiles_n);
        geom->grid[1] = 1;
        geom->grid[2] = a.batch > 1 ? a.batch : 1;
        geom->block[0] = Cfg::NT;
        geom->block[1] = geom->block[2] = 1;
        geom->dyn_lds = Cfg::LDS_BYTES;
    }
    if (dry_run) return hipSuccess;
    static LdsLimitOnce lds_limit; // per instantiation
    if (hipError_t e = lds_limit.ensure((const void*)kern, Cfg::LDS_BYTES); e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(args.tiles_m * args.tiles_n, 1, a.batch > 1 ? a.batch : 1), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, ACC950_HEAD_OF(args), args);
    return hipGetLastError();
}

} // namespace acc950
