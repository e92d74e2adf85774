// LDS-tiled, multi-stage MFMA GEMM with the prologue/epilogue fused into the
// accumulator write-back, for gfx950 (CDNA4) only.
//
// This is the hand-written replacement for what the reference's tensorized GPU plan
// lowers to: per-warp MMA fragment loads / mma_sync passes / fragment store with
// epilogue (/root/reference/accera/transforms/src/exec/ExecutionPlanToAffineLoweringPass.cpp:5986-6533),
// the workgroup-cooperative block_copy of A/B tiles into shared memory
// (/root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:364-628),
// its double buffering (ExecutionPlanToAffineLoweringPass.cpp:5240-5371) and the
// accumulator (MMA_FRAGMENT) cache of C (:2705-2726).  None of that code is reused:
//
//  * MFMA: v_mfma_f32_32x32x16_{f16,bf16} and v_mfma_i32_32x32x32_i8 -- one
//    instruction consumes 32 bytes of K per row, 16 bytes per lane.
//  * An operand whose K index is contiguous in memory ("KC": row-major A,
//    column-major B) is staged as [row][KB bytes of K] and read with one
//    ds_read_b128 per fragment.  An operand whose M/N index is contiguous ("MC":
//    row-major B) is staged as [k][row bytes] exactly as it lies in memory and read
//    with the gfx950 LDS transpose reads ds_read_b64_tr_b16 / _tr_b8, which hand
//    each lane the K-run of its own column.
//  * 16-byte chunks are XOR-swizzled inside each LDS row so both the fragment reads
//    and the tile fills are bank-conflict free without padding.
//  * Tiles are filled either through registers (global_load_dwordx4 + ds_write_b128)
//    or directly with global_load_lds_dwordx4, which needs no staging registers; in
//    the direct form the swizzle is applied to the global address each lane fetches
//    because the LDS destination of lane l is fixed at base + 16*l.
//  * STAGES LDS buffers, one barrier per K tile: the fill of tile t+STAGES-1 is
//    issued at the start of the MFMAs of tile t, and only the fills of tile t+1 are
//    waited for (s_waitcnt vmcnt(n) with the younger fills still in flight).
//  * Workgroup ids are remapped so that each of the 8 XCDs (own L2 each) works on a
//    compact rectangle of output tiles.
#pragma once
#include "common.h"
#include <type_traits>

namespace acc950 {

enum : int { IN_F16 = 0, IN_BF16 = 1, IN_I8 = 2, IN_F32 = 3 };

template <int IN> struct InTraits { static constexpr int ES = 2; using acc_t = f32x16; using scalar_t = float; };
template <> struct InTraits<IN_I8> { static constexpr int ES = 1; using acc_t = i32x16; using scalar_t = int; };
template <> struct InTraits<IN_F32> { static constexpr int ES = 4; using acc_t = f32x16; using scalar_t = float; };

template <int IN>
__device__ __forceinline__ void mfma32(const i32x4& a, const i32x4& b, typename InTraits<IN>::acc_t& c)
{
    if constexpr (IN == IN_F16)
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    else if constexpr (IN == IN_BF16)
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else if constexpr (IN == IN_F32) {
        // fp32: v_mfma_f32_32x32x2_f32 sums two k per instruction, one from each half of the wave.  A fragment holds four
        // consecutive k of its row per lane (k 0..3 in lanes 0-31, k 4..7 in lanes 32-63 of the 32-byte step), the same for
        // both operands, so instruction e pairs k = e with k = 4 + e and four of them sum the step.
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int ai = a[e], bi = b[e]; // (into scalars first: a bit cast applied to the element expression itself reads element 0)
            c = __builtin_amdgcn_mfma_f32_32x32x2f32(__int_as_float(ai), __int_as_float(bi), c, 0, 0, 0);
        }
    } else
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Staging and fragment access for one operand tile of R rows (M or N extent) and KB
// bytes of K (64 or 128), i.e. BK = KB / element-size K elements.
// MI16: fragments are read for the 16x16 MFMA shapes (16 rows, 64 bytes of K per step).
template <int IN, int R, bool KC, int NT, int KB, bool MI16 = false>
struct OperandTile {
    static_assert(KB == 64 || KB == 128, "K tile is 64 or 128 bytes");
    static constexpr int ES = InTraits<IN>::ES;
    static constexpr int BK = KB / ES;                   // K elements per tile
    static constexpr int KSTEPS = KB / 32;               // MFMA steps per tile
    static constexpr int TILE_BYTES = R * KB;            // same for KC and MC
    static constexpr int CHUNKS = TILE_BYTES / 16;
    // Fill instructions per thread.  When the tile does not split evenly over the
    // workgroup (direct fills only), the waves past the end of the last pass wrap around
    // and fetch chunks from the start of the tile a second time.
    static constexpr int PER_THREAD = (CHUNKS + NT - 1) / NT;
    static constexpr bool EVEN_SPLIT = CHUNKS % NT == 0;
    static_assert(CHUNKS % 64 == 0, "whole waves");
    // KC: one LDS row is one matrix row (KB bytes); MC: one LDS row is one k (R elements).
    static constexpr int ROW_BYTES = KC ? KB : R * ES;
    static constexpr int CPR = ROW_BYTES / 16;           // 16-byte chunks per LDS row

    // LDS chunk position <-> logical chunk of the same row (an involution).
    //  KC, 128-byte rows: a 16-lane read phase touches rows r..r+15 at one chunk; rows
    //      two apart are 256 bytes (all banks) apart, so the row pair index picks the chunk.
    //  KC,  64-byte rows: four rows fill the 256-byte bank span, so row/4 picks the chunk.  (For the
    //      16-row fragments this leaves two-way conflicts; a conflict-free map exists and measured
    //      2 % slower in the ping-pong kernel, where the reads hide behind the sibling's MFMAs.)
    //  MC: a transpose read touches 4 (16-bit) or 8 (8-bit) consecutive k rows, which are
    //      a multiple of 256 bytes apart; k picks a 64- / 32-byte group inside the row.
    __device__ static __forceinline__ int swizzle(int row, int c)
    {
        if constexpr (KC) return KB == 128 ? c ^ ((row >> 1) & 7) : c ^ ((row >> 2) & 3);
        else if constexpr (ES == 4) {
            // 32-bit elements are read one per lane (32 neighbouring columns of a k row = 128 bytes: all banks of one half); the
            // two halves of a wave read k rows four apart and share their banks -- two passes per read, which the 64-cycle
            // fp32 instructions hide, so there is no swizzle to keep in step with the fills
            return c;
        } else if constexpr (!MI16) {
            if constexpr (ES == 2) return c ^ (((row & 3) << 2) & (CPR - 1));
            else return c ^ (((row & 7) << 1) & (CPR - 1));
        } else {
            // 16-row fragments: neighbouring groups of 16 lanes read the same columns 8 (16-bit) or
            // 16 (8-bit) k rows apart; that bit of k moves them to the other half of the group
            if constexpr (ES == 2) return c ^ ((((row & 3) << 2) | (((row >> 3) & 1) << 1)) & (CPR - 1));
            else return c ^ ((((row & 7) << 1) | ((row >> 4) & 1)) & (CPR - 1));
        }
    }
    static constexpr int SWIZZLE_PERIOD = KC ? 16 : ES == 4 ? 1 : (ES == 2 ? (MI16 ? 16 : 4) : (MI16 ? 32 : 8)); // rows after which it repeats

    // Byte offset in global memory of logical chunk (row, c) of the tile whose first
    // row is r0 (M/N index) and first K element is k0.  ld = leading dimension in elements.
    __device__ static __forceinline__ int64_t global_off(int row, int c, int r0, int k0, int64_t ld)
    {
        if constexpr (KC) return ((int64_t)(r0 + row) * ld + k0) * ES + c * 16;
        else return ((int64_t)(k0 + row) * ld + r0) * ES + c * 16;
    }

    // EDGE: is logical chunk (row, c) inside the matrix?  (rmax = M or N, K multiple of 16/ES)
    __device__ static __forceinline__ bool in_bounds(int row, int c, int r0, int k0, int rmax, int K)
    {
        if constexpr (KC) return (r0 + row) < rmax && (k0 + c * (16 / ES)) < K;
        else return (k0 + row) < K && (r0 + c * (16 / ES)) < rmax;
    }

    // ---- register-staged fill ----
    // EDGE 0: full tiles.  1: tiles that end past M / N / K, every row of the operand 16 bytes aligned and K (and the
    // contiguous extent) a multiple of the 16-byte vector: chunks are in or out as a whole.  2: any sizes, leading
    // dimensions and pointers: chunks lie anywhere (the loads are declared unaligned; the hardware takes them), and the
    // chunk that straddles the end of a row is put together from single elements.
    template <int EDGE>
    __device__ static __forceinline__ void load_global(i32x4 (&regs)[PER_THREAD], const char* base, int r0, int k0,
                                                       int64_t ld, int rmax, int K, int tid)
    {
        typedef i32x4 __attribute__((aligned(1))) i32x4_any;
        constexpr int VEC = 16 / ES;
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            int id = tid + i * NT;
            int row = id / CPR, c = id % CPR;
            if constexpr (EDGE == 2) {
                // elements of this chunk inside the matrix: all of them, the first few, or none
                const bool row_in = KC ? (r0 + row) < rmax : (k0 + row) < K;
                const int left = KC ? K - (k0 + c * VEC) : rmax - (r0 + c * VEC);
                const int n = row_in ? (left < 0 ? 0 : left) : 0;
                const char* src = base + global_off(row, c, r0, k0, ld);
                if (n >= VEC) regs[i] = *(const i32x4_any*)src;
                else {
                    i32x4 v = {0, 0, 0, 0};
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        if (e >= n) break;
                        if constexpr (ES == 4) {
                            v[e] = *(const int*)(src + 4 * e);
                        } else if constexpr (ES == 2) {
                            const unsigned x = *(const unsigned short*)(src + 2 * e);
                            v[e >> 1] |= (int)(x << ((e & 1) * 16));
                        } else {
                            const unsigned x = *(const unsigned char*)(src + e);
                            v[e >> 2] |= (int)(x << ((e & 3) * 8));
                        }
                    }
                    regs[i] = v;
                }
            } else if constexpr (EDGE == 1) {
                if (in_bounds(row, c, r0, k0, rmax, K))
                    regs[i] = *(const i32x4*)(base + global_off(row, c, r0, k0, ld));
                else
                    regs[i] = i32x4{0, 0, 0, 0};
            } else {
                regs[i] = *(const i32x4*)(base + global_off(row, c, r0, k0, ld));
            }
        }
    }
    __device__ static __forceinline__ void store_lds(const i32x4 (&regs)[PER_THREAD], char* lds, int tid)
    {
#pragma unroll
        for (int i = 0; i < PER_THREAD; ++i) {
            int id = tid + i * NT;
            int row = id / CPR, c = id % CPR;
            *(i32x4*)(lds + row * ROW_BYTES + swizzle(row, c) * 16) = regs[i];
        }
    }

    // ---- direct global -> LDS fill (global_load_lds_dwordx4) ----
    // Lane l of a wave writes LDS bytes [M0 + 16*l, +16), so LDS chunk position
    // id = tid + i*NT is fixed and the lane fetches the logical chunk that the swizzle
    // maps there.  The swizzle only depends on the low row bits, which are the same
    // for every i, so one per-lane 32-bit offset serves all fills of the kernel and
    // the rest of the address is wave-uniform (SGPR base, advanced per K tile).
    static constexpr int ROWS_PER_PASS = NT / CPR; // rows covered by one fill instruction of the workgroup
    static_assert(NT % CPR == 0 && ROWS_PER_PASS % SWIZZLE_PERIOD == 0, "swizzle must repeat every pass");

    __device__ static __forceinline__ unsigned direct_lane_offset(int64_t ld, int tid)
    {
        int row = tid / CPR, cpos = tid % CPR;
        return (unsigned)global_off(row, swizzle(row, cpos), 0, 0, ld);
    }
    // Global byte distance covered by all LDS rows of the tile (for the wrap-around above).
    __device__ static __forceinline__ int64_t wrap_bytes(int64_t ld) { return global_off(CHUNKS / CPR, 0, 0, 0, ld); }
    static_assert(EVEN_SPLIT || (CHUNKS / CPR) % SWIZZLE_PERIOD == 0, "wrap-around keeps the swizzle phase");
    // Uniform base of fill i for the tile at (r0, k0).
    __device__ static __forceinline__ const char* direct_base(const char* base, int i, int r0, int k0, int64_t ld)
    {
        return base + global_off(i * ROWS_PER_PASS, 0, r0, k0, ld);
    }
    // The instruction is issued from inline assembly so that the compiler does not
    // serialise later LDS reads of the *other* buffers behind it; the kernel waits with
    // an explicit s_waitcnt vmcnt(n) before the barrier that publishes the tile.
    __device__ static __forceinline__ void direct_issue(unsigned lds_addr, unsigned lane_off, const char* sbase)
    {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(lds_addr), "v"(lane_off), "s"(sbase)
                     : "memory");
    }

    // Same for an address the register allocator may have put into vector registers although it is the same in every
    // lane (scalar registers run short around the hand-laid loop): lane 0's copy is taken explicitly.
    __device__ static __forceinline__ void direct_issue_uniform(unsigned lds_addr, unsigned lane_off, const char* sbase)
    {
        const unsigned long long a = (unsigned long long)sbase;
        const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
        direct_issue(__builtin_amdgcn_readfirstlane(lds_addr), lane_off, (const char*)(((unsigned long long)hi << 32) | lo));
    }

    // ---- fragment read: 32 rows starting at row0, k-step ks (32 bytes of K) ----
    __device__ static __forceinline__ i32x4 read_frag(const char* lds, int row0, int ks, int lane)
    {
        if constexpr (KC) {
            int row = row0 + (lane & 31);
            int c = ks * 2 + (lane >> 5);
            return *(const i32x4*)(lds + row * ROW_BYTES + swizzle(row, c) * 16);
        } else if constexpr (ES == 4) {
            // 32-bit elements, staged [k][row]: the lane's column (row0 + lane % 32) of the four k rows of its half
            const int col_byte = (row0 + (lane & 31)) * 4;
            const int c = col_byte >> 4, within = col_byte & 15;
            i32x4 out;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int k = ks * 8 + (lane >> 5) * 4 + e;
                out[e] = *(const int*)(lds + k * ROW_BYTES + swizzle(k, c) * 16 + within);
            }
            return out;
        } else if constexpr (ES == 2) {
            // ds_read_b64_tr_b16: in each group of 16 lanes, lanes 4j..4j+3 point at k-row j
            // (4 x 8 bytes = 16 columns); lane i receives column i of those 4 rows.
            int h = lane >> 5, g = (lane >> 4) & 1, i = lane & 15;
            int col_byte = (row0 + g * 16 + (i & 3) * 4) * 2;
            int c = col_byte >> 4, within = col_byte & 15;
            i32x4 out;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                int k = ks * 16 + h * 8 + q * 4 + (i >> 2);
                const char* p = lds + k * ROW_BYTES + swizzle(k, c) * 16 + within;
                s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ACC950_LDS s16x4*)p);
                i32x2 w = __builtin_bit_cast(i32x2, v);
                out[q * 2] = w[0];
                out[q * 2 + 1] = w[1];
            }
            return out;
        } else {
            // ds_read_b64_tr_b8: lanes 2j, 2j+1 point at k-row j (2 x 8 bytes = 16 columns);
            // lane i receives column i of those 8 rows.
            int h = lane >> 5, g = (lane >> 4) & 1, i = lane & 15;
            int col_byte = row0 + g * 16 + (i & 1) * 8;
            int c = col_byte >> 4, within = col_byte & 15;
            i32x4 out;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                int k = ks * 32 + h * 16 + q * 8 + (i >> 1);
                const char* p = lds + k * ROW_BYTES + swizzle(k, c) * 16 + within;
                i32x2 w = __builtin_amdgcn_ds_read_tr8_b64_v2i32((ACC950_LDS i32x2*)p);
                out[q * 2] = w[0];
                out[q * 2 + 1] = w[1];
            }
            return out;
        }
    }

    // ---- fragment read for the 16x16 shapes: 16 rows starting at row0, k-step ks (64 bytes of K).
    // Lane l gets row (l % 16) and the 16 bytes of K number (l / 16) of the step.
    __device__ static __forceinline__ i32x4 read_frag16(const char* lds, int row0, int ks, int lane)
    {
        static_assert(MI16, "tile staged for the 32x32 shapes");
        const int kg = lane >> 4, i = lane & 15;
        if constexpr (KC) {
            int row = row0 + i;
            int c = ks * 4 + kg;
            return *(const i32x4*)(lds + row * ROW_BYTES + swizzle(row, c) * 16);
        } else if constexpr (ES == 2) {
            // ds_read_b64_tr_b16 (see read_frag): all four groups of 16 lanes read the same 16 columns
            int col_byte = (row0 + (i & 3) * 4) * 2;
            int c = col_byte >> 4, within = col_byte & 15;
            i32x4 out;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                int k = ks * 32 + kg * 8 + q * 4 + (i >> 2);
                const char* p = lds + k * ROW_BYTES + swizzle(k, c) * 16 + within;
                s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ACC950_LDS s16x4*)p);
                i32x2 w = __builtin_bit_cast(i32x2, v);
                out[q * 2] = w[0];
                out[q * 2 + 1] = w[1];
            }
            return out;
        } else {
            int col_byte = row0 + (i & 1) * 8;
            int c = col_byte >> 4, within = col_byte & 15;
            i32x4 out;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                int k = ks * 64 + kg * 16 + q * 8 + (i >> 1);
                const char* p = lds + k * ROW_BYTES + swizzle(k, c) * 16 + within;
                i32x2 w = __builtin_amdgcn_ds_read_tr8_b64_v2i32((ACC950_LDS i32x2*)p);
                out[q * 2] = w[0];
                out[q * 2 + 1] = w[1];
            }
            return out;
        }
    }
};

// Output tile -> (tile_m, tile_n).  Consecutive workgroup ids go to different XCDs
// (id % 8), so ids are first regrouped per XCD and then walked in column-major order
// inside bands of GROUP_M tile rows, which makes the tiles resident on one XCD at any
// time a compact rectangle that shares A and B tiles through that XCD's L2.
__device__ __forceinline__ void tile_coords(int pid, int tiles_m, int tiles_n, int& tm, int& tn)
{
    constexpr int XCDS = 8, GROUP_M = 4;
    int total = tiles_m * tiles_n;
    if (total % XCDS == 0) pid = (pid % XCDS) * (total / XCDS) + pid / XCDS;
    int per_group = GROUP_M * tiles_n;
    int group = pid / per_group;
    int first_m = group * GROUP_M;
    int gsz = tiles_m - first_m < GROUP_M ? tiles_m - first_m : GROUP_M;
    int in_group = pid % per_group;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

// Compile-time description of one kernel instantiation.
template <int IN_, int BM_, int BN_, int WAVES_M_, int WAVES_N_, bool A_KC_, bool B_KC_, bool DIRECT_, bool EDGE_, int KB_, int STAGES_,
          bool PINGPONG_ = false, bool TIMED_ = false, bool ANY_ = false>
struct MfmaConfig {
    // ANY (an EDGE build): operands of any size, leading dimension and alignment (see OperandTile::load_global)
    static constexpr bool ANY = ANY_;
    static_assert(!ANY_ || EDGE_, "the any-shape fill is a form of the edge fill");
    static constexpr bool PINGPONG = PINGPONG_;
    // TIMED: wave 0 of every workgroup reads the shader-clock counter and the constant
    // 100 MHz counter at kernel entry, after the prologue, after the main loop and at the
    // end, and writes them to GemmArgs::stamps (phase times and the clock the engine ran at).
    static constexpr bool TIMED = TIMED_;
    // workgroups meant to share a CU: as many as the LDS allows, at most 2 waves per SIMD in all
    static constexpr int WGS_PER_CU = (WAVES_M_ * WAVES_N_ <= 4 && 2 * STAGES_ * (BM_ + BN_) * KB_ <= 160 * 1024 && BM_ * BN_ <= 256 * 128) ? 2 : 1;
    static constexpr int IN = IN_, BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, KB = KB_, STAGES = STAGES_;
    static constexpr bool A_KC = A_KC_, B_KC = B_KC_, DIRECT = DIRECT_, EDGE = EDGE_;
    static constexpr int NT = WAVES_M * WAVES_N * 64;
    static constexpr int LDS_BYTES = STAGES * (BM + BN) * KB;
    static_assert(!(DIRECT && EDGE), "edge tiles are zero-filled through registers");
    static_assert(DIRECT || STAGES == 2, "the register-staged fill is double-buffered");
    static_assert(STAGES >= 2 && STAGES <= 4, "2 to 4 LDS stages");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget of one CU");
    static_assert(!PINGPONG || (DIRECT && WAVES_M * WAVES_N == 8), "ping-pong needs 8 waves and direct fills");
};

// ---- buffer access to the output tile ---------------------------------------------------
// A raw buffer descriptor (base in scalar registers, 32-bit offsets) over the part of C a
// workgroup or wave writes; reads and writes name an element by a per-lane offset, a scalar
// offset and an immediate.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
struct CTile {
    __amdgpu_buffer_rsrc_t rsrc;
};
// Descriptor that starts `back` bytes before element (row, col) of C (elements of `os` bytes) and ends with the
// last row of C: the kernels test the edges themselves, and an access that slips past the end of the matrix all
// the same is dropped by the hardware's range check instead of reaching memory.
__device__ __forceinline__ CTile c_tile(const GemmArgs& p, int row, int col, unsigned os, unsigned back = 0)
{
    char* base = (char*)p.C + ((int64_t)row * p.c_rs + col) * os - back;
    // (rounded up to the end of the dword that holds the last element: reads of sub-dword elements fetch the aligned dword
    // around them, and the range check is on the whole access)
    const int64_t bytes = ((((int64_t)(p.M - 1 - row) * p.c_rs + (p.N - col)) * os + back) + 3) & ~(int64_t)3;
    const unsigned records = bytes <= 0 ? 0u : bytes > 0xffffffffll ? 0xffffffffu : (unsigned)bytes;
    return CTile{__builtin_amdgcn_make_buffer_rsrc(base, 0, records, 0x00020000)};
}
template <typename T>
__device__ __forceinline__ T c_load(CTile t, unsigned voff, unsigned soff)
{
    if constexpr (sizeof(T) == 4) return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b32(t.rsrc, voff, soff, 0));
    else if constexpr (sizeof(T) == 2) return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b16(t.rsrc, voff, soff, 0));
    else return __builtin_bit_cast(T, __builtin_amdgcn_raw_buffer_load_b8(t.rsrc, voff, soff, 0));
}
// (AUX: the cache policy.  Only stores that write whole 128-byte lines go through the L2 -- see C_STORE_AUX; pieces of
// lines, as the edge kernels and the element-wise narrow stores write them, would each become a read-modify-write in
// memory: 600x64x196 fp16 with beta = 1 on the any-alignment kernel took 20 us that way instead of 10.)
template <typename T, int AUX = 0>
__device__ __forceinline__ void c_store(CTile t, unsigned voff, unsigned soff, T v)
{
    if constexpr (sizeof(T) == 4) __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), t.rsrc, voff, soff, AUX);
    else if constexpr (sizeof(T) == 2) __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, v), t.rsrc, voff, soff, AUX);
    else __builtin_amdgcn_raw_buffer_store_b8(__builtin_bit_cast(unsigned char, v), t.rsrc, voff, soff, AUX);
}

// Whether a kernel takes fewer rows of A than its tile has (see short_m in the kernel): direct fills of a row-major A whose
// fill instructions split evenly over the workgroup.  The launcher refuses such a problem for every other instantiation.
template <typename Cfg>
constexpr bool mfma_takes_short_m()
{
    return Cfg::DIRECT && !Cfg::EDGE && Cfg::A_KC && OperandTile<Cfg::IN, Cfg::BM, Cfg::A_KC, Cfg::NT, Cfg::KB>::EVEN_SPLIT;
}

template <typename Cfg>
__global__ void __launch_bounds__(Cfg::NT, Cfg::WGS_PER_CU) gemm_mfma_kernel(ACC950_HEAD_PARAMS, GemmArgs p)
{
    constexpr int IN = Cfg::IN, BM = Cfg::BM, BN = Cfg::BN, WAVES_M = Cfg::WAVES_M, WAVES_N = Cfg::WAVES_N;
    constexpr int KB = Cfg::KB, STAGES = Cfg::STAGES, NT = Cfg::NT;
    constexpr bool A_KC = Cfg::A_KC, B_KC = Cfg::B_KC, DIRECT = Cfg::DIRECT, EDGE = Cfg::EDGE;
    constexpr int FILL_MODE = Cfg::ANY ? 2 : (EDGE ? 1 : 0);
    constexpr int ES = InTraits<IN>::ES;
    constexpr int BK = KB / ES;
    constexpr int KSTEPS = KB / 32;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile is made of 32x32 MFMA blocks");
    using TA = OperandTile<IN, BM, A_KC, NT, KB>;
    using TB = OperandTile<IN, BN, B_KC, NT, KB>;
    using acc_t = typename InTraits<IN>::acc_t;
    using scalar_t = typename InTraits<IN>::scalar_t;
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
    // Full-tile builds: M and N need not be multiples of the tile -- the last row / column of tiles is moved to end at
    // M / N and overlaps its neighbour, and what both compute gets the same bits from both (the host allows this only when C
    // is not read, and only for sizes whose moved tile still starts on a 16-byte boundary of the operands' and C's rows).
    // (fewer rows than one tile has -- the tiles with direct fills of a row-major A take that, see short_m below: the one row of tiles starts at row 0)
    const int m0 = EDGE || tile_m * BM + BM <= p.M ? tile_m * BM : p.M >= BM ? p.M - BM : 0;
    const int n0 = EDGE || tile_n * BN + BN <= p.N ? tile_n * BN : p.N - BN;

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

    // LDS byte address of the tile buffers as the hardware sees it (for M0).
    const unsigned smem_addr = (unsigned)(size_t)(ACC950_LDS char*)smem;
    const unsigned wave_lds = __builtin_amdgcn_readfirstlane((unsigned)(wave * 1024));
    unsigned a_lane_off = 0, b_lane_off = 0;
    if constexpr (DIRECT) {
        a_lane_off = TA::direct_lane_offset(lda, tid);
        b_lane_off = TB::direct_lane_offset(ldb, tid);
    }
    constexpr int FILLS_A = TA::PER_THREAD, FILLS_B = TB::PER_THREAD, FILLS = FILLS_A + FILLS_B;
    // Fewer rows of A than the tile has (A with K contiguous, direct fills): the fills of rows past the end
    // fetch A's last row instead -- every lane its own offset from the tile's first row, per fill instruction -- and what the
    // matrix cores make of those rows is dropped by the range check of C's descriptor, which ends with C's last row.
    constexpr bool SHORT_M_OK = mfma_takes_short_m<Cfg>();
    const bool short_m = SHORT_M_OK && p.M < BM;
    unsigned a_short_off[SHORT_M_OK ? FILLS_A : 1];
    if constexpr (SHORT_M_OK) {
#pragma unroll
        for (int f = 0; f < FILLS_A; ++f) {
            const int row = f * TA::ROWS_PER_PASS + tid / TA::CPR, cpos = tid % TA::CPR;
            const int row_g = short_m && row >= p.M ? p.M - 1 : row;
            a_short_off[f] = (unsigned)TA::global_off(row_g, TA::swizzle(row, cpos), 0, 0, lda);
        }
    }
    // fill number f of the tile starting at K element k0 into stage buffer `stage`
    static_assert(DIRECT || (TA::EVEN_SPLIT && TB::EVEN_SPLIT), "register-staged fills need an even split");
    auto fill_one = [&](auto tile_tag, int f, unsigned lds_tile, unsigned lane_off, const char* base, int r0, int k0,
                        int64_t ld) {
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
        if constexpr (SHORT_M_OK) {
            // (always this way, short rows or not: every fill of A from the base of the first, the rows in the lanes' offsets
            // -- a test of short_m here would split the K loop into blocks and put waits for memory where they join)
            if (f < FILLS_A) {
                TA::direct_issue(smem_addr + stage * STAGE_BYTES + wave_lds + f * NT * 16, a_short_off[f], TA::direct_base(Ab, 0, m0, k0, lda));
                return;
            }
        }
        if (f < FILLS_A) fill_one(TA{}, f, smem_addr + stage * STAGE_BYTES, a_lane_off, Ab, m0, k0, lda);
        else fill_one(TB{}, f - FILLS_A, smem_addr + stage * STAGE_BYTES + TA::TILE_BYTES, b_lane_off, Bb, n0, k0, ldb);
    };

    // MFMAs of one K tile.  Fragments are double-buffered across the k-steps: the LDS
    // reads of step ks+1 are issued between the MFMAs of step ks, one per MFMA slot,
    // and (direct form) the fills of a later tile go out with the first MFMA slots so
    // that they have the rest of this tile, and the following ones, to land.  With
    // CROSS the reads issued during the last k-step fetch step 0 of the *next* tile
    // (already published), so no LDS latency is exposed after the barrier.  A
    // sched_barrier after every slot pins this order against the machine scheduler.
    constexpr int SLOTS = TM * TN;
    constexpr int FILLS_PER_SLOT = (FILLS + SLOTS - 1) / SLOTS; // all fills within the first k-step
    constexpr int READS_PER_SLOT = (TM + TN + SLOTS - 1) / SLOTS; // (more than one only for wave tiles of one or two blocks)
    static_assert(KSTEPS % 2 == 0, "fragment buffers alternate per k-step and must line up across tiles");
    i32x4 af[2][TM], bf[2][TN];
    auto load_first_frags = [&](const char* sa, const char* sb) {
#pragma unroll
        for (int i = 0; i < TM; ++i) af[0][i] = TA::read_frag(sa, wr0 + i * 32, 0, lane);
#pragma unroll
        for (int j = 0; j < TN; ++j) bf[0][j] = TB::read_frag(sb, wc0 + j * 32, 0, lane);
    };
    auto mma_tile = [&](const char* sa, const char* sb, const char* next_sa, const char* next_sb, auto fill_tag,
                        auto cross_tag, int fill_stage, int fill_k0) {
        constexpr bool fill = decltype(fill_tag)::value;
        constexpr bool cross = decltype(cross_tag)::value;
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
            const bool last = ks + 1 == KSTEPS;
            const char* ra = last ? next_sa : sa;
            const char* rb = last ? next_sb : sb;
            const int rks = last ? 0 : ks + 1;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const int slot = i * TN + j;
                    mfma32<IN>(af[ks & 1][i], bf[ks & 1][j], acc[i][j]);
                    if (!last || cross) {
                        // B fragments first: the first MFMAs of the next step need bf[0] and af[0]
#pragma unroll
                        for (int u = 0; u < READS_PER_SLOT; ++u) {
                            const int q = slot * READS_PER_SLOT + u;
                            if (q < TN) bf[(ks + 1) & 1][q] = TB::read_frag(rb, wc0 + q * 32, rks, lane);
                            else if (q - TN < TM) af[(ks + 1) & 1][q - TN] = TA::read_frag(ra, wr0 + (q - TN) * 32, rks, lane);
                        }
                    }
                    if constexpr (DIRECT && fill) {
                        if (ks == 0) {
#pragma unroll
                            for (int u = 0; u < FILLS_PER_SLOT; ++u) {
                                const int f = slot * FILLS_PER_SLOT + u;
                                if (f < FILLS) issue_fill(f, fill_stage, fill_k0);
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
    };

    if constexpr (Cfg::PINGPONG) {
        // Ping-pong schedule for 8 waves (two per SIMD).  Every k-step is split into a
        // memory cluster (fragment reads from LDS, a share of the fills of tile kt+D) and
        // a compute cluster (the MFMAs of that step), each closed by a barrier.  Waves
        // 4..7 run one cluster behind waves 0..3, so on every SIMD one wave is in its
        // compute cluster while its sibling is in its memory cluster: LDS and fill latency
        // is hidden by the sibling's MFMAs instead of by software pipelining.
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
        // CL k-steps form one cluster: the whole K tile when it has 2 steps, half of it when 4
        constexpr int CL = 2, CLUSTERS = KSTEPS / CL, FPC = (FILLS + CLUSTERS - 1) / CLUSTERS;
        auto pp_tile = [&](int kt, auto fill_tag) {
            constexpr bool fill = decltype(fill_tag)::value;
            const char* sa = smem + (kt % STAGES) * STAGE_BYTES;
            const char* sb = sa + TA::TILE_BYTES;
#pragma unroll
            for (int c = 0; c < CLUSTERS; ++c) {
                // ---- memory cluster
#pragma unroll
                for (int q = 0; q < CL; ++q) {
#pragma unroll
                    for (int j = 0; j < TN; ++j) bf[q][j] = TB::read_frag(sb, wc0 + j * 32, c * CL + q, lane);
#pragma unroll
                    for (int i = 0; i < TM; ++i) af[q][i] = TA::read_frag(sa, wr0 + i * 32, c * CL + q, lane);
                }
                if constexpr (fill) {
#pragma unroll
                    for (int u = 0; u < FPC; ++u)
                        if (c * FPC + u < FILLS) issue_fill(c * FPC + u, (kt + D) % STAGES, (kt + D) * BK);
                }
                if (c + 1 == CLUSTERS) { // own fills of tile kt+1 have landed before the barrier publishes them
                    if constexpr (fill) wait_vmcnt<(D - 1) * FILLS>();
                    else wait_vmcnt<0>();
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // fragments are in registers: the buffer may be refilled
                raw_barrier();
                // ---- compute cluster
                __builtin_amdgcn_s_setprio(2);
#pragma unroll
                for (int q = 0; q < CL; ++q)
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j) mfma32<IN>(af[q][i], bf[q][j], acc[i][j]);
                __builtin_amdgcn_s_setprio(0);
                raw_barrier();
            }
        };
        int kt = 0;
        for (; kt + D < KT; ++kt) pp_tile(kt, std::true_type{});
        for (; kt < KT; ++kt) pp_tile(kt, std::false_type{});
        if (group == 0) raw_barrier(); // match the extra barrier of the other group
    } else if constexpr (DIRECT) {
        // D tiles are in flight beyond the one being computed; AHEAD of them are already
        // published (landed and behind a barrier) when a tile starts.
        constexpr int D = STAGES - 1;
        constexpr int AHEAD = STAGES >= 3 ? 2 : 1;
        constexpr bool CROSS = AHEAD >= 2;
        constexpr int YOUNGER = (D - AHEAD) * FILLS; // fills allowed to be outstanding at the end of a tile
        using cross_t = std::integral_constant<bool, CROSS>;
#pragma unroll
        for (int s = 0; s < D; ++s)
            if (s < KT) {
#pragma unroll
                for (int f = 0; f < FILLS; ++f) issue_fill(f, s, s * BK);
            }
        if (KT >= D) wait_vmcnt<YOUNGER>();
        else wait_vmcnt<0>();
        __syncthreads();
        stamp(1);
        if constexpr (CROSS) load_first_frags(smem, smem + TA::TILE_BYTES);
        int kt = 0;
        // steady state: tile kt+D exists and is fetched now
        for (; kt + D < KT; ++kt) {
            const char* cur = smem + (kt % STAGES) * STAGE_BYTES;
            const char* nxt = smem + ((kt + 1) % STAGES) * STAGE_BYTES;
            if constexpr (!CROSS) load_first_frags(cur, cur + TA::TILE_BYTES);
            mma_tile(cur, cur + TA::TILE_BYTES, nxt, nxt + TA::TILE_BYTES, std::true_type{}, cross_t{}, (kt + D) % STAGES,
                     (kt + D) * BK);
            wait_vmcnt<YOUNGER>(); // tile kt+AHEAD has landed
            __syncthreads();
        }
        // drain: nothing left to fetch (the cross prefetch of the last tile reads a stale buffer, unused)
        for (; kt < KT; ++kt) {
            const char* cur = smem + (kt % STAGES) * STAGE_BYTES;
            const char* nxt = smem + ((kt + 1) % STAGES) * STAGE_BYTES;
            if constexpr (!CROSS) load_first_frags(cur, cur + TA::TILE_BYTES);
            mma_tile(cur, cur + TA::TILE_BYTES, nxt, nxt + TA::TILE_BYTES, std::false_type{}, cross_t{}, 0, 0);
            if (kt + 1 < KT) {
                wait_vmcnt<0>();
                __syncthreads();
            }
        }
    } else {
        // Register-staged fill: a K tile travels global memory -> registers -> LDS.  The LDS side is double-buffered; the
        // register side is a ring of R tiles, so that R loads are in flight while one tile is multiplied (a 64 x 64 tile is
        // multiplied in a fraction of the time its load takes: with one tile in flight a k-step costs the memory latency).
        // Tile t sits in slot t % R; the slot of the tile that has just gone to LDS is refilled with tile t + R.
        // (measured on the odd shapes of the reference's lists, ring of three against one: fp16 7 - 10 % faster -- 1000^3 12.5 ->
        // 11.7 us, 5041x192x720 10.2 -> 9.1, 600x64x196 6.7 -> 5.8 -- int8 3 - 4 % slower, so 16-bit inputs only)
        constexpr int R = Cfg::ANY && BM * BN <= 64 * 64 && ES == 2 ? 3 : 1;
        i32x4 ra[R][TA::PER_THREAD], rb[R][TB::PER_THREAD];
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (r < KT) {
                TA::template load_global<FILL_MODE>(ra[r], Ab, m0, r * BK, lda, p.M, p.K, tid);
                TB::template load_global<FILL_MODE>(rb[r], Bb, n0, r * BK, ldb, p.N, p.K, tid);
            }
        TA::store_lds(ra[0], smem, tid);
        TB::store_lds(rb[0], smem + TA::TILE_BYTES, tid);
        __syncthreads();
        for (int kt0 = 0; kt0 < KT; kt0 += R) {
#pragma unroll
            for (int u = 0; u < R; ++u) {
                const int kt = kt0 + u;
                if (kt >= KT) break;
                char* cur = smem + (kt & 1) * STAGE_BYTES;
                char* nxt = smem + ((kt + 1) & 1) * STAGE_BYTES;
                if (kt + R < KT) {
                    TA::template load_global<FILL_MODE>(ra[u], Ab, m0, (kt + R) * BK, lda, p.M, p.K, tid);
                    TB::template load_global<FILL_MODE>(rb[u], Bb, n0, (kt + R) * BK, ldb, p.N, p.K, tid);
                }
                load_first_frags(cur, cur + TA::TILE_BYTES);
                mma_tile(cur, cur + TA::TILE_BYTES, cur, cur + TA::TILE_BYTES, std::false_type{}, std::false_type{}, 0, 0);
                if (kt + 1 < KT) {
                    TA::store_lds(ra[(u + 1) % R], nxt, tid);
                    TB::store_lds(rb[(u + 1) % R], nxt + TA::TILE_BYTES, tid);
                }
                __syncthreads();
            }
        }
    }

    stamp(2);
    // Write-back in three passes over the accumulator registers, so that every piece of
    // code exists once per thing it depends on (element type or op), not once per combination:
    //   A. prologue NONE / SCALE: acc += (arg *) C        (one copy per output type)
    //   B. prologue SET constant and the epilogue op, in place   (one copy per op)
    //   C. narrowing store                                 (one copy per output type)
    // MFMA 32x32 accumulator layout: register r of lane l holds
    //   row = (r/4)*8 + (l/32)*4 + r%4,  column = l%32.
    // C is row-major here (the host transposes the problem otherwise).  All accesses to C are
    // buffer instructions on a descriptor of the workgroup's tile: the lane's place in the tile
    // is one 32-bit register, the row of the access a scalar offset and the column block an
    // immediate, so no address registers compete with the live accumulators.
    const int row_in_tile = wr0 + (lane >> 5) * 4, col_in_tile = wc0 + (lane & 31);
    // fn(descriptor, lane offset, row offset, acc element) -> acc element, for every element of the wave tile
    auto for_each_element = [&](auto out_tag, auto&& fn) {
        using out_t = decltype(out_tag);
        constexpr unsigned OS = sizeof(out_t);
        const CTile tile = c_tile(p, m0, n0, OS); // uniform
        const unsigned row_bytes = (unsigned)p.c_rs * OS;
        const unsigned lane_off = (unsigned)row_in_tile * row_bytes + (unsigned)col_in_tile * OS;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row_off = i * 32 + (r >> 2) * 8 + (r & 3);
                const unsigned soff = (unsigned)row_off * row_bytes; // scalar
                if (EDGE && m0 + row_in_tile + row_off >= p.M) continue;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if (EDGE && n0 + col_in_tile + j * 32 >= p.N) continue;
                    acc[i][j][r] = fn(tile, lane_off + j * 32 * OS, soff, acc[i][j][r]);
                }
                if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0); // keep loads of pass A near their use: no second copy of the tile in registers
            }
    };
    auto for_each_acc = [&](auto&& fn) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = fn(acc[i][j][r]);
                __builtin_amdgcn_sched_barrier(0); // block by block, in place
            }
    };

    auto general_ops = [&]() {
    // ---- pass A
    const bool accumulate = p.prologue != PRO_SET; // NONE, SCALE: C is read
    if (accumulate) {
        const scalar_t c_mul = p.prologue == PRO_SCALE ? (scalar_t)p.prologue_arg : scalar_t(1); // x1 is exact
        // One copy for all output types of the kernel (a switch over the load widths would hand the
        // register allocator one version of every accumulator per type to merge): the aligned dword
        // that holds the element is read and the element cut out of it.
        const unsigned sh = (p.out_type == T_I32 || p.out_type == T_F32) ? 2 : (p.out_type == T_I8 ? 0 : 1);
        const unsigned m_f32 = p.out_type == T_F32 ? ~0u : 0u, m_f16 = p.out_type == T_F16 ? ~0u : 0u, m_bf16 = p.out_type == T_BF16 ? ~0u : 0u;
        char* tile_base = (char*)p.C + (((int64_t)m0 * p.c_rs + n0) << sh);
        const unsigned base_mis = (unsigned)(size_t)tile_base & 3u;  // the descriptor starts at the dword that holds the tile's first element
        const CTile tile = c_tile(p, m0, n0, 1u << sh, base_mis);
        const unsigned row_bytes = (unsigned)p.c_rs << sh;
        const unsigned lane_off = base_mis + (unsigned)row_in_tile * row_bytes + ((unsigned)col_in_tile << sh);
        // (sum, word, byte of the element inside the word) -> the sum with the element added
        auto add_c = [&](scalar_t sum, unsigned word, unsigned mis) -> scalar_t {
            if constexpr (IN == IN_I8) { // int16 / int8 widen with their sign
                const int c = sh == 2 ? (int)word : __builtin_amdgcn_sbfe((int)word, mis * 8, 8u << sh);
                return wrap_add(sum, wrap_mul(c, c_mul));
            } else {
                // the three readings of the word, blended with wave-uniform masks (selects on a
                // uniform condition come back as one branch per element)
                const unsigned half = word >> (mis * 8);
                const unsigned as_f16 = __float_as_uint((float)__builtin_bit_cast(_Float16, (unsigned short)half));
                const unsigned bits = (word & m_f32) | (as_f16 & m_f16) | ((half << 16) & m_bf16);
                return sum + __uint_as_float(bits) * c_mul;
            }
        };
        auto offset_of = [&](int i, int r, int j) { return lane_off + ((unsigned)(i * 32 + (r >> 2) * 8 + (r & 3)) * row_bytes + ((unsigned)(j * 32) << sh)); };
        if constexpr (TM * TN * 16 <= 64) {
            // A small wave tile (64 sums per lane) has the registers for a second copy: all of its loads are issued before the
            // first is used, so the tile of C costs one trip through memory instead of one per eight loads (left to the
            // compiler's own order: 7 us of a 29 us launch at 2048^3 with 128 x 128 tiles).  The edge kernels read the same
            // way, their tests of the edges around the load alone: with the use inside the test as well, every load waited
            // for the one before (a wait for memory sits where the skipped and the loaded paths join), 16 to 64 trips
            // through memory in a row -- 600x64x196 int8 with beta = 1: 10.0 us, 5.0 this way.  (Loads without any test,
            // the descriptor's range check as the only guard, were tried too: the compiler then put a wait for memory in
            // front of every store of the fp16 / bf16 kernels.)
            unsigned words[TM][16][TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r)
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        const bool inside = !EDGE || (m0 + row_in_tile + i * 32 + (r >> 2) * 8 + (r & 3) < p.M && n0 + col_in_tile + j * 32 < p.N);
                        const unsigned off = offset_of(i, r, j) & ~3u;
                        if constexpr (IN == IN_I8) {
                            // (a lane outside reads at an offset beyond any descriptor's range: the range check answers with 0)
                            words[i][r][j] = __builtin_amdgcn_raw_buffer_load_b32(tile.rsrc, inside ? off : 0xfffffffcu, 0, 0);
                        } else {
                            words[i][r][j] = 0;
                            if (inside) words[i][r][j] = __builtin_amdgcn_raw_buffer_load_b32(tile.rsrc, off, 0, 0);
                        }
                    }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r)
#pragma unroll
                    for (int j = 0; j < TN; ++j) acc[i][j][r] = add_c(acc[i][j][r], words[i][r][j], offset_of(i, r, j) & 3u);
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row_off = i * 32 + (r >> 2) * 8 + (r & 3);
                    if (EDGE && m0 + row_in_tile + row_off >= p.M) continue;
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        if (EDGE && n0 + col_in_tile + j * 32 >= p.N) continue;
                        const unsigned off = offset_of(i, r, j);
                        acc[i][j][r] = add_c(acc[i][j][r], __builtin_amdgcn_raw_buffer_load_b32(tile.rsrc, off & ~3u, 0, 0), off & 3u);
                    }
                    if ((r & 3) == 3) __builtin_amdgcn_sched_barrier(0); // keep the loads near their use: no second copy of a large tile in registers
                }
        }
    }

    // ---- pass B (ReLU after a SET-0 prologue is the fused hot path: one max per element; every other
    // combination shares one copy with wave-uniform selects)
    if (p.epilogue == EPI_RELU && !(p.prologue == PRO_SET && p.prologue_arg != 0.f)) {
        for_each_acc([&](scalar_t v) { return v > scalar_t(0) ? v : scalar_t(0); });
    } else if (p.epilogue != EPI_NONE || (p.prologue == PRO_SET && p.prologue_arg != 0.f)) {
        const scalar_t set_value = p.prologue == PRO_SET ? (scalar_t)p.prologue_arg : scalar_t(0);
        const scalar_t epi_arg = (scalar_t)p.epilogue_arg;
        const bool is_relu = p.epilogue == EPI_RELU, is_nocond = p.epilogue == EPI_RELU_NOCOND, is_scale = p.epilogue == EPI_SCALE,
                   is_set = p.epilogue == EPI_SET;
        for_each_acc([&](scalar_t v) {
            v = wrap_add(v, set_value);
            const scalar_t r = v > scalar_t(0) ? v : scalar_t(0);
            const scalar_t n = v * (v > scalar_t(0) ? scalar_t(1) : scalar_t(0));
            const scalar_t m = wrap_mul(v, epi_arg);
            return is_relu ? r : (is_nocond ? n : (is_scale ? m : (is_set ? epi_arg : v)));
        });
    }
    };

    // ---- pass C
    // Narrow outputs: a lane's accumulators are one column wide, so direct stores write
    // 64- or 32-byte pieces of a row per instruction.  Instead each wave stages 32 rows of its
    // tile in a private slab of the (now idle) LDS tile buffers and streams them out as
    // 16-byte pieces that cover whole rows of the wave tile.
    constexpr int PITCH_DW = (WTN / 2) % 32 == 16 ? WTN / 2 : WTN / 2 + 16; // rows r, r+1 in different bank halves
    constexpr int PITCH_B = PITCH_DW * 4;
    constexpr bool CAN_STAGE = !EDGE && (NT / 64) * 32 * PITCH_B <= Cfg::LDS_BYTES;
    // the wave's slab of 32 rows leaves as 16-byte pieces: rows i*32 .. i*32+31 of the wave tile
    auto stream_slab = [&](auto out_tag, const char* slab, int i) {
        constexpr int OS = sizeof(decltype(out_tag));
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        const CTile tile = c_tile(p, m0 + (wave_u / WAVES_N) * WTM, n0 + (wave_u % WAVES_N) * WTN, OS);
        const unsigned row_bytes = (unsigned)p.c_rs * OS;
        constexpr int CPRW = WTN * OS / 16;       // 16-byte pieces per row of the wave tile
        constexpr int PIECES = 32 * CPRW / 64;    // per lane and 32-row slab
        static_assert((32 * CPRW) % 64 == 0, "pieces divide evenly over the lanes");
#pragma unroll
        for (int it = 0; it < PIECES; ++it) {
            const int id = it * 64 + lane;
            const int row = id / CPRW, cc = id % CPRW;
            const i32x4 v = *(const i32x4*)(slab + row * PITCH_B + cc * 16);
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), tile.rsrc, (unsigned)row * row_bytes + cc * 16,
                                                   (unsigned)(i * 32) * row_bytes, C_STORE_AUX);
        }
    };
    // fp16 / bf16: two columns packed per dword after a swap with the neighbouring lane
    auto store_staged = [&](auto out_tag, auto relu_tag) {
        auto fin = [&](float v) { return decltype(relu_tag)::value ? (v > 0.f ? v : 0.f) : v; };
        using out_t = decltype(out_tag);
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        unsigned* slab = (unsigned*)(smem + wave_u * (32 * PITCH_B));
        const int odd = lane & 1;
        const int wrow = (lane >> 5) * 4 + odd, wcol = (lane & 31) >> 1;
        // (lo, hi) = (own row 2t, own row 2t+1) narrowed with round-to-nearest-even
        auto pack2 = [&](float lo, float hi) -> unsigned {
            if constexpr (std::is_same<out_t, _Float16>::value) {
                typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                return __builtin_bit_cast(unsigned, h2{(_Float16)lo, (_Float16)hi});
            } else {
                typedef __bf16 b2 __attribute__((ext_vector_type(2)));
                return __builtin_bit_cast(unsigned, b2{(__bf16)lo, (__bf16)hi});
            }
        };
        // even lane (column c):   row 2t   <- (own lo, neighbour lo) = columns c, c+1
        // odd lane  (column c+1): row 2t+1 <- (neighbour hi, own hi)
        const unsigned sel = odd ? 0x03020706u : 0x05040100u; // v_perm_b32: bytes 0-3 from own, 4-7 from neighbour
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const unsigned own = pack2(fin(acc[i][j][2 * t]), fin(acc[i][j][2 * t + 1]));
                    const unsigned nbr = (unsigned)__builtin_amdgcn_update_dpp(0, (int)own, 0xB1, 0xF, 0xF, true); // lane ^ 1
                    const int row = (t >> 1) * 8 + (t & 1) * 2 + wrow;
                    slab[row * PITCH_DW + j * 16 + wcol] = __builtin_amdgcn_perm(nbr, own, sel);
                }
            stream_slab(uint16_t{}, (const char*)slab, i);
        }
    };
    // int16 / int8: the low bits of the int32 sums, written into the slab at their row-major place
    auto store_staged_int = [&](auto out_tag) {
        using out_t = decltype(out_tag);
        constexpr int OS = sizeof(out_t);
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        char* slab = smem + wave_u * (32 * PITCH_B);
        const int srow = (lane >> 5) * 4, scol = lane & 31;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = (r >> 2) * 8 + (r & 3) + srow;
                    *(out_t*)(slab + row * PITCH_B + (j * 32 + scol) * OS) = (out_t)acc[i][j][r];
                }
            stream_slab(out_tag, slab, i);
        }
    };
    auto store_all = [&](auto relu_tag) {
        auto fin = [&](scalar_t v) { return decltype(relu_tag)::value ? (v > scalar_t(0) ? v : scalar_t(0)) : v; };
        const unsigned os = p.out_type == T_I8 ? 1 : (p.out_type == T_F32 || p.out_type == T_I32) ? 4 : 2;
        // (whole 16-byte pieces of rows: rows 16 bytes apart, and a tile -- a moved last one may start at any column when B is K-contiguous -- on a 16-byte boundary)
        const bool staged = CAN_STAGE && (p.c_rs * os) % 16 == 0 && ((size_t)p.C & 15) == 0 && ((unsigned)n0 * os) % 16 == 0;
        if constexpr (IN == IN_I8) {
            if (p.out_type == T_I32) for_each_element(int{}, [&](CTile t, unsigned vo, unsigned so, int v) { c_store<int, EDGE ? 0 : C_STORE_AUX>(t, vo, so, fin(v)); return v; });
            else if (CAN_STAGE && staged) {
                if constexpr (CAN_STAGE) {
                    __syncthreads(); // every wave is done reading the tile buffers
                    if (p.out_type == T_I16) store_staged_int(int16_t{});
                    else store_staged_int(int8_t{});
                }
            } else if (p.out_type == T_I16) for_each_element(int16_t{}, [&](CTile t, unsigned vo, unsigned so, int v) { c_store<int16_t>(t, vo, so, (int16_t)fin(v)); return v; });
            else for_each_element(int8_t{}, [&](CTile t, unsigned vo, unsigned so, int v) { c_store<int8_t>(t, vo, so, (int8_t)fin(v)); return v; });
        } else if (p.out_type == T_F32) for_each_element(float{}, [&](CTile t, unsigned vo, unsigned so, float v) { c_store<float, EDGE ? 0 : C_STORE_AUX>(t, vo, so, fin(v)); return v; });
        else if (CAN_STAGE && staged) {
            if constexpr (CAN_STAGE) {
                __syncthreads(); // every wave is done reading the tile buffers
                if (p.out_type == T_F16) store_staged(_Float16{}, relu_tag);
                else store_staged(uint16_t{}, relu_tag);
            }
        } else if (p.out_type == T_F16) for_each_element(_Float16{}, [&](CTile t, unsigned vo, unsigned so, float v) { c_store<_Float16>(t, vo, so, (_Float16)fin(v)); return v; }); // RNE
        else for_each_element(uint16_t{}, [&](CTile t, unsigned vo, unsigned so, float v) { c_store<uint16_t>(t, vo, so, float_to_bf16_bits(fin(v))); return v; });
    };
    // One straight line through the passes: splitting the fused matmul + ReLU case off into a
    // branch of its own makes the register allocator spill hundreds of accumulators.
    general_ops();
    __builtin_amdgcn_sched_barrier(0);
    store_all(std::false_type{});
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
hipError_t launch_mfma(const GemmArgs& a, hipStream_t stream, LaunchGeom* geom, bool dry_run)
{
    auto kern = gemm_mfma_kernel<Cfg>;
    // an int8 C is written in 16-byte pieces of 16-byte aligned rows; no kernel here has a path for anything else
    if (a.out_type == T_I8 && (a.c_rs % 16 || ((size_t)a.C & 15) || (a.batch > 1 && a.c_bs % 16))) return hipErrorInvalidValue;
    // fewer rows than one tile: only where the fills fetch A's last row for the missing ones (or the edge build tests every row)
    if (!Cfg::EDGE && a.M < Cfg::BM && !mfma_takes_short_m<Cfg>()) return hipErrorInvalidValue;
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
