// C ABI of the library (include/accera_mi355x_gemm.h): argument checking, kernel
// selection, the host-pointer path and the launch-geometry query.
#include "../../include/accera_mi355x_gemm.h"
#include "common.h"
#include "skinny.h"
#include "host_path.h"
#include <algorithm>
#include <cmath>
#include <vector>
#include "variants.h"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <utility>

using namespace acc950;

namespace {

thread_local std::string t_last_error;

int fail(int code, const std::string& msg)
{
    t_last_error = msg;
    return code;
}
int fail_hip(hipError_t e, const char* what)
{
    return fail(ACC950_HIP_ERROR, std::string(what) + ": " + hipGetErrorString(e));
}

int elem_size(int t)
{
    switch (t) {
    case T_F32: case T_I32: return 4;
    case T_F16: case T_BF16: case T_I16: return 2;
    case T_I8: return 1;
    default: return 0;
    }
}

bool type_pair_ok(int in, int out)
{
    if (in == T_I8) return out == T_I32 || out == T_I16 || out == T_I8;
    if (in == T_F32) return out == T_F32;
    if (in == T_F16 || in == T_BF16) return out == T_F32 || out == T_F16 || out == T_BF16;
    return false;
}

const MfmaVariant* mfma_table(int in_type, int* n)
{
    switch (in_type) {
    case T_F16: return mfma_variants_f16(n);
    case T_BF16: return mfma_variants_bf16(n);
    case T_I8: return mfma_variants_i8(n);
    case T_F32: return mfma_variants_f32(n);
    default: *n = 0; return nullptr;
    }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Problem after validation; C is made row-major by computing the transposed product
// C^T = B^T * A^T when the caller's C is column-major.
struct Problem {
    GemmArgs g;
    bool have_pointers;
};

// Batch of independent problems: count and element distance between consecutive A, B, C.
struct Batch {
    int count = 1;
    int64_t a_bs = 0, b_bs = 0, c_bs = 0;
};

int make_problem(int in_type, int out_type, int M, int N, int K,
                 const void* A, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_rs, int64_t b_cs,
                 void* C, int64_t c_rs, int64_t c_cs, int prologue, int epilogue, bool need_pointers, Problem* out,
                 double prologue_arg = 0.0, double epilogue_arg = 0.0, Batch batch = Batch())
{
    if (batch.count < 0 || batch.a_bs < 0 || batch.b_bs < 0 || batch.c_bs < 0) return fail(ACC950_INVALID_ARGUMENT, "negative batch count or stride");
    if (batch.count > 65535) return fail(ACC950_INVALID_ARGUMENT, "at most 65535 problems per batch");
    if (!type_pair_ok(in_type, out_type)) return fail(ACC950_INVALID_ARGUMENT, "unsupported input/output element type pair");
    if (M < 0 || N < 0 || K < 0) return fail(ACC950_INVALID_ARGUMENT, "negative matrix dimension");
    if (a_rs < 0 || a_cs < 0 || b_rs < 0 || b_cs < 0 || c_rs < 0 || c_cs < 0)
        return fail(ACC950_INVALID_ARGUMENT, "negative strides are not supported");
    if (prologue != PRO_NONE && prologue != PRO_SET && prologue != PRO_SCALE) return fail(ACC950_INVALID_ARGUMENT, "unknown prologue op");
    if (epilogue != EPI_NONE && epilogue != EPI_RELU && epilogue != EPI_RELU_NOCOND && epilogue != EPI_SCALE && epilogue != EPI_SET)
        return fail(ACC950_INVALID_ARGUMENT, "unknown epilogue op");
    if (prologue_arg != prologue_arg || epilogue_arg != epilogue_arg) return fail(ACC950_INVALID_ARGUMENT, "NaN op argument");
    if (need_pointers && M > 0 && N > 0 && (!C || (K > 0 && (!A || !B))))
        return fail(ACC950_INVALID_ARGUMENT, "null matrix pointer");
    GemmArgs g{};
    g.in_type = in_type; g.out_type = out_type;
    g.prologue = prologue; g.epilogue = epilogue;
    g.prologue_arg = prologue == PRO_NONE ? 0.f : (float)prologue_arg;
    g.epilogue_arg = (epilogue == EPI_SCALE || epilogue == EPI_SET) ? (float)epilogue_arg : 0.f;
    const bool transpose = c_cs != 1 && c_rs == 1 && N > 1;
    if (!transpose) {
        g.A = A; g.B = B; g.C = C; g.M = M; g.N = N; g.K = K;
        g.a_rs = a_rs; g.a_cs = a_cs; g.b_rs = b_rs; g.b_cs = b_cs; g.c_rs = c_rs; g.c_cs = c_cs;
    } else {
        g.A = B; g.B = A; g.C = C; g.M = N; g.N = M; g.K = K;
        g.a_rs = b_cs; g.a_cs = b_rs; g.b_rs = a_cs; g.b_cs = a_rs; g.c_rs = c_cs; g.c_cs = c_rs;
    }
    // (the kernels take these two strides as 32-bit arguments)
    if (g.a_cs > 0x7fffffffll || g.b_cs > 0x7fffffffll)
        return fail(ACC950_UNSUPPORTED, "the stride of A between consecutive k and the stride of B between consecutive columns must be below 2^31 elements");
    g.batch = batch.count;
    g.a_bs = transpose ? batch.b_bs : batch.a_bs;
    g.b_bs = transpose ? batch.a_bs : batch.b_bs;
    g.c_bs = batch.c_bs;
    if (batch.count == 0) g.M = 0; // nothing to do
    out->g = g;
    out->have_pointers = need_pointers;
    return ACC950_OK;
}

// ---- eligibility ------------------------------------------------------------------

bool mfma_can_take(const MfmaVariant& v, const Problem& pb)
{
    const GemmArgs& g = pb.g;
    if (!v.launch) return false; // (a place in the table this input type has no kernel for)
    if (g.M <= 0 || g.N <= 0 || g.K <= 0) return false;
    const int es = elem_size(g.in_type), vec = 16 / es, bk = v.kb / es;
    if (g.c_cs != 1) return false;                          // C row-major
    if (v.a_kc ? g.a_cs != 1 : g.a_rs != 1) return false;   // A with K contiguous (row-major) or M contiguous
    if (v.b_kc ? g.b_rs != 1 : g.b_cs != 1) return false;
    const int64_t lda = v.a_kc ? g.a_rs : g.a_cs, ldb = v.b_kc ? g.b_cs : g.b_rs;
    // (the any-shape edge kernels load unaligned chunks: no condition on leading dimensions, pointers or batch strides)
    if (!v.any) {
        if (lda % vec || ldb % vec) return false;
        if (pb.have_pointers && (!aligned16(g.A) || !aligned16(g.B))) return false;
        if (g.batch > 1 && (g.a_bs % vec || g.b_bs % vec)) return false; // every problem of the batch 16-byte aligned
    }
    // int8 outputs need rows of C that start 16 bytes apart: byte-wise stores to rows at odd distances
    // are switched off (that path faulted on the device in its first run and the cause is not known)
    if (g.out_type == T_I8) {
        if (g.c_rs % 16 || (g.batch > 1 && g.c_bs % 16)) return false;
        if (pb.have_pointers && !aligned16(g.C)) return false;
    }
    if (v.w4) {
        // every op, except that an int8 C is only written (SET prologue), never read
        const int os = elem_size(g.out_type);
        const bool lean = g.prologue == PRO_SET || os >= 2;
        if (!lean || g.K % bk || g.K < 4 * bk || (g.c_rs * os) % 16 || (g.batch > 1 && (g.c_bs * os) % 16)) return false;
        if (pb.have_pointers && !aligned16(g.C)) return false;
        // any M, N >= one tile: the last row / column of tiles is moved to end at M / N (its first column must still be
        // 16 bytes aligned in B's and C's rows); when C is read, the moved tile does not store what it shares with its neighbour
        if (g.M % v.bm && (g.M < v.bm || (!v.a_kc && g.M % vec))) return false;
        if (g.N % v.bn && (g.N < v.bn || g.N % vec || (g.N * os) % 16)) return false;
        if (g.K % bk) return false;
    }
    if (v.edge) {
        if (!v.any && (g.K % vec || (!v.b_kc && g.N % vec) || (!v.a_kc && g.M % vec))) return false;
    } else {
        if (!v.w4 && g.K % bk) return false;
        if (!v.w4) {
            // the 32x32-shape kernels move the last row / column of tiles to end at M / N when C is only written; the
            // eight-wave kernels on the 16x16 shapes take whole tiles only
            const int os = elem_size(g.out_type);
            const bool movable = !v.mi16 && g.prologue == PRO_SET;
            // (fewer rows than one tile has, A with K contiguous: the fills fetch A's last row for the missing ones,
            // and C's descriptor drops what comes of them -- any prologue, nothing overlaps)
            const bool short_m = g.M < v.bm && v.a_kc && v.direct && !v.mi16;
            if (g.M % v.bm && !short_m && (!movable || g.M < v.bm || (!v.a_kc && g.M % vec))) return false;
            // (a K-contiguous B has no row that the moved tile's first column could split, and a C of 16- or 32-bit elements
            // is then stored element by element where the tile does not start on a 16-byte boundary: any N -- the odd
            // vocabulary sizes of language-model heads, 4096x50257x4096 with B as the framework keeps it)
            const bool any_n = v.b_kc && os >= 2;
            if (g.N % v.bn && (!movable || g.N < v.bn || (!any_n && (g.N % vec || (g.N * os) % 16)))) return false;
        }
    }
    // offsets inside one output tile are 32-bit in the write-back
    if ((int64_t)v.bm * g.c_rs * 4 >= (1ll << 32)) return false;
    // per-lane global offsets of the direct fill are 32-bit
    if ((int64_t)(v.a_kc ? v.bm : bk) * lda * es >= (1ll << 31) || (int64_t)(v.b_kc ? v.bn : bk) * ldb * es >= (1ll << 31)) return false;
    return true;
}

bool skinny_can_take(const Problem& pb, int sv)
{
    const GemmArgs& g = pb.g;
    const SkinnyVariant& v = skinny_variant(sv);
    if (g.in_type != T_F16 && g.in_type != T_BF16 && !(g.in_type == T_I8 && v.i8)) return false;
    const int es = elem_size(g.in_type), vec = 16 / es; // elements per 16-byte piece
    const int k_step = skinny_k_step(v, g.in_type);
    if (g.M < 1 || g.M > v.max_m || g.N < vec || g.K < k_step) return false;
    if (g.a_cs != 1 || g.b_cs != 1 || g.c_cs != 1) return false;
    if (g.N % vec || g.K % k_step || g.b_rs % vec) return false;
    if (g.a_rs % (v.mfma ? vec : 2)) return false; // A pieces are fetched 16 (4) bytes at a time
    // per-lane offsets of the direct-to-LDS fills are 32-bit: inside one step of a wave for the MFMA family (every step has
    // its own 64-bit base, so B itself may be of any size), inside a workgroup's whole K range for the dot-product family
    const int64_t b_reach = (v.mfma ? (int64_t)k_step : (int64_t)g.K) * g.b_rs * es + (int64_t)g.N * es;
    if (b_reach >= (1ll << 32) || (int64_t)v.max_m * g.a_rs * es >= (1ll << 32)) return false;
    if (pb.have_pointers && (!aligned16(g.B) || (reinterpret_cast<uintptr_t>(g.A) & (v.mfma ? 15u : 3u)))) return false;
    if (g.batch > 1 && (g.b_bs % vec || g.a_bs % (v.mfma ? vec : 2))) return false;
    return true;
}

// First skinny variant that takes the problem (the table lists the MFMA family first, best
// first), or -1.
int auto_skinny_variant(const Problem& pb)
{
    for (int sv = 0; sv < skinny_num_variants(); ++sv)
        if (skinny_can_take(pb, sv)) return sv;
    return -1;
}

// ---- workspace of the skinny kernels' K split ------------------------------------------
// Partial sums (fp32) and one arrival counter per column block.  One workspace per (device, stream): launches on one
// stream run one after the other and may share it, launches on different streams may overlap and must not.  A
// workspace only grows, and an outgrown block stays allocated, because launches queued earlier may still be using
// it, until acc950_release_workspaces frees everything on an idle device.  The pointers are copied out while the
// lock is held.
struct Workspace {
    float* scratch = nullptr;
    size_t floats = 0;
    unsigned* counters = nullptr; // zero between launches: the kernels leave them so
    size_t n_counters = 0;
};
std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, Workspace> g_ws;
std::vector<std::pair<int, void*>> g_ws_retired; // (device, block) outgrown by its workspace: freed by acc950_release_workspaces
std::atomic<unsigned long long> g_device_allocations{0}; // hipMalloc calls made by the GEMM entry points (acc950_allocation_probe)

hipError_t workspace_for(hipStream_t stream, size_t floats, size_t counters, float** scratch, unsigned** cnt)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace& w = g_ws[std::make_pair(dev, stream)];
    if (floats > w.floats) {
        const size_t want = floats < (1u << 20) ? (1u << 20) : floats + floats / 2;
        float* p = nullptr;
        e = hipMalloc((void**)&p, want * sizeof(float));
        if (e != hipSuccess) return e;
        ++g_device_allocations;
        if (w.scratch) g_ws_retired.emplace_back(dev, (void*)w.scratch); // (left to the launches queued earlier)
        w.scratch = p;
        w.floats = want;
    }
    if (counters > w.n_counters) {
        const size_t want = counters < 4096 ? 4096 : counters + counters / 2;
        unsigned* p = nullptr;
        e = hipMalloc((void**)&p, want * sizeof(unsigned));
        if (e != hipSuccess) return e;
        ++g_device_allocations;
        e = hipMemset(p, 0, want * sizeof(unsigned));
        if (e != hipSuccess) { (void)hipFree(p); return e; }
        if (w.counters) g_ws_retired.emplace_back(dev, (void*)w.counters);
        w.counters = p;
        w.n_counters = want;
    }
    *scratch = w.scratch;
    *cnt = w.counters;
    return hipSuccess;
}

// ---- the workspace that is never allocated (acc950_gemm_ops_static) ------------------------
// Lives in the library's own device image: kStaticFloats partial sums followed by kStaticCounters arrival counters.
// Zero when the image is loaded; the kernels leave the counters zero.  Every GPU holds its own copy at its own
// address, looked up once per device.
constexpr size_t kStaticFloats = ACC950_STATIC_WORKSPACE_BYTES / sizeof(float) - 4096;
constexpr size_t kStaticCounters = 4096;
static __device__ __align__(256) float scratch[kStaticFloats + kStaticCounters];
constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
float* g_static_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (the array's name is only a host-side handle).
hipError_t static_workspace(float** ptr)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        g_static_ptr[dev] = (float*)p;
    }
    *ptr = g_static_ptr[dev];
    return hipSuccess;
}

int auto_skinny_splits(int variant, const GemmArgs& g)
{
    // One workgroup per column block streams all of K unless that leaves most CUs idle;
    // splitting K costs a trip through the scratch buffer, so it is only used to reach
    // about one workgroup per CU, with at least 256 k rows per slice.
    // (a batch is one launch: the column blocks of all its problems fill the chip together -- 128 problems of 8 x 128 x 4096
    // took 96.7 us in 16 slices each, which a single problem of that shape would want, and take a quarter of that unsplit)
    const int64_t all_blocks = (int64_t)skinny_column_blocks(variant, g.N) * (g.batch > 1 ? g.batch : 1);
    const int blocks = all_blocks > 4096 ? 4096 : (int)all_blocks;
    int splits = blocks >= 128 ? 1 : (256 + blocks - 1) / blocks;
    const int max_splits = g.K / 256 > 0 ? g.K / 256 : 1;
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    return splits;
}

// Automatic MFMA tile choice.  Cost of a candidate = rounds of workgroups over the 256 CUs
// x tile area (time per round), with two workgroups sharing a CU for the tiles whose LDS
// and register budget allows it; ties go to the larger tile (more reuse per byte fetched).
// Among equal tiles the ping-pong kernel with four 64-byte stages is preferred, then the
// others in table order; partial tiles only fit the edge kernel.
bool streamed_b(const Problem& pb, int64_t least_bytes);

// only_tile: 0, or the edge length of the (square) tiles to choose among.  short_rows: also the 64-row tiles with direct fills
// on fewer rows than they have, whatever the size of B.
int auto_mfma_variant(const Problem& pb, int only_tile = 0, bool short_rows = false)
{
    int n = 0;
    const MfmaVariant* tab = mfma_table(pb.g.in_type, &n);
    if (!tab) return -1;
    int best = -1;
    double best_cost = 0;
    int best_rank = 0;
    for (int i = 0; i < n; ++i) {
        const MfmaVariant& v = tab[i];
        if (only_tile && (v.bm != only_tile || v.bn != only_tile)) continue;
        if (!mfma_can_take(v, pb)) continue;
        // (a tile with direct fills on fewer rows than it has: taken only where B has at least 16 MB, see streamed_b_tile --
        // elsewhere the choices stand as the sweeps of the reference's lists found them, none of whose rows is of this kind)
        if (!v.edge && !v.w4 && pb.g.M < v.bm && !short_rows && !streamed_b(pb, (int64_t)16 << 20)) continue;
        // (the any-alignment form on 256 x 256 tiles pays where the K-contiguous operands' rows are 16 bytes aligned and the
        // odd size is N or M -- 4096x50257x4096 with a row-major B: 2397 us on 128 x 128 tiles, 1832 on these -- and loses
        // where every row of a K-contiguous operand starts unaligned: 4100^3 326 / 361, 1234x5678x4321 205 / 256)
        if (v.any && v.bm == 256) {
            const int vec_k = 16 / elem_size(pb.g.in_type);
            if ((v.a_kc && pb.g.a_rs % vec_k) || (v.b_kc && pb.g.b_cs % vec_k)) continue;
        }
        // (a batch is one launch: its problems' tiles fill the chip together)
        const int64_t tiles = (((int64_t)pb.g.M + v.bm - 1) / v.bm) * (((int64_t)pb.g.N + v.bn - 1) / v.bn) * (pb.g.batch > 1 ? pb.g.batch : 1);
        // 8- and 16-bit inputs: rounds of workgroups over the compute units, two side by side where the tile leaves room and
        // there are more tiles than units (a workgroup of the 4-wave kernels is bound by its own waits, so two run almost as
        // fast as one; 4096x2304x768 fp16: 576 tiles of 128x128 take 23.9 us, 144 of 256x256 18.9).  fp32, bound by its slow
        // MFMAs: what one unit has to get through, its share of the tiles one after the other (3072x1024x1024: 768 tiles of
        // 64x64, three per unit, 53 us; 192 of 128x128 on 192 units 66 us).
        const bool fp32 = pb.g.in_type == T_F32;
        const int64_t per_cu = (tiles + kComputeUnits - 1) / kComputeUnits;
        const int wgs_per_cu = ((fp32 ? per_cu >= 2 : tiles > kComputeUnits) && v.waves_m * v.waves_n <= 4 &&
                                2 * v.stages * (v.bm + v.bn) * v.kb <= 160 * 1024 && v.bm * v.bn <= 256 * 128) ? 2 : 1;
        const int64_t slots = (int64_t)kComputeUnits * wgs_per_cu;
        double rounds = (double)((tiles + slots - 1) / slots);
        // A last round that is not full costs less than a full one when K is long: the part is at its power limit there, and
        // the workgroups of a half-empty chip run at a higher clock (fp16, K = 4096, tiles of 256 x 256: 256 of them 97 us,
        // 192 78 us, 384 161 us, where whole rounds would say 97 and 194).  Half of the missing part is charged.
        if ((int64_t)pb.g.K * elem_size(pb.g.in_type) >= 4096 && tiles > slots) rounds = 0.5 * (rounds + (double)tiles / (double)slots);
        double cost = fp32 ? (double)per_cu * v.bm * v.bn : rounds * wgs_per_cu * v.bm * v.bn;
        if (v.edge) cost *= v.any ? 2.0 : 1.5;   // register-staged fill, bounds checks (unaligned chunks cost more requests)
        if (!v.direct) cost *= 1.2;
        // measured on sweeps: 4-wave tiles reach about 80 % of the ping-pong kernel's rate when two
        // workgroups share a CU and about 70 % when a workgroup has the CU to itself
        // (fp32, bound by the MFMA rate whatever the tile: the 4-wave tiles are level or ahead -- 6144x4608x8192 3.29 ms on
        // 128 x 128 tiles against 4.10 on the 256 x 256 ping-pong kernel, 50176x512x256 110 against 146 us)
        if (v.waves_m * v.waves_n <= 4 && !v.w4) cost /= fp32 ? (wgs_per_cu == 2 ? 1.1 : 1.0) : (wgs_per_cu == 2 ? 0.8 : 0.7);
        // smaller tiles fetch more bytes and read more fragments per MFMA
        // (measured, 64x64 against 128x128 tiles: fp32, bound by its slow MFMAs, 1024^3 20.7 against 63.7 us and 3072x1024x1024
        // 53 against 66; 8- and 16-bit inputs win while a CU has at most two of them -- fp16 1024^3 6.6 against 9.5 us,
        // 1536x1152x2048 14.4 against 17.0 -- and lose beyond: 3072x1024x1024 13.1 against 9.8, 2048^3 30.3 against 21.2)
        if (v.bm * v.bn <= 64 * 64) cost /= pb.g.in_type == T_F32 ? 1.0 : per_cu <= 2 ? 0.75 : 0.5;
        else if (v.bm * v.bn <= 128 * 64) cost /= 0.8;
        // rank inside one tile shape: ping-pong kb64 x4 > ping-pong others > 8-wave > 4-wave (kb64 x4 first)
        int rank = v.pingpong ? (v.kb == 64 && v.stages == 4 ? 8 : 6) : (v.waves_m * v.waves_n == 8 ? 4 : 2);
        if (!v.pingpong && v.kb == 64 && v.stages == 4) rank += 1;
        // one tile per CU at most: the deepest prefetch wins (four stages of 128 bytes of K; 2048^3: 21.8 against 25-26 us), where
        // more tiles than CUs want two workgroups per CU, which only the smaller stages leave room for; below 32 tiles of K the
        // four stages of 64 bytes are ahead (2048x2048x512 fp16: 7.5 against 8.2 us)
        if (!v.pingpong && v.direct && v.kb == 128 && v.stages == 4 && tiles <= kComputeUnits && (int64_t)pb.g.K * elem_size(pb.g.in_type) >= 4096) rank += 2;
        // 128 x 128 tiles, two workgroups per CU: two stages of 128 bytes of K are ahead of four of 64 (3072x2304x4096 fp16:
        // 59.8 against 69.6 us; 3072x2048x1024 19.2 against 22.0; 12544x512x1024 16.5 against 17.9)
        if (!v.pingpong && v.direct && v.kb == 128 && v.stages == 2 && v.bm == 128 && v.bn == 128 && tiles > kComputeUnits &&
            (int64_t)pb.g.K * elem_size(pb.g.in_type) >= 1024) rank += 2;
        // 16x16 shapes: measured 4-9 % faster than the 32x32 shapes on every large problem, in the lean build
        // (C = A*B, C = relu(A*B)); their full build reads C element by element and lost 20 % to the 32x32 form
        const bool lean = pb.g.prologue == PRO_SET && pb.g.prologue_arg == 0.f && (pb.g.epilogue == EPI_RELU || pb.g.epilogue == EPI_NONE);
        if (v.mi16) rank += lean ? 4 : -8;
        // four waves with 128x128 wave tiles: measured 3-9 % faster than the eight-wave form on large problems
        // (a third less LDS traffic, and the part is at its power limit there)
        // (walking several tiles per workgroup pays when there is more than one round of tiles over the CUs)
        // (a column-major A: the two forms measured level -- 8192^3 tA fp16 774 against 784 us, int8 393 against 391,
        // 8192 x 8192 x 4096 410 against 407 -- and the one-tile form stays the choice)
        if (v.w4) rank = v.persist ? (v.a_kc && tiles / (pb.g.batch > 1 ? pb.g.batch : 1) > kComputeUnits ? 14 : 12) : 13; // (tiles of one problem: a workgroup walks inside its own)
        const bool better = best < 0 || cost < best_cost * 0.999 ||
                            (cost <= best_cost * 1.001 && ((int64_t)v.bm * v.bn > (int64_t)tab[best].bm * tab[best].bn ||
                                                           ((int64_t)v.bm * v.bn == (int64_t)tab[best].bm * tab[best].bn && rank > best_rank)));
        if (better) { best = i; best_cost = cost; best_rank = rank; }
    }
    return best;
}

// ---- K split of an MFMA variant: the kernel runs as a batch of partial products over consecutive ranges of K into a
// workspace of 32-bit sums, and a second kernel adds the slices in order and does the prologue / epilogue ops
// (gemm_splitk.hip).  Every slice but the last spans `ks` elements of K (whole K tiles), the last what is left.
struct SplitPlan {
    int splits, ks, k_last;
};
constexpr size_t kMaxSplitFloats = (size_t)1 << 28; // 1 GiB of partial sums

GemmArgs split_first_step(const GemmArgs& g, const SplitPlan& sp, void* ws)
{
    GemmArgs q = g;
    q.C = ws;
    q.c_rs = g.N; q.c_cs = 1;
    q.out_type = g.in_type == T_I8 ? T_I32 : T_F32;
    q.prologue = PRO_SET; q.prologue_arg = 0.f;
    q.epilogue = EPI_NONE; q.epilogue_arg = 0.f;
    q.K = sp.ks; q.k_last = sp.k_last;
    q.batch = sp.splits;
    q.a_bs = (int64_t)sp.ks * g.a_cs; q.b_bs = (int64_t)sp.ks * g.b_rs; q.c_bs = (int64_t)g.M * g.N;
    return q;
}

// Slices for `want` splits of this problem on variant v (fewer when K has too few K tiles); false when the variant
// cannot run the problem split (a batch, one slice only, partial products it does not take).
bool plan_split(const MfmaVariant& v, const Problem& pb, int want, SplitPlan* sp, size_t max_floats = kMaxSplitFloats)
{
    const GemmArgs& g = pb.g;
    if (g.batch > 1 || want <= 1) return false;
    // (never more slices than the workspace at hand holds)
    const size_t per_slice = (size_t)g.M * (size_t)g.N;
    if (per_slice == 0 || max_floats / per_slice < 2) return false;
    if ((size_t)want > max_floats / per_slice) want = (int)(max_floats / per_slice);
    const int bk = v.kb / elem_size(g.in_type);
    const int kt = (g.K + bk - 1) / bk, least = v.w4 ? 4 : 1; // K tiles in all; K tiles a slice needs
    int splits = want < kt / least ? want : kt / least;
    if (splits <= 1) return false;
    const int per = (kt + splits - 1) / splits;
    splits = (kt + per - 1) / per;
    if (splits > 1 && g.K - (splits - 1) * per * bk < least * bk) --splits; // (the last slice takes what a too short one would have left)
    if (splits <= 1) return false;
    if ((size_t)splits * per_slice > max_floats) return false;
    sp->splits = splits;
    sp->ks = per * bk;
    sp->k_last = g.K - (splits - 1) * sp->ks;
    Problem q{split_first_step(g, *sp, nullptr), pb.have_pointers};
    if (!mfma_can_take(v, q)) return false;
    q.g.K = sp->k_last;
    return mfma_can_take(v, q);
}

// Splits the library takes by itself: only when the tiles leave at least half of the compute units idle and K is long
// enough for the second kernel (a few microseconds) to pay.  Measured on small outputs with a long K (512 x 512 x 8192,
// 256 x 256 x 16384, 1024 x 1024 x 4096, 768 x 320 x 30522, 1024 x 80 x 30522; 16-bit inputs): the best split fills the
// compute units once or twice and leaves a slice 4 to 60 k-steps of 64 bytes.
int auto_mfma_splits(const MfmaVariant& v, const Problem& pb, size_t max_floats = kMaxSplitFloats)
{
    const GemmArgs& g = pb.g;
    if (g.batch > 1) return 1;
    const int64_t tiles = (((int64_t)g.M + v.bm - 1) / v.bm) * (((int64_t)g.N + v.bn - 1) / v.bn);
    if (tiles * 2 > kComputeUnits) return 1;
    // K in steps of 64 bytes, and in units of 0.1 us: what such a step costs a 64 x 64 tile with direct fills.  The
    // register-staged kernels take about three times as long per step, a 128 x 128 tile about twice and a 256 x 256 tile
    // about five times as long as a 64 x 64 one, fp32 twice as long as the 8- and 16-bit types.
    const int64_t area = (int64_t)v.bm * v.bn;
    const int64_t steps = (int64_t)g.K * elem_size(g.in_type) / 64;
    const int64_t worth = steps * (v.direct ? 1 : 3) * (area <= 64 * 64 ? 1 : area <= 128 * 128 ? 2 : 4) * (g.in_type == T_F32 ? 2 : 1);
    // The second kernel costs 3 to 5 us: a K worth less than 48 units only loses by a split, however few the tiles (launches
    // back to back from a C++ loop, fp16, 64 x 64 tiles, unsplit / split in us -- direct: 64x1536x256 4.1 / 6.7; 256^3
    // 5.0 / 7.7; 64x320x1728 8.4 / 7.4; 576x192x3136 11.9 / 7.9; register-staged: 196x48x400 6.6 / 8.3; 6272x32x512
    // 7.3 / 8.8; 512x32x196 with a column-major A 7.2 / 9.3; 196x64x800 8.5 in four slices, 7.8 in six; int8 363x64x3025
    // 46.9 / 10.8).
    if (worth < 48) return 1;
    // Slices of about 32 k-steps; shorter ones, down to 4, while that keeps the workgroups at or below one per compute unit;
    // never more workgroups than the compute units hold at once (two of the 64 x 64 tiles each), never more than 32 slices.
    // Measured with 64 x 64 tiles, fp16, us by slices 4 / 8 / 16 / 32: 768x320x30522 84 / 53 / 49 / 53; 1024x80x30522
    // 81 / 49 / 33 / 36; 288x64x21609 61 / 35 / 22 / 16; 363x64x3025 16 / 11 / 10 / 11; 576x96x5329 18 / 13 / 12 / 14;
    // 512x512x8192 15 / 15 / 18 / 25; 256x256x16384 22 / 15 / 15 / 17; 384x96x1225 7.9 / 6.9 / 7.2 / 6.9.
    const int64_t slots = kComputeUnits * (v.bm * v.bn <= 64 * 64 ? 2 : 1);
    const int64_t few = steps / 4 < kComputeUnits / tiles ? steps / 4 : kComputeUnits / tiles;
    int64_t want = steps / 32 > few ? steps / 32 : few;
    if (want > slots / tiles) want = slots / tiles;
    if (want > 32) want = 32;
    if ((size_t)want * (size_t)g.M * (size_t)g.N > ((size_t)1 << 24)) return 1; // 64 MiB of partial sums at most without being asked
    // What the slices save against what the second kernel costs, 3.5 us and 0.65 us per MB of partial sums written and read
    // (2048x256x1536 on 128 tiles: 8.2 us unsplit, 10.7 in two slices with their 4 MB; 2048x448x2048: 10.0 / 13.9).
    if (want > 1 && (double)worth * (double)(want - 1) / (double)want < 35.0 + 6.5e-6 * 4.0 * (double)want * (double)g.M * (double)g.N) return 1;
    SplitPlan sp;
    return want > 1 && plan_split(v, pb, (int)want, &sp, max_floats) ? sp.splits : 1;
}

// A few dozen to a few hundred rows of A against a B far larger than the caches (prefill of a short prompt, a batch of decode
// steps): the problem is a stream of B out of HBM, and what counts is that B is streamed once -- a tile as tall as A, so
// that no second row of tiles fetches it again -- by enough workgroups to keep the memory system busy, which takes a K
// split where the tiles are few.  The general rule above knows neither: it weighs MFMA work, takes 64 x 64 tiles for
// 128 x 16384 x 16384 (512 of them: B is read twice; 181 us) where 128 x 128 tiles in two slices take 106, and never
// splits more tiles than half the CUs.  Swept over M = 33 ... 256 x (N, K) = (8192, 28672) ... (65536, 4096), fp16, every
// tile and 1 ... 32 slices (us, general rule / this rule's choice): 33x8192x28672 231 / 94, 64x16384x16384 111 / 111,
// 96x28672x8192 167 / 110, 128x8192x28672 174 / 98, 128x16384x16384 181 / 106, 192x8192x28672 250 / 152, 256x8192x28672
// 288 / 135.  The best forms have about 256 workgroups with direct fills and about 512 with register-staged ones.
// Returns the tile edge to choose among (0: the general rule) and the number of workgroups to aim for.
// (The tile only for a B of 192 MB and more, most of the 256 MB Infinity Cache, out of which a second pass over B costs little; the
// slices from 64 MB on -- 16 MB with fewer than 64 rows --, whatever tile the general rule takes: 33x11008x4096, 90 MB, 44.5 us on
// 172 unsplit 64 x 64 tiles, 22.3 in four slices.)
bool streamed_b(const Problem& pb, int64_t least_bytes)
{
    const GemmArgs& g = pb.g;
    // (up to 32 rows the streaming kernels come first; this is for what they do not take: a column-major B or A)
    return g.batch <= 1 && g.in_type != T_F32 && g.M <= 256 && (int64_t)g.N * g.K * elem_size(g.in_type) >= least_bytes;
}

int streamed_b_tile(const Problem& pb)
{
    const GemmArgs& g = pb.g;
    if (!streamed_b(pb, (int64_t)192 << 20)) return 0;
    // (a tile that holds all rows of A: up to 64 rows the small tiles, up to 128 rows the 128 x 128 tiles, up to 256 the
    // 256 x 256 ones; with direct fills all take fewer rows than they have when A is row-major (the four-wave kernel, which
    // moves its last row of tiles instead, only from 256 rows on), else the register-staged edge forms apply -- of which
    // the caller prefers the 128 x 128 one -- or, beyond 128 rows, the general rule)
    return g.M <= 64 ? 64 : g.M <= 128 ? 128 : 256;
}

// K slices for the tile the rule above has taken: about 256 workgroups for the direct-fill kernels of the larger tiles (one
// workgroup per CU), about 512 for the 64 x 64 tiles and the register-staged kernels (two per CU, fewer bytes in flight
// each), a power of two, none from 160 tiles on with direct fills; a slice keeps at least 1024 elements of K, and the
// partial sums (written and read once more) stay below a sixth of B's bytes (256x32000x4096: 74 us unsplit, 87 in two
// slices with their 65 MB; 256x28672x8192 in two slices 132 against 165).
int streamed_b_splits(const MfmaVariant& v, const Problem& pb, size_t max_floats)
{
    const GemmArgs& g = pb.g;
    const int64_t tiles = (((int64_t)g.M + v.bm - 1) / v.bm) * (((int64_t)g.N + v.bn - 1) / v.bn);
    if (v.direct && tiles >= 160) return 1;
    const int64_t target = v.direct && v.bm * v.bn > 64 * 64 ? kComputeUnits : 2 * kComputeUnits;
    int64_t want = 1;
    while (want * 2 * tiles <= target && want < 32) want *= 2;
    const int64_t b_bytes = (int64_t)g.N * g.K * elem_size(g.in_type);
    while (want > 1 && (g.K / want < 1024 || want * (int64_t)g.M * g.N * 4 > b_bytes / 6)) want /= 2;
    if (want < 2) return 1;
    if ((size_t)want * (size_t)g.M * (size_t)g.N > ((size_t)1 << 24)) return 1; // 64 MiB of partial sums at most without being asked
    SplitPlan sp;
    return plan_split(v, pb, (int)want, &sp, max_floats) ? sp.splits : 1;
}

struct Choice {
    int variant;
    int splits;
};

// Few rows of A, a large B (decode shapes with a long K or many columns): the 256-column blocks of the streaming kernel
// against its 64-column default.  A 64-column block fetches B in pieces of one cache line (half a line for int8), and
// the memory system delivers such pieces at 5.0-5.3 TB/s (int8: 3.8-4.4) however many workgroups ask for them; 256-column
// blocks fetch 512 (256) bytes of a row per request and reach 6.2-6.6 (5.9), but there are a quarter as many of them, one
// workgroup at a time per CU (its rings fill the LDS), so they need a K split to occupy the chip while there are fewer
// than about 150, and the split's second trip through memory (5-11 us, more with more rows) has to be worth it.  Measured
// on grids of N = 4096 ... 128256 x K = 2048 ... 53248 for 8, 16 and 32 rows, fp16 and int8, B out of HBM (fp16, 8 rows, us,
// 64-column default / best 256-column form): 8x16384x8192 54.4 / 47.4 in three slices, 8x22016x8192 97.4 / 65.7 in two,
// 8x65536x8192 216.6 / 176.3 unsplit, 8x128256x8192 394.2 / 338.9; int8 8x12288x16384 69.2 / 42.2 in four, 8x65536x16384
// 285.2 / 185.7; while the default stays ahead for N <= 12288 with fp16 (8x11008x4096 18.0 / 22.1) and for a short K.
// Over the grids the default alone took 1.14 (fp16, 8 rows) to 1.39 (int8) times the best form's time on average, this rule 1.01-1.03.
// splits: what the 256-column form should run with; false: stay with the default.
bool wide_skinny_blocks_pay(const Problem& pb, int sv_wide, size_t max_floats, size_t max_counters, int* splits)
{
    const GemmArgs& g = pb.g;
    if (g.batch > 1) return false;
    const bool i8 = g.in_type == T_I8;
    const int nb = (g.N + 255) / 256, nb_narrow = (g.N + 63) / 64;
    if ((size_t)nb > max_counters) return false;
    // with a split: only where the default has no idle CUs to share its slow blocks with (fp16, bf16: more than 200 blocks
    // of 64 columns) or streams half lines (int8, from 32 blocks of 256 columns), the slices stay long enough for the
    // second trip to be worth it, and the workgroups fill most of the chip in one round
    if (nb <= 128 && (i8 ? nb >= 32 : nb_narrow > 200)) {
        const int k_min = g.M <= 8 ? 2048 : 4096;
        const int w_min = i8 && nb <= 40 ? 128 : 160;
        for (int s : {8, 6, 4, 3, 2}) {
            if (nb * s > kComputeUnits || g.K / s < k_min) continue;
            if (nb * s < w_min || skinny_scratch_floats(sv_wide, g.N, s) > max_floats) break;
            *splits = s;
            return true;
        }
    }
    // unsplit, from about a hundred blocks: whole rounds of 256 blocks at the chip's rate for wide pieces and a last partial
    // round (W blocks on W CUs reach less: 64 of them 3.2 TB/s, 125 5.5, 160 5.6, 208 6.0; never shorter than one block at a
    // CU's rate), against all of B at the rate of the narrow pieces, which also loses what its last round of 256 blocks
    // lacks (344 narrow blocks: 3.7 TB/s, 513: 3.8, 640: 4.3; less so from three rounds on, where workgroups of different
    // rounds share CUs).  Rates in millions of bytes per us.
    if (nb < 100 || g.K < 1024) return false;
    const double chip_wide = i8 ? 5.9 : 6.3, cu_wide = i8 ? 0.042 : 0.050, chip_narrow = i8 ? 4.2 : 5.3;
    const int full = nb / kComputeUnits, rem = nb % kComputeUnits;
    const double rem_rate = std::min(rem * cu_wide, chip_wide * (0.75 + 0.25 * rem / kComputeUnits));
    const double t_wide = full * kComputeUnits / chip_wide + (rem ? std::max(rem / rem_rate, 1.0 / cu_wide) : 0.0);
    const double rounds = (double)nb_narrow / kComputeUnits;
    double lost = std::ceil(rounds) / rounds;
    if (rounds > 3) lost = 1 + 0.5 * (lost - 1);
    if (t_wide >= 0.92 * (nb / chip_narrow * lost)) return false;
    *splits = 1;
    return true;
}

// max_split_floats: 32-bit partial sums the workspace of this call holds (the built-in array of acc950_gemm_ops_static
// is smaller than what the allocating entry points may ask for): an MFMA kernel's K split never plans more slices.
int choose(const Problem& pb, int variant, int k_splits, Choice* c, size_t max_split_floats = kMaxSplitFloats, size_t max_counters = ~(size_t)0)
{
    c->splits = 1;
    if (variant == ACC950_VARIANT_AUTO) {
        const int sv = auto_skinny_variant(pb);
        if (sv >= 0) {
            c->variant = ACC950_VARIANT_SKINNY_BASE + sv;
            c->splits = k_splits > 0 ? k_splits : auto_skinny_splits(sv, pb.g);
            // A batch of problems with few rows and a narrow B (rows of B of at most 512 bytes: the P x V product of a decode
            // step's attention, 8 x 128 x 4096 per head): the streaming kernels' pieces of such short rows come in slowly
            // (128 problems: 59.7 us, 2.3 TB/s), the 64 x 64 tiles with direct fills, which take fewer rows than a tile
            // has, stream whole rows (22.6 us, the vendor library's batched call 22.6; 256 problems of 1 x 128 x 8192: 207 /
            // 87.7 / 94.9) -- when the batch has enough tiles for the chip, as a batch is not split over K.
            if (k_splits == 0 && pb.g.batch > 1 && pb.g.N <= 256 && pb.g.N * elem_size(pb.g.in_type) <= 512) {
                const int mv = auto_mfma_variant(pb, 64, true);
                int n = 0;
                const MfmaVariant* tab = mfma_table(pb.g.in_type, &n);
                if (mv >= 0 && tab[mv].direct && (int64_t)((pb.g.N + 63) / 64) * pb.g.batch >= kComputeUnits / 2) {
                    c->variant = mv;
                    c->splits = 1;
                    return ACC950_OK;
                }
            }
            // (the table's first entry is the MFMA family's 64-column form, kSkinnyWide its 256-column one)
            int wide_splits = 1;
            if (k_splits == 0 && sv == 0 && skinny_can_take(pb, kSkinnyWide) && wide_skinny_blocks_pay(pb, kSkinnyWide, max_split_floats, max_counters, &wide_splits)) {
                c->variant = ACC950_VARIANT_SKINNY_BASE + kSkinnyWide;
                c->splits = wide_splits;
            }
            return ACC950_OK;
        }
        int mv = -1, streamed_splits = 0;
        if (k_splits == 0) {
            if (const int tile = streamed_b_tile(pb)) {
                mv = auto_mfma_variant(pb, tile);
                if (tile == 64 && pb.g.M < 64) { // (33x16384x16384: 102 us on 128 x 128 edge tiles, 110 on the 64 x 64 ones)
                    int n = 0;
                    if (mv < 0 || !mfma_table(pb.g.in_type, &n)[mv].direct) mv = auto_mfma_variant(pb, 128);
                }
                if (mv >= 0) {
                    int n = 0;
                    const MfmaVariant& v = mfma_table(pb.g.in_type, &n)[mv];
                    streamed_splits = streamed_b_splits(v, pb, max_split_floats);
                    // (too few workgroups to stream with, and no split to make more: the general rule's smaller tiles)
                    const int64_t tiles = (((int64_t)pb.g.M + v.bm - 1) / v.bm) * (((int64_t)pb.g.N + v.bn - 1) / v.bn);
                    if (tiles * streamed_splits < 100) { mv = -1; streamed_splits = 0; }
                }
            }
        }
        if (mv < 0) mv = auto_mfma_variant(pb);
        if (pb.g.in_type == T_F32 && f32_can_take(pb.g)) {
            // fp32: the kernel of 32 x 32 blocks against the LDS-tiled kernels.  The kernel of blocks is ahead while its blocks
            // are at most one round over the chip and K is short (sweep of the reference's 339 shapes: best on 81 of the 86
            // problems with up to 256 blocks and K <= 640 -- 512^3 7.5 us against 8.9 to 10.4, 256x1024x196 with a
            // column-major A 4.8 against 10.6 -- and on 6 of the 74 with a longer K, where the tiled kernels split K:
            // 64x192x1728 9.9 us in 16 slices against 18.5); with more blocks the tiled kernels with direct fills win
            // (768x576x1024: 17.1 in four slices against 26.3; 2048x192x1280: 17.3 against 27.4).  Against the
            // register-staged tiled kernels (unaligned operands) the kernel of blocks also wins with a K up to 768, and with a
            // longer one while the tiles x K slices leave half of the chip idle.
            int slices = 1;
            if (mv >= 0) {
                int n = 0;
                const MfmaVariant& v = mfma_table(pb.g.in_type, &n)[mv];
                SplitPlan sp;
                slices = k_splits > 1 ? (plan_split(v, pb, k_splits, &sp, max_split_floats) ? sp.splits : 1) : k_splits == 0 ? auto_mfma_splits(v, pb, max_split_floats) : 1;
                const int64_t tiles = (((int64_t)pb.g.M + v.bm - 1) / v.bm) * (((int64_t)pb.g.N + v.bn - 1) / v.bn);
                // (or more workgroups than there are 32 x 32 blocks: a small output with a long K, which only the tiled kernels split)
                const int64_t blocks = (((int64_t)pb.g.M + 31) / 32) * (((int64_t)pb.g.N + 31) / 32);
                const bool one_round = blocks <= kComputeUnits && pb.g.K <= 640;
                // (against the register-staged kernels a short K is enough: 2304x256x196 with a column-major A, 576 blocks,
                // 8.4 against 14.1 us; 4608x512x49, 2304 blocks, 16.8 against 19.0; but 1728x192x1225 24.1 against 19.8)
                if (one_round || (!v.direct && (pb.g.K <= 768 || (tiles * slices * 2 < kComputeUnits && tiles * slices <= blocks)))) mv = -1;
            }
            if (mv < 0) { c->variant = ACC950_VARIANT_F32_MFMA; return ACC950_OK; }
        }
        c->variant = mv >= 0 ? mv : ACC950_VARIANT_GENERIC;
        if (mv >= 0) {
            int n = 0;
            const MfmaVariant& v = mfma_table(pb.g.in_type, &n)[mv];
            SplitPlan sp;
            if (k_splits > 1) c->splits = plan_split(v, pb, k_splits, &sp, max_split_floats) ? sp.splits : 1;
            else if (k_splits == 0) {
                // (from 64 MB of B on; with fewer than 64 rows, where the tiles with direct fills on short rows come into play and
                // the general rule never splits more tiles than half the CUs, from 16 MB: 33x4096x4096 17.1 -> 10.8 us in four
                // slices, 8x11008x2048 with a K-contiguous B 22.8 -> 10.6 on direct fills; with 64 rows and more the smaller
                // problems keep the general rule's slices -- 64x8192x2048 10.9 us unsplit, 12.7 in two)
                if (!streamed_splits && streamed_b(pb, (int64_t)(pb.g.M < 64 ? 16 : 64) << 20)) streamed_splits = streamed_b_splits(v, pb, max_split_floats);
                c->splits = streamed_splits > 1 ? streamed_splits : auto_mfma_splits(v, pb, max_split_floats);
            }
        }
        return ACC950_OK;
    }
    if (variant == ACC950_VARIANT_GENERIC) { c->variant = variant; return ACC950_OK; }
    if (variant == ACC950_VARIANT_F32_MFMA) {
        if (!f32_can_take(pb.g)) return fail(ACC950_UNSUPPORTED, "the fp32 MFMA kernel needs fp32 inputs and K > 0");
        c->variant = variant;
        return ACC950_OK;
    }
    if (variant >= ACC950_VARIANT_SKINNY_BASE && variant < ACC950_VARIANT_SKINNY_BASE + skinny_num_variants()) {
        const int sv = variant - ACC950_VARIANT_SKINNY_BASE;
        if (!skinny_can_take(pb, sv))
            return fail(ACC950_UNSUPPORTED, "skinny kernel needs row-major A/B/C, rows of B in whole 16-byte pieces, and M <= 32, K a multiple of 32 bytes, 8- or 16-bit inputs (MFMA family) "
                                            "or M <= 8, K % 2 == 0, 16-bit inputs (dot-product family)");
        c->variant = variant;
        c->splits = k_splits > 0 ? k_splits : auto_skinny_splits(sv, pb.g);
        const int max_splits = pb.g.K / skinny_k_step(skinny_variant(sv), pb.g.in_type);
        if (c->splits > max_splits) c->splits = max_splits;
        return ACC950_OK;
    }
    int n = 0;
    const MfmaVariant* tab = mfma_table(pb.g.in_type, &n);
    if (variant < 0 || variant >= n) return fail(ACC950_INVALID_ARGUMENT, "unknown kernel variant");
    if (!mfma_can_take(tab[variant], pb)) return fail(ACC950_UNSUPPORTED, "MFMA variant cannot take this shape / layout / alignment");
    c->variant = variant;
    if (k_splits > 1) { // (a named variant is split only when asked)
        SplitPlan sp;
        if (!plan_split(tab[variant], pb, k_splits, &sp, max_split_floats))
            return fail(ACC950_UNSUPPORTED, "this MFMA variant cannot run the problem with K split (a batch, too few K tiles, partial products it does not take, or slices the workspace does not hold)");
        c->splits = sp.splits;
    }
    return ACC950_OK;
}

// static_ws: the K-split workspace is the one in the library's own device image; nothing is allocated
int run(const Problem& pb, const Choice& c, hipStream_t stream, LaunchGeom* geom, bool dry_run, bool static_ws = false)
{
    const GemmArgs& g = pb.g;
    if (g.M == 0 || g.N == 0) {
        if (geom) std::memset(geom, 0, sizeof(*geom));
        return ACC950_OK;
    }
    hipError_t e;
    if (c.variant == ACC950_VARIANT_GENERIC) {
        e = launch_generic(g, stream, geom, dry_run);
    } else if (c.variant == ACC950_VARIANT_F32_MFMA) {
        e = launch_f32(g, stream, geom, dry_run);
    } else if (c.variant >= ACC950_VARIANT_SKINNY_BASE) {
        const int sv = c.variant - ACC950_VARIANT_SKINNY_BASE;
        SkinnyArgs s{};
        s.A = g.A; s.B = g.B; s.C = g.C; s.M = g.M; s.N = g.N; s.K = g.K;
        s.a_rs = g.a_rs; s.b_rs = g.b_rs; s.c_rs = g.c_rs;
        s.in_type = g.in_type; s.out_type = g.out_type; s.prologue = g.prologue; s.epilogue = g.epilogue;
        s.prologue_arg = g.prologue_arg; s.epilogue_arg = g.epilogue_arg;
        s.splits = c.splits;
        s.batch = g.batch; s.a_bs = g.a_bs; s.b_bs = g.b_bs; s.c_bs = g.c_bs;
        s.extra_phase = -1;
        // 64-column MFMA blocks, no K split, dense rows of a multiple of 512 bytes: blocks whose
        // 128-byte lines have address bits 8:7 = 11 stream ~25 % slower (measured), so they are
        // shared by two workgroups each; the otherwise idle CUs take the second halves.
        const SkinnyVariant& skv = skinny_variant(sv);
        // (Which blocks those are follows B's address.  A query without pointers reports phase 0: no phase has more blocks,
        // so the grid it names is what launches or one workgroup more.)
        if (skv.mfma && skv.cols == 64 && g.in_type != T_I8 && c.splits == 1 && (g.b_rs * 2) % 512 == 0 &&
            skinny_column_blocks(sv, g.N) >= 128 && skinny_column_blocks(sv, g.N) <= 200 && g.K >= 512 &&
            (g.batch <= 1 || (g.b_bs * 2) % 512 == 0))
            s.extra_phase = pb.have_pointers ? (int)((3u - (unsigned)(reinterpret_cast<uintptr_t>(g.B) >> 7)) & 3u) : 0;
        const int ws_splits = s.extra_phase >= 0 ? 2 : c.splits;
        if (!dry_run && ws_splits > 1) {
            const size_t nb = g.batch > 1 ? (size_t)g.batch : 1;
            s.scratch_bs = (int64_t)skinny_scratch_floats(sv, g.N, ws_splits);
            s.counter_bs = skinny_column_blocks(sv, g.N);
            const size_t floats = nb * (size_t)s.scratch_bs, counters = nb * (size_t)s.counter_bs;
            if (static_ws) {
                if (floats > kStaticFloats || counters > kStaticCounters)
                    return fail(ACC950_UNSUPPORTED, "this problem's K split needs " + std::to_string(floats * sizeof(float)) + " bytes of partial sums and " +
                                std::to_string(counters) + " counters; the built-in workspace holds " + std::to_string(kStaticFloats * sizeof(float)) +
                                " bytes and " + std::to_string(kStaticCounters) + " counters");
                float* base = nullptr;
                e = static_workspace(&base);
                if (e != hipSuccess) return fail_hip(e, "address of the built-in workspace");
                s.scratch = base;
                s.counters = (unsigned*)(base + kStaticFloats);
            } else {
                e = workspace_for(stream, floats, counters, &s.scratch, &s.counters);
                if (e != hipSuccess) return fail_hip(e, "workspace allocation");
            }
        }
        e = launch_skinny(sv, s, stream, geom, dry_run);
    } else {
        int n = 0;
        const MfmaVariant* tab = mfma_table(g.in_type, &n);
        // kernels with a lean build take C = A*B and C = relu(A*B) there, everything else in the full build
        const MfmaVariant& mv = tab[c.variant];
        const bool lean = g.prologue == PRO_SET && g.prologue_arg == 0.f && (g.epilogue == EPI_RELU || g.epilogue == EPI_NONE);
        SplitPlan sp;
        // (the choice was made for the workspace of this call: the same plan comes out again)
        const bool split = c.splits > 1 && plan_split(mv, pb, c.splits, &sp, static_ws ? kStaticFloats : kMaxSplitFloats);
        if (split) {
            float* ws = nullptr;
            if (!dry_run) {
                const size_t floats = (size_t)sp.splits * (size_t)g.M * (size_t)g.N;
                unsigned* unused = nullptr;
                if (static_ws) {
                    e = static_workspace(&ws);
                    if (e != hipSuccess) return fail_hip(e, "address of the built-in workspace");
                } else {
                    e = workspace_for(stream, floats, 0, &ws, &unused);
                    if (e != hipSuccess) return fail_hip(e, "workspace allocation");
                }
            }
            e = mv.launch(split_first_step(g, sp, ws), stream, geom, dry_run); // partial products: C = A*B, nothing else
            if (e == hipSuccess && !dry_run) e = launch_splitk_reduce(g, ws, sp.splits, stream);
        } else {
            e = (mv.launch_general && !lean ? mv.launch_general : mv.launch)(g, stream, geom, dry_run);
        }
    }
    if (e != hipSuccess) return fail_hip(e, "kernel launch");
    return ACC950_OK;
}

size_t extent_elems(int rows, int cols, int64_t rs, int64_t cs)
{
    if (rows <= 0 || cols <= 0) return 0;
    return (size_t)(1 + (int64_t)(rows - 1) * rs + (int64_t)(cols - 1) * cs);
}

} // namespace

extern "C" {

const char* acc950_last_error(void) { return t_last_error.c_str(); }

int acc950_init(int device_id)
{
    hipError_t e = hipSetDevice(device_id);
    if (e != hipSuccess) return fail_hip(e, "hipSetDevice");
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, device_id);
    if (e != hipSuccess) return fail_hip(e, "hipGetDeviceProperties");
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(ACC950_UNSUPPORTED, std::string("this library is built for gfx950 only, device is ") + prop.gcnArchName);
    float* ws = nullptr; // this device's copy of the built-in workspace, so that acc950_gemm_ops_static need not look it up
    e = static_workspace(&ws);
    if (e != hipSuccess) return fail_hip(e, "address of the built-in workspace");
    return ACC950_OK;
}

int acc950_gemm_ops(int in_type, int out_type, int M, int N, int K,
                    const void* A, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_rs, int64_t b_cs,
                    void* C, int64_t c_rs, int64_t c_cs, int prologue, double prologue_arg, int epilogue, double epilogue_arg,
                    int variant, int k_splits, void* stream)
{
    Problem pb;
    int rc = make_problem(in_type, out_type, M, N, K, A, a_rs, a_cs, B, b_rs, b_cs, C, c_rs, c_cs, prologue, epilogue, true, &pb,
                          prologue_arg, epilogue_arg);
    if (rc) return rc;
    Choice c;
    rc = choose(pb, variant, k_splits, &c);
    if (rc) return rc;
    return run(pb, c, (hipStream_t)stream, nullptr, false);
}

int acc950_gemm_ops_static(int in_type, int out_type, int M, int N, int K,
                           const void* A, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_rs, int64_t b_cs,
                           void* C, int64_t c_rs, int64_t c_cs, int prologue, double prologue_arg, int epilogue, double epilogue_arg,
                           int variant, int k_splits, void* stream)
{
    Problem pb;
    int rc = make_problem(in_type, out_type, M, N, K, A, a_rs, a_cs, B, b_rs, b_cs, C, c_rs, c_cs, prologue, epilogue, true, &pb,
                          prologue_arg, epilogue_arg);
    if (rc) return rc;
    Choice c;
    rc = choose(pb, variant, k_splits, &c, kStaticFloats, kStaticCounters);
    if (rc) return rc;
    return run(pb, c, (hipStream_t)stream, nullptr, false, true);
}

int acc950_gemm_batched(int in_type, int out_type, int batch, int M, int N, int K,
                        const void* A, int64_t a_bs, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_bs, int64_t b_rs, int64_t b_cs,
                        void* C, int64_t c_bs, int64_t c_rs, int64_t c_cs, int prologue, double prologue_arg, int epilogue,
                        double epilogue_arg, int variant, int k_splits, void* stream)
{
    Problem pb;
    Batch bt;
    bt.count = batch; bt.a_bs = a_bs; bt.b_bs = b_bs; bt.c_bs = c_bs;
    int rc = make_problem(in_type, out_type, M, N, K, A, a_rs, a_cs, B, b_rs, b_cs, C, c_rs, c_cs, prologue, epilogue, true, &pb,
                          prologue_arg, epilogue_arg, bt);
    if (rc) return rc;
    Choice c;
    rc = choose(pb, variant, k_splits, &c);
    if (rc) return rc;
    return run(pb, c, (hipStream_t)stream, nullptr, false);
}

// ---- bound calls: validate and choose once, launch many times -------------------------
struct BoundCall {
    Problem pb;
    Choice choice;
    hipStream_t stream;
    bool live;
};
std::mutex g_bound_mutex;
std::vector<BoundCall> g_bound;

int acc950_bind(int in_type, int out_type, int batch, int M, int N, int K,
                const void* A, int64_t a_bs, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_bs, int64_t b_rs, int64_t b_cs,
                void* C, int64_t c_bs, int64_t c_rs, int64_t c_cs, int prologue, double prologue_arg, int epilogue,
                double epilogue_arg, int variant, int k_splits, void* stream, int* handle)
{
    if (!handle) return fail(ACC950_INVALID_ARGUMENT, "null handle pointer");
    BoundCall bc{};
    Batch bt;
    bt.count = batch; bt.a_bs = a_bs; bt.b_bs = b_bs; bt.c_bs = c_bs;
    int rc = make_problem(in_type, out_type, M, N, K, A, a_rs, a_cs, B, b_rs, b_cs, C, c_rs, c_cs, prologue, epilogue, true, &bc.pb,
                          prologue_arg, epilogue_arg, bt);
    if (rc) return rc;
    rc = choose(bc.pb, variant, k_splits, &bc.choice);
    if (rc) return rc;
    bc.stream = (hipStream_t)stream;
    bc.live = true;
    std::lock_guard<std::mutex> lock(g_bound_mutex);
    for (size_t i = 0; i < g_bound.size(); ++i)
        if (!g_bound[i].live) { g_bound[i] = bc; *handle = (int)i; return ACC950_OK; }
    g_bound.push_back(bc);
    *handle = (int)g_bound.size() - 1;
    return ACC950_OK;
}

int acc950_launch(int handle)
{
    BoundCall bc;
    {
        std::lock_guard<std::mutex> lock(g_bound_mutex);
        if (handle < 0 || (size_t)handle >= g_bound.size() || !g_bound[handle].live) return fail(ACC950_INVALID_ARGUMENT, "unknown call handle");
        bc = g_bound[handle];
    }
    return run(bc.pb, bc.choice, bc.stream, nullptr, false);
}

int acc950_bound_choice(int handle, int* variant, int* k_splits)
{
    std::lock_guard<std::mutex> lock(g_bound_mutex);
    if (handle < 0 || (size_t)handle >= g_bound.size() || !g_bound[handle].live) return fail(ACC950_INVALID_ARGUMENT, "unknown call handle");
    if (variant) *variant = g_bound[handle].choice.variant;
    if (k_splits) *k_splits = g_bound[handle].choice.splits;
    return ACC950_OK;
}

int acc950_unbind(int handle)
{
    std::lock_guard<std::mutex> lock(g_bound_mutex);
    if (handle < 0 || (size_t)handle >= g_bound.size() || !g_bound[handle].live) return fail(ACC950_INVALID_ARGUMENT, "unknown call handle");
    g_bound[handle].live = false;
    return ACC950_OK;
}

int acc950_gemm_relu_ex(int in_type, int out_type, int M, int N, int K,
                        const void* A, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_rs, int64_t b_cs,
                        void* C, int64_t c_rs, int64_t c_cs, int prologue, int epilogue, int variant, int k_splits,
                        void* stream)
{
    return acc950_gemm_ops(in_type, out_type, M, N, K, A, a_rs, a_cs, B, b_rs, b_cs, C, c_rs, c_cs, prologue, 0.0, epilogue, 0.0,
                           variant, k_splits, stream);
}

int acc950_gemm_relu(int in_type, int out_type, int M, int N, int K,
                     const void* A, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_rs, int64_t b_cs,
                     void* C, int64_t c_rs, int64_t c_cs, int prologue, int epilogue, void* stream)
{
    return acc950_gemm_relu_ex(in_type, out_type, M, N, K, A, a_rs, a_cs, B, b_rs, b_cs, C, c_rs, c_cs, prologue, epilogue,
                               ACC950_VARIANT_AUTO, 0, stream);
}

int acc950_allocation_probe(unsigned long long* count)
{
    if (!count) return fail(ACC950_INVALID_ARGUMENT, "null output");
    *count = g_device_allocations.load();
    return ACC950_OK;
}

int acc950_release_workspaces(void)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail_hip(e, "hipGetDevice");
    e = hipDeviceSynchronize(); // nothing queued earlier still uses a block
    if (e != hipSuccess) return fail_hip(e, "hipDeviceSynchronize");
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    hipError_t first = hipSuccess;
    auto release = [&](void* p) { if (p) { hipError_t r = hipFree(p); if (r != hipSuccess && first == hipSuccess) first = r; } };
    for (auto it = g_ws.begin(); it != g_ws.end();) {
        if (it->first.first != dev) { ++it; continue; }
        release(it->second.scratch);
        release(it->second.counters);
        it = g_ws.erase(it);
    }
    for (auto it = g_ws_retired.begin(); it != g_ws_retired.end();) {
        if (it->first != dev) { ++it; continue; }
        release(it->second);
        it = g_ws_retired.erase(it);
    }
    if (first != hipSuccess) return fail_hip(first, "hipFree");
    // the host-pointer path's idle contexts: device copies of the largest operands they have carried, 16 MiB of pinned staging each
    e = host_path_release_idle(dev);
    if (e != hipSuccess) return fail_hip(e, "releasing the host-pointer path's buffers");
    return ACC950_OK;
}

int acc950_workspace_probe(void* stream, void** partial_sums, void** counters)
{
    if (!partial_sums || !counters) return fail(ACC950_INVALID_ARGUMENT, "null output");
    float* f = nullptr;
    unsigned* c = nullptr;
    hipError_t e = workspace_for((hipStream_t)stream, 1, 1, &f, &c);
    if (e != hipSuccess) return fail_hip(e, "workspace allocation");
    *partial_sums = f;
    *counters = c;
    return ACC950_OK;
}

int acc950_launch_geometry(int in_type, int out_type, int M, int N, int K,
                           int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t c_rs, int64_t c_cs,
                           int variant, int k_splits, unsigned grid[3], unsigned block[3], unsigned* dyn_lds, int* chosen)
{
    Problem pb;
    int rc = make_problem(in_type, out_type, M, N, K, nullptr, a_rs, a_cs, nullptr, b_rs, b_cs, nullptr, c_rs, c_cs,
                          PRO_SET0, EPI_NONE, false, &pb);
    if (rc) return rc;
    Choice c;
    rc = choose(pb, variant, k_splits, &c);
    if (rc) return rc;
    LaunchGeom geom{};
    rc = run(pb, c, nullptr, &geom, true);
    if (rc) return rc;
    for (int i = 0; i < 3; ++i) { if (grid) grid[i] = geom.grid[i]; if (block) block[i] = geom.block[i]; }
    if (dyn_lds) *dyn_lds = geom.dyn_lds;
    if (chosen) *chosen = c.variant;
    return ACC950_OK;
}

int acc950_gemm_relu_host(int in_type, int out_type, int M, int N, int K,
                          const void* A, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_rs, int64_t b_cs,
                          void* C, int64_t c_rs, int64_t c_cs, int prologue, int epilogue)
{
    return acc950_gemm_ops_host(in_type, out_type, M, N, K, A, a_rs, a_cs, B, b_rs, b_cs, C, c_rs, c_cs, prologue, 0.0, epilogue, 0.0);
}

int acc950_gemm_ops_host(int in_type, int out_type, int M, int N, int K,
                         const void* A, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_rs, int64_t b_cs,
                         void* C, int64_t c_rs, int64_t c_cs, int prologue, double prologue_arg, int epilogue, double epilogue_arg)
{
    return acc950_gemm_batched_host(in_type, out_type, 1, M, N, K, A, 0, a_rs, a_cs, B, 0, b_rs, b_cs, C, 0, c_rs, c_cs, prologue,
                                    prologue_arg, epilogue, epilogue_arg, ACC950_VARIANT_AUTO, 0);
}

int acc950_gemm_batched_host(int in_type, int out_type, int batch, int M, int N, int K,
                             const void* A, int64_t a_bs, int64_t a_rs, int64_t a_cs, const void* B, int64_t b_bs, int64_t b_rs,
                             int64_t b_cs, void* C, int64_t c_bs, int64_t c_rs, int64_t c_cs, int prologue, double prologue_arg,
                             int epilogue, double epilogue_arg, int variant, int k_splits)
{
    Problem check;
    Batch bt;
    bt.count = batch; bt.a_bs = a_bs; bt.b_bs = b_bs; bt.c_bs = c_bs;
    int rc = make_problem(in_type, out_type, M, N, K, A, a_rs, a_cs, B, b_rs, b_cs, C, c_rs, c_cs, prologue, epilogue, true, &check,
                          prologue_arg, epilogue_arg, bt);
    if (rc) return rc;
    if (M == 0 || N == 0 || batch == 0) return ACC950_OK;
    const size_t nb = (size_t)(batch - 1);
    const size_t a_elems = extent_elems(M, K, a_rs, a_cs), b_elems = extent_elems(K, N, b_rs, b_cs), c_elems = extent_elems(M, N, c_rs, c_cs);
    const size_t a_bytes = (a_elems ? nb * a_bs + a_elems : 0) * elem_size(in_type);
    const size_t b_bytes = (b_elems ? nb * b_bs + b_elems : 0) * elem_size(in_type);
    const size_t c_bytes = (nb * c_bs + c_elems) * elem_size(out_type);
    const bool c_dense = c_elems == (size_t)M * (size_t)N && (batch == 1 || (size_t)c_bs == c_elems);

    // Through pinned staging on a context of this call's own (host_path.hip): calls from different host threads do not
    // wait for each other.
    static const bool counted = (host_path_count_allocations(&g_device_allocations), true);
    (void)counted;
    HostOperands h{A, B, C, a_bytes, b_bytes, c_bytes, prologue != PRO_SET || !c_dense};
    int status = ACC950_OK;
    const hipError_t e = host_path_run(h, [&](void* dA, void* dB, void* dC, hipStream_t stream) {
        return acc950_gemm_batched(in_type, out_type, batch, M, N, K, dA, a_bs, a_rs, a_cs, dB, b_bs, b_rs, b_cs, dC, c_bs, c_rs, c_cs,
                                   prologue, prologue_arg, epilogue, epilogue_arg, variant, k_splits, stream);
    }, &status);
    if (status != ACC950_OK) return status; // (the launcher's own error text stands)
    if (e != hipSuccess) return fail_hip(e, "host-pointer path (allocation or copy)");
    return ACC950_OK;
}

int acc950_num_variants(void)
{
    int n = 0;
    mfma_variants_f16(&n);
    return n;
}

int acc950_num_skinny_variants(void) { return skinny_num_variants(); }

int acc950_variant_name(int variant, char* buf, size_t buf_len)
{
    if (!buf || buf_len == 0) return fail(ACC950_INVALID_ARGUMENT, "null buffer");
    if (variant == ACC950_VARIANT_GENERIC) {
        std::snprintf(buf, buf_len, "generic thread-bound 64x64 tile");
        return ACC950_OK;
    }
    if (variant == ACC950_VARIANT_F32_MFMA) {
        std::snprintf(buf, buf_len, "fp32 mfma 32x32 tile, K split over 4 waves");
        return ACC950_OK;
    }
    if (variant >= ACC950_VARIANT_SKINNY_BASE && variant < ACC950_VARIANT_SKINNY_BASE + skinny_num_variants()) {
        int lpr, waves, depth;
        skinny_variant_info(variant - ACC950_VARIANT_SKINNY_BASE, &lpr, &waves, &depth);
        std::snprintf(buf, buf_len, "skinny %s cols/wg=%d waves=%d depth=%d",
                      skinny_variant(variant - ACC950_VARIANT_SKINNY_BASE).mfma ? "mfma" : "dot2", lpr * 8, waves, depth);
        return ACC950_OK;
    }
    int n = 0;
    const MfmaVariant* tab = mfma_variants_f16(&n);
    if (variant < 0 || variant >= n) return fail(ACC950_INVALID_ARGUMENT, "unknown kernel variant");
    const MfmaVariant& v = tab[variant];
    std::snprintf(buf, buf_len, "mfma %dx%d kb%d waves %dx%d %sB=%s fill=%s stages=%d%s%s%s", v.bm, v.bn, v.kb, v.waves_m, v.waves_n,
                  v.a_kc ? "" : "A=col-major ", v.b_kc ? "col-major" : "row-major", v.direct ? "direct" : "registers", v.stages,
                  v.edge ? (v.any ? " edge any-alignment" : " edge") : "", v.pingpong ? " pingpong" : "", v.w4 ? (v.persist ? " mi16 hand-laid loop multi-tile" : " mi16 hand-laid loop") : v.mi16 ? " mi16" : "");
    return ACC950_OK;
}

} // extern "C"
