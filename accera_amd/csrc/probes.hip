// libaccera_mi355x_probes.so: measurement aids used by the benchmark and by the tests of the benchmark's aids; the product
// library (libaccera_mi355x.so) holds none of this.
//
// Measurement aids used by the benchmark: what this particular GPU can sustain, so that
// a kernel's distance from the nominal peak can be split into "kernel" and "machine".
//
//   * MFMA ceiling: a register-resident loop of independent MFMAs of the 16x16 shapes the
//     large-tile kernels use (no memory traffic at all) on operands that are zero, constant, or random.  On MI355X the sustained
//     engine clock under MFMA load depends strongly on the operand data (power), so the
//     random-data figure -- not the nominal peak -- is the practical compute roof for
//     random GEMM inputs.
//   * Copy kernel of known size: reference point for scaling the rocprof FETCH_SIZE /
//     WRITE_SIZE counters, and a streaming read kernel for the achievable HBM rate.
#include "../../include/accera_mi355x_gemm.h"
#include "../../include/accera_mi355x_probes.h"
#include "common.h"
#include "probe_timed.h"

#include <cstdlib>
#include <string>
#include <vector>

using namespace acc950;

namespace {

thread_local std::string t_probe_error; // why the phase probe refused its last call on this thread

// 8 waves per workgroup (two per SIMD, as in the GEMM kernels), 16 independent 16x16 accumulators
// per wave, the instruction written out so that every MFMA accumulates in place.
template <int IN>
__global__ void __launch_bounds__(512) mfma_ceiling_kernel(const i32x4* src, float* out, long long* clk, int iters)
{
    i32x4 a[4], b[4];
    for (int j = 0; j < 4; ++j) a[j] = src[(threadIdx.x + 64 * j) & 1023];
    for (int j = 0; j < 4; ++j) b[j] = src[(threadIdx.x + 512 + 64 * j) & 1023];
    f32x4 acc[16];
    for (int j = 0; j < 16; ++j) acc[j] = f32x4{};
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            if constexpr (IN == T_I8) asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc[j]) : "v"(a[j >> 2]), "v"(b[j & 3]));
            else if constexpr (IN == T_BF16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[j]) : "v"(a[j >> 2]), "v"(b[j & 3]));
            else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[j]) : "v"(a[j >> 2]), "v"(b[j & 3]));
        }
    }
    const long long c1 = clock64(), w1 = wall_clock64();
    float s = 0;
    for (int j = 0; j < 16; ++j)
        for (int r = 0; r < 4; ++r) {
            const float x = acc[j][r];
            s += IN == T_I8 ? (float)__float_as_int(x) : x;
        }
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (threadIdx.x == 0 && blockIdx.x == 0) { clk[0] = c1 - c0; clk[1] = w1 - w0; }
}

// The four-wave GEMM loop's traffic next to its MFMAs, piece by piece: per wave and step 64 MFMAs on random register operands
// (as above; two waves per SIMD, which is what keeps the matrix pipe full when every MFMA is a statement of its own) and,
// depending on `traffic`, what the real loop issues per 64 MFMAs:
//   1  its 24 LDS reads (8 ds_read_b128 + 16 ds_read_b64_tr_b16) out of random data,
//   2  also its 8 direct-to-LDS fills of 1 KB (8 KB per wave and step) from a buffer that stays in L2,
//   3  the same fills from a buffer far larger than the caches.
// Nothing read is used: the question is what the traffic costs the matrix cores in clock (power) and issue slots.
template <int IN>
__global__ void __launch_bounds__(512) mfma_traffic_kernel(const i32x4* src, const char* stream, size_t stream_bytes, float* out,
                                                           long long* clk, int iters, int traffic)
{
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const unsigned wave = __builtin_amdgcn_readfirstlane((unsigned)(tid >> 6));
    // 128 KB of LDS: two stages of 64 KB (8 KB per wave), filled with the random words once
    constexpr unsigned STAGE = 65536;
    for (int i = tid; i < 8192; i += 512) ((i32x4*)lds)[i] = src[i & 1023];
    __syncthreads();
    i32x4 a[4], b[4];
    for (int j = 0; j < 4; ++j) a[j] = src[(tid + 64 * j) & 1023];
    for (int j = 0; j < 4; ++j) b[j] = src[(tid + 512 + 64 * j) & 1023];
    f32x4 acc[16];
    for (int j = 0; j < 16; ++j) acc[j] = f32x4{};
    const unsigned lds_base = (unsigned)(size_t)(ACC950_LDS char*)lds;
    const unsigned rd128 = lds_base + (unsigned)(lane * 16);                      // a wave reads 1 KB per ds_read_b128
    const unsigned rdtr = lds_base + (unsigned)((lane >> 2) * 512 + (lane & 3) * 8); // + (j - 8) * 1024 below: at most 23 KB into a stage of 64 KB
    // every workgroup streams its own 64 KB per step, wrapping inside the buffer
    const size_t per_wg = STAGE;
    size_t pos = ((size_t)blockIdx.x * 977 * per_wg) % stream_bytes;
    const unsigned lane_off = (unsigned)(lane * 16);
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
        const unsigned stage = (unsigned)(it & 1) * STAGE;
#pragma unroll
        for (int j = 0; j < 64; ++j) {
            const int k = j & 15;
            if constexpr (IN == T_I8) asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc[k]) : "v"(a[k >> 2]), "v"(b[k & 3]));
            else if constexpr (IN == T_BF16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[k]) : "v"(a[k >> 2]), "v"(b[k & 3]));
            else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[k]) : "v"(a[k >> 2]), "v"(b[k & 3]));
            if (traffic >= 1) { // uniform
                // (the data of an LDS read lands some time after the instruction, so the destinations are registers the compiler
                // has nothing in: the accumulation-register file, which only these statements touch in this kernel)
                if (j < 8) asm volatile("ds_read_b128 a[0:3], %0 offset:%1" : : "v"(rd128 + (stage ^ STAGE)), "n"(0) : "memory", "a0", "a1", "a2", "a3");
                else if (j < 24)
                    asm volatile("ds_read_b64_tr_b16 a[4:5], %0" : : "v"(rdtr + (stage ^ STAGE) + (unsigned)((j - 8) * 1024 % 16384)) : "memory", "a4", "a5");
            }
            if (traffic >= 2 && j >= 32 && j < 64 && (j & 3) == 0) {
                // fill number (j - 32) / 4 of the step: 1 KB of this wave's 8 KB, into the stage not being read
                const unsigned f = (unsigned)(j - 32) >> 2;
                const char* g = stream + pos + wave * 8192 + f * 1024;
                const unsigned long long ga = (unsigned long long)g;
                const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)ga), hi = __builtin_amdgcn_readfirstlane((unsigned)(ga >> 32));
                const unsigned m0v = __builtin_amdgcn_readfirstlane(lds_base + stage + wave * 8192 + f * 1024);
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                             :
                             : "s"(m0v), "v"(lane_off), "s"((const char*)(((unsigned long long)hi << 32) | lo))
                             : "memory");
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (traffic >= 2) {
            asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); // the previous step's fills have landed
            pos += per_wg * 256;
            if (pos + per_wg > stream_bytes) pos = (size_t)blockIdx.x * per_wg;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const long long c1 = clock64(), w1 = wall_clock64();
    float s = 0;
    for (int j = 0; j < 16; ++j)
        for (int r = 0; r < 4; ++r) {
            const float x = acc[j][r];
            s += IN == T_I8 ? (float)__float_as_int(x) : x;
        }
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (threadIdx.x == 0 && blockIdx.x == 0) { clk[0] = c1 - c0; clk[1] = w1 - w0; }
}

__global__ void __launch_bounds__(256) acc950_copy_kernel(const i32x4* __restrict__ src, i32x4* __restrict__ dst, size_t n16)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

__global__ void __launch_bounds__(256) acc950_stream_read_kernel(const i32x4* __restrict__ src, int* out, size_t n16)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    i32x4 acc = {0, 0, 0, 0};
    for (; i + 3 * stride < n16; i += 4 * stride) {
        i32x4 v0 = __builtin_nontemporal_load(src + i), v1 = __builtin_nontemporal_load(src + i + stride);
        i32x4 v2 = __builtin_nontemporal_load(src + i + 2 * stride), v3 = __builtin_nontemporal_load(src + i + 3 * stride);
        acc ^= v0 ^ v1 ^ v2 ^ v3;
    }
    for (; i < n16; i += stride) acc ^= src[i];
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678) out[0] = 1;
}

} // namespace

extern "C" {

int acc950_mfma_ceiling(int in_type, int data_mode, int iters, double* tera_ops, double* clock_ghz)
{
    if (in_type != T_F16 && in_type != T_BF16 && in_type != T_I8) return ACC950_INVALID_ARGUMENT;
    if (iters <= 0 || data_mode < 0 || data_mode > 2) return ACC950_INVALID_ARGUMENT;
    std::vector<uint16_t> h(8192);
    unsigned state = 12345u;
    auto rnd = [&]() { state = state * 1664525u + 1013904223u; return state >> 8; };
    for (auto& x : h) {
        if (data_mode == 0) x = 0;
        else if (data_mode == 1) x = in_type == T_I8 ? 0x0101 : (in_type == T_F16 ? 0x3c00 : 0x3f80);
        else if (in_type == T_I8) x = (uint16_t)rnd();
        else if (in_type == T_F16) x = (uint16_t)(((rnd() & 1) << 15) | (0x2c00 + rnd() % 0x1000)); // |x| in [2^-4, 1)
        else x = (uint16_t)(((rnd() & 1) << 15) | (0x3d80 + rnd() % 0x200));
    }
    i32x4* src = nullptr; float* out = nullptr; long long* clk = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = ACC950_HIP_ERROR;
    do {
        if (hipMalloc((void**)&src, 16384) != hipSuccess || hipMalloc((void**)&out, 256 * 512 * 4) != hipSuccess ||
            hipMalloc((void**)&clk, 16) != hipSuccess) break;
        if (hipMemcpy(src, h.data(), 16384, hipMemcpyHostToDevice) != hipSuccess) break;
        if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) break;
        auto launch = [&](int n) {
            if (in_type == T_I8) hipLaunchKernelGGL(mfma_ceiling_kernel<T_I8>, dim3(256), dim3(512), 0, 0, src, out, clk, n);
            else if (in_type == T_BF16) hipLaunchKernelGGL(mfma_ceiling_kernel<T_BF16>, dim3(256), dim3(512), 0, 0, src, out, clk, n);
            else hipLaunchKernelGGL(mfma_ceiling_kernel<T_F16>, dim3(256), dim3(512), 0, 0, src, out, clk, n);
        };
        launch(200);
        if (hipDeviceSynchronize() != hipSuccess) break;
        if (hipEventRecord(e0, 0) != hipSuccess) break;
        launch(iters);
        if (hipEventRecord(e1, 0) != hipSuccess) break;
        if (hipDeviceSynchronize() != hipSuccess) break;
        float ms = 0;
        if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) break;
        long long c[2];
        if (hipMemcpy(c, clk, 16, hipMemcpyDeviceToHost) != hipSuccess) break;
        const double ops = 256.0 * 8 * iters * 16 * (in_type == T_I8 ? 32768.0 : 16384.0);
        if (tera_ops) *tera_ops = ops / (ms * 1e-3) / 1e12;
        if (clock_ghz) *clock_ghz = c[1] > 0 ? (double)c[0] / (c[1] * 10.0) : 0.0; // wall clock ticks at 100 MHz
        rc = ACC950_OK;
    } while (false);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(src); (void)hipFree(out); (void)hipFree(clk);
    return rc;
}

int acc950_mfma_traffic_probe(int in_type, int traffic, int iters, double* tera_ops, double* clock_ghz)
{
    if (in_type != T_F16 && in_type != T_BF16 && in_type != T_I8) return ACC950_INVALID_ARGUMENT;
    if (iters <= 0 || traffic < 0 || traffic > 3) return ACC950_INVALID_ARGUMENT;
    std::vector<uint16_t> h(8192);
    unsigned state = 12345u;
    auto rnd = [&]() { state = state * 1664525u + 1013904223u; return state >> 8; };
    for (auto& x : h) {
        if (in_type == T_I8) x = (uint16_t)rnd();
        else if (in_type == T_F16) x = (uint16_t)(((rnd() & 1) << 15) | (0x2c00 + rnd() % 0x1000));
        else x = (uint16_t)(((rnd() & 1) << 15) | (0x3d80 + rnd() % 0x200));
    }
    // 16 MiB: every workgroup re-reads its own 64 KB, 2 MiB per XCD, which stay in its 4 MiB L2; 1 GiB is streamed through once per 64 steps
    const size_t stream_bytes = traffic == 3 ? ((size_t)1 << 30) : ((size_t)16 << 20);
    i32x4* src = nullptr; float* out = nullptr; long long* clk = nullptr; char* stream = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = ACC950_HIP_ERROR;
    do {
        if (hipMalloc((void**)&src, 16384) != hipSuccess || hipMalloc((void**)&out, 256 * 512 * 4) != hipSuccess ||
            hipMalloc((void**)&clk, 16) != hipSuccess || hipMalloc((void**)&stream, stream_bytes) != hipSuccess) break;
        if (hipMemcpy(src, h.data(), 16384, hipMemcpyHostToDevice) != hipSuccess) break;
        // random bytes everywhere (what is fetched also costs power by its content): the 16 KB pattern, doubled until the buffer is full
        bool filled = hipMemcpy(stream, src, 16384, hipMemcpyDeviceToDevice) == hipSuccess;
        for (size_t n = 16384; filled && n < stream_bytes; n *= 2)
            filled = hipMemcpy(stream + n, stream, n < stream_bytes - n ? n : stream_bytes - n, hipMemcpyDeviceToDevice) == hipSuccess;
        if (!filled) break;
        if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) break;
        auto kern = in_type == T_I8 ? mfma_traffic_kernel<T_I8> : in_type == T_BF16 ? mfma_traffic_kernel<T_BF16> : mfma_traffic_kernel<T_F16>;
        if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 131072) != hipSuccess) break;
        auto launch = [&](int n) { hipLaunchKernelGGL(kern, dim3(256), dim3(512), 131072, 0, src, stream, stream_bytes, out, clk, n, traffic); };
        launch(50);
        if (hipDeviceSynchronize() != hipSuccess) break;
        if (hipEventRecord(e0, 0) != hipSuccess) break;
        launch(iters);
        if (hipEventRecord(e1, 0) != hipSuccess) break;
        if (hipDeviceSynchronize() != hipSuccess) break;
        float ms = 0;
        if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) break;
        long long c[2];
        if (hipMemcpy(c, clk, 16, hipMemcpyDeviceToHost) != hipSuccess) break;
        const double ops = 256.0 * 8 * iters * 64 * (in_type == T_I8 ? 32768.0 : 16384.0);
        if (tera_ops) *tera_ops = ops / (ms * 1e-3) / 1e12;
        if (clock_ghz) *clock_ghz = c[1] > 0 ? (double)c[0] / (c[1] * 10.0) : 0.0;
        rc = ACC950_OK;
    } while (false);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(src); (void)hipFree(out); (void)hipFree(clk); (void)hipFree(stream);
    return rc;
}

int acc950_copy_probe(void* dst, const void* src, size_t bytes, void* stream)
{
    if (!dst || !src || bytes % 16) return ACC950_INVALID_ARGUMENT;
    hipLaunchKernelGGL(acc950_copy_kernel, dim3(4096), dim3(256), 0, (hipStream_t)stream, (const i32x4*)src, (i32x4*)dst, bytes / 16);
    return hipGetLastError() == hipSuccess ? ACC950_OK : ACC950_HIP_ERROR;
}

int acc950_stream_read_probe(const void* src, size_t bytes, void* scratch4, void* stream)
{
    if (!src || !scratch4 || bytes % 16) return ACC950_INVALID_ARGUMENT;
    hipLaunchKernelGGL(acc950_stream_read_kernel, dim3(512), dim3(256), 0, (hipStream_t)stream, (const i32x4*)src, (int*)scratch4, bytes / 16);
    return hipGetLastError() == hipSuccess ? ACC950_OK : ACC950_HIP_ERROR;
}

const char* acc950_probes_last_error(void) { return t_probe_error.c_str(); }

int acc950_mfma_phase_probe(int in_type, int out_type, int M, int N, int K, const void* A, const void* B, void* C, double* out)
{
    // The timed kernels take whole 256x256 tiles of dense row-major operands only (the four-wave form from four K tiles of
    // 64 bytes up, the eight-wave form below): everything else is refused here, before anything is sized or launched.
    auto refuse = [&](int code, const char* why) { t_probe_error = why; return code; };
    if (!out || !A || !B || !C) return refuse(ACC950_INVALID_ARGUMENT, "null pointer");
    if (in_type != T_F16 && in_type != T_BF16 && in_type != T_I8) return refuse(ACC950_UNSUPPORTED, "the phase probe runs the 256x256 kernels: 8/16-bit inputs");
    const bool out_ok = in_type == T_I8 ? (out_type == T_I32 || out_type == T_I16 || out_type == T_I8) : (out_type == T_F32 || out_type == T_F16 || out_type == T_BF16);
    if (!out_ok) return refuse(ACC950_INVALID_ARGUMENT, "unsupported input/output element type pair");
    const int es = in_type == T_I8 ? 1 : 2, bk = 64 / es;
    if (M < 256 || N < 256 || K < bk || M % 256 || N % 256 || K % bk)
        return refuse(ACC950_UNSUPPORTED, "the phase probe runs the 256x256 kernels: dense row-major A, B, C, M and N multiples of 256, K a multiple of 64 bytes");
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)C) & 15) return refuse(ACC950_UNSUPPORTED, "the phase probe needs 16-byte aligned operands");
    // (32-bit offsets inside a tile, as the product's own check has them)
    if ((int64_t)256 * N * 4 >= (1ll << 32) || (int64_t)256 * K * es >= (1ll << 31) || (int64_t)bk * N * es >= (1ll << 31))
        return refuse(ACC950_UNSUPPORTED, "the phase probe's tiles use 32-bit offsets: rows too long");
    GemmArgs g{};
    g.A = A; g.B = B; g.C = C; g.M = M; g.N = N; g.K = K;
    g.a_rs = K; g.a_cs = 1; g.b_rs = N; g.b_cs = 1; g.c_rs = N; g.c_cs = 1;
    g.in_type = in_type; g.out_type = out_type;
    g.prologue = PRO_SET0; g.epilogue = EPI_RELU;
    g.batch = 1;
    // one record of four stamps per tile the launcher walks: its own count of tiles
    LaunchGeom geom{};
    auto launch = [&](bool dry) {
        return in_type == T_I8 ? launch_mfma_timed_i8(g, nullptr, &geom, dry)
               : in_type == T_BF16 ? launch_mfma_timed_bf16(g, nullptr, &geom, dry) : launch_mfma_timed_f16(g, nullptr, &geom, dry);
    };
    const int tiles = (M / 256) * (N / 256);
    hipError_t e = hipMalloc((void**)&g.stamps, (size_t)tiles * 8 * sizeof(unsigned long long));
    if (e != hipSuccess) return refuse(ACC950_HIP_ERROR, hipGetErrorString(e));
    std::vector<unsigned long long> h((size_t)tiles * 8);
    const int reps = 20; // the last launch is the one read back; the others settle the clocks
    for (int i = 0; i < reps && e == hipSuccess; ++i) e = launch(false);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipMemcpy(h.data(), g.stamps, h.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost);
    hipError_t e2 = hipFree(g.stamps);
    if (e != hipSuccess) return refuse(ACC950_HIP_ERROR, hipGetErrorString(e));
    if (e2 != hipSuccess) return refuse(ACC950_HIP_ERROR, hipGetErrorString(e2));
    // per phase: average wall time (100 MHz counter) and average shader cycles over the workgroups
    unsigned long long first = ~0ull, last = 0;
    double ns[3] = {0, 0, 0}, cyc[3] = {0, 0, 0};
    for (int t = 0; t < tiles; ++t) {
        const unsigned long long* w = &h[(size_t)t * 8];
        first = w[1] < first ? w[1] : first;
        last = w[7] > last ? w[7] : last;
        for (int q = 0; q < 3; ++q) {
            ns[q] += (double)(w[(q + 1) * 2 + 1] - w[q * 2 + 1]) * 10.0;
            cyc[q] += (double)(w[(q + 1) * 2] - w[q * 2]);
        }
    }
    for (int q = 0; q < 3; ++q) {
        out[q] = ns[q] / tiles;                       // prologue, main loop, write-back [ns]
        out[3 + q] = ns[q] > 0 ? cyc[q] / ns[q] : 0;  // shader clock in that phase [GHz]
    }
    out[6] = (double)(last - first) * 10.0;           // first workgroup start to last workgroup end [ns]
    // MFMA pipe occupancy of the main loop: per SIMD, 512 MFMA cycles per 32 bytes of K (two waves x 8 MFMAs of 32 cycles,
    // or one wave x 32 MFMAs of 16 cycles)
    const double mfma_cycles = 2.0 * 8.0 * 32.0 * ((double)K * es / 32.0);
    out[7] = cyc[1] > 0 ? mfma_cycles / (cyc[1] / tiles) : 0;
    t_probe_error.clear();
    return ACC950_OK;
}

} // extern "C"
