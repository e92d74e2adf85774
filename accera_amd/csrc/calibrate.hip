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

#include <cstdlib>
#include <vector>

using namespace acc950;

namespace {

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

} // extern "C"
