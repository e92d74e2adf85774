/*
 * accera_mi355x_gemm.h -- C ABI of the MI355X (gfx950) matmul + fused-epilogue kernels.
 *
 * The library replaces, for one GPU, what the reference's GPU plan path emits for an
 * `acc.Nest` matmul with a fused elementwise epilogue (C += A*B, then ReLU): the
 * generated `<fn>__gpu__` kernels and their host launcher stubs.  Each entry point
 * below names the reference interface it stands in for.  Plain pointers and sizes
 * only; no exceptions cross this boundary; every function returns an ACC950_* status.
 *
 * Matrices are described the way a .hat file describes an `affine_array`
 * (/root/reference/accera/ir/src/TranslateToHeader.cpp:713-762): shape plus element
 * strides (`affine_map`); row-major M x N has strides (N, 1), column-major (1, M).
 * Strides are 64-bit and not negative; A's stride between consecutive k and B's stride between consecutive
 * columns (after the exchange of operands that a column-major C brings) must be below 2^31 elements, or the
 * call is refused with ACC950_UNSUPPORTED: the kernels take those two as 32-bit arguments.
 */
#ifndef ACCERA_MI355X_GEMM_H
#define ACCERA_MI355X_GEMM_H

#include <stddef.h>
#include <stdint.h>

#if defined(__cplusplus)
extern "C" {
#endif

/* element types; the .hat element_type names are float, float16_t, bfloat16_t,
 * int8_t, int16_t, int32_t (TranslateToHeader.cpp:165-192, 329-400).  Pairs taken:
 * f32 -> f32; f16 / bf16 -> f32, f16, bf16; i8 -> i32, i16, i8 (the output pairs of the reference's
 * MI100 tensor-core table, /root/reference/accera/python/accera/Targets.py:796-821).  int16 / int8
 * outputs widen with their sign when C is read and keep the low bits of the int32 result. */
#define ACC950_F32 0
#define ACC950_F16 1
#define ACC950_BF16 2
#define ACC950_I8 3
#define ACC950_I32 4
#define ACC950_I16 5

/* prologue / epilogue ops of plan.tensorize
 * (/root/reference/accera/python/accera/lang/Plan.py:208-379;
 *  device helpers /root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:630-655) */
#define ACC950_PROLOGUE_NONE 0  /* C = epilogue(C + A*B) */
#define ACC950_PROLOGUE_SET0 1  /* C = epilogue(A*B)           (MMAFragmentOp.SET with 0) */
#define ACC950_PROLOGUE_SET 1   /* C = epilogue(arg + A*B)     (MMAFragmentOp.SET, acc950_gemm_ops) */
#define ACC950_PROLOGUE_SCALE 2 /* C = epilogue(arg*C + A*B)   (MMAFragmentOp.SCALE: the beta of a GEMM) */
#define ACC950_EPILOGUE_NONE 0
#define ACC950_EPILOGUE_RELU 1           /* v > 0 ? v : 0 */
#define ACC950_EPILOGUE_RELU_NOCOND 2    /* v *= (v > 0)  */
#define ACC950_EPILOGUE_SCALE 3          /* v *= arg      (the alpha of a GEMM) */
#define ACC950_EPILOGUE_SET 4            /* v = arg */

/* status codes */
#define ACC950_OK 0
#define ACC950_INVALID_ARGUMENT 1 /* bad type pair, negative size, null pointer, unknown op */
#define ACC950_UNSUPPORTED 2      /* the requested kernel variant cannot take this problem */
#define ACC950_HIP_ERROR 3        /* a HIP call failed; see acc950_last_error() */

/* kernel selection for acc950_gemm_relu_ex */
#define ACC950_VARIANT_AUTO (-1)
#define ACC950_VARIANT_SKINNY_BASE 100 /* 100 + i : streaming kernel i for M <= 8 */
#define ACC950_VARIANT_GENERIC 200     /* thread-bound kernel, any shape / stride / type */
#define ACC950_VARIANT_F32_MFMA 201    /* fp32 MFMA kernel (fp32 inputs) */

/*
 * Selects the device and checks that it is a gfx950 part.  Optional: the other entry
 * points use the current HIP device.  Stands in for hatlib's device selection
 * (`device_id=` of hat.run_benchmark, /root/reference/tools/benchmarkers/accera_gemm.py:612-626).
 */
int acc950_init(int device_id);

/*
 * C = epilogue((prologue == SET0 ? 0 : C) + A * B) on DEVICE pointers, asynchronously on
 * `stream` (a hipStream_t, or NULL for the default stream).  A is M x K, B is K x N,
 * C is M x N.  in_type F16/BF16 -> out_type F32/F16/BF16 (fp32 accumulate);
 * I8 -> I32 (exact, wrap-around); F32 -> F32.
 *
 * Replaces the generated host launcher `fn(A,B,C){ fn__gpu__<<<grid,block,lds>>>(A,B,C); }`
 * which likewise takes device pointers
 * (/root/reference/accera/acc-translate/src/Target/Cpp/GpuDialectCppPrinter.cpp:532-561)
 * and the kernel body the tensorize / cache / bind lowering produces
 * (/root/reference/accera/transforms/src/exec/ExecutionPlanToAffineLoweringPass.cpp:5986-6533).
 */
int acc950_gemm_relu(int in_type, int out_type, int M, int N, int K,
                     const void* A, int64_t a_row_stride, int64_t a_col_stride,
                     const void* B, int64_t b_row_stride, int64_t b_col_stride,
                     void* C, int64_t c_row_stride, int64_t c_col_stride,
                     int prologue, int epilogue, void* stream);

/*
 * Same, with the kernel variant chosen by the caller: the counterpart of building one
 * point of the reference's tuning space (tile sizes, cache strategy, double buffering:
 * /root/reference/tools/benchmarkers/accera_gemm.py:187-348).  `variant` is
 * ACC950_VARIANT_AUTO, an index < acc950_num_variants() into the MFMA table,
 * ACC950_VARIANT_SKINNY_BASE + i, ACC950_VARIANT_F32_MFMA or ACC950_VARIANT_GENERIC.  `k_splits` splits K
 * over workgroups (skinny and MFMA kernels; 0 = the library decides -- for a named MFMA variant: no split --,
 * 1 = no split, n > 1 = at most n slices).  The slices are added in a fixed order, so a split result does not
 * vary from run to run; an MFMA kernel's split goes through a workspace of 4 * slices * M * N bytes (held per
 * stream, or the built-in one of acc950_gemm_ops_static) and a second kernel that adds the slices and applies
 * the prologue / epilogue ops.  A named variant that does not take the
 * problem -- its sizes, layouts, alignment, or its prologue / epilogue ops (the four-wave kernels
 * do not read an int8 C) -- returns ACC950_UNSUPPORTED; nothing runs.
 */
int acc950_gemm_relu_ex(int in_type, int out_type, int M, int N, int K,
                        const void* A, int64_t a_row_stride, int64_t a_col_stride,
                        const void* B, int64_t b_row_stride, int64_t b_col_stride,
                        void* C, int64_t c_row_stride, int64_t c_col_stride,
                        int prologue, int epilogue, int variant, int k_splits, void* stream);

/*
 * General form with the operands of the fragment ops: every prologue / epilogue op of
 * the reference's tensorized plan (/root/reference/accera/python/accera/lang/Plan.py:208-379;
 * helpers set / scale / relu / relu_no_conditional,
 * /root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:630-655; GEMM alpha / beta table,
 * /root/reference/docs/Tutorials/GPU/Tensor_MatMul_ElementWiseOps_GPU.md:85-99).  The operands are cast to
 * the accumulator type (float, or int for int8 inputs) as the reference's helpers do; an
 * operand of an op that takes none is ignored.  acc950_gemm_relu_ex is this call with both
 * operands 0.  acc950_gemm_ops_host is the same on HOST pointers (see below).
 */
int acc950_gemm_ops(int in_type, int out_type, int M, int N, int K,
                    const void* A, int64_t a_row_stride, int64_t a_col_stride,
                    const void* B, int64_t b_row_stride, int64_t b_col_stride,
                    void* C, int64_t c_row_stride, int64_t c_col_stride,
                    int prologue, double prologue_arg, int epilogue, double epilogue_arg,
                    int variant, int k_splits, void* stream);
int acc950_gemm_ops_host(int in_type, int out_type, int M, int N, int K,
                         const void* A, int64_t a_row_stride, int64_t a_col_stride,
                         const void* B, int64_t b_row_stride, int64_t b_col_stride,
                         void* C, int64_t c_row_stride, int64_t c_col_stride,
                         int prologue, double prologue_arg, int epilogue, double epilogue_arg);

/*
 * acc950_gemm_ops for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid it).  It has no counterpart in the reference.  Same arguments, same kernels, same
 * results; the difference is where the skinny kernels' partial sums and arrival counters live when workgroups
 * combine their sums (a K split, or the shared column blocks of the default decode kernel), and the slices of an
 * MFMA kernel's K split: in a fixed array of
 * ACC950_STATIC_WORKSPACE_BYTES inside the library's device image (each GPU the library runs on holds its own
 * copy until the process ends) instead of a per-stream allocation.  The call makes no hipMalloc / hipFree and no
 * other allocating call; a skinny problem whose workspace would not fit returns ACC950_UNSUPPORTED and runs nothing
 * (8 x 11008 x 4096 needs 2.7 MiB); an MFMA problem is split into as many slices as fit the array (the kernel is
 * chosen for that number), so its sums can be added in a different order than acc950_gemm_ops adds them -- the
 * results are the same bits only when the allocating entry point's split fits the array too.  All calls on one GPU share that array: calls that overlap on a GPU (different
 * streams, different host threads) race on it -- keep them on one stream or use acc950_gemm_ops.  The kernels leave
 * the counters at zero, which is how the array starts.  Launch each kernel once outside a capture first: the first
 * launch of a kernel loads its code and may raise its LDS limit.
 */
#define ACC950_STATIC_WORKSPACE_BYTES (4u << 20)
int acc950_gemm_ops_static(int in_type, int out_type, int M, int N, int K,
                           const void* A, int64_t a_row_stride, int64_t a_col_stride,
                           const void* B, int64_t b_row_stride, int64_t b_col_stride,
                           void* C, int64_t c_row_stride, int64_t c_col_stride,
                           int prologue, double prologue_arg, int epilogue, double epilogue_arg,
                           int variant, int k_splits, void* stream);

/*
 * Batch of `batch` independent problems of one shape, one launch (grid.z = batch):
 * C[b] = epilogue(prologue(C[b]) + A[b] * B[b]); x_batch_stride is the element distance
 * between consecutive matrices (0 broadcasts one matrix to every problem).  Counterpart of
 * the reference's batch matmul nest C[b,i,j] += A[b,i,k] * B[b,k,j] with the batch index
 * bound to the grid (/root/reference/accera/python/accera/test/mfma_tests.py:435-549, 2519-2549).
 * acc950_gemm_batched_host is the same on HOST pointers.
 */
int acc950_gemm_batched(int in_type, int out_type, int batch, int M, int N, int K,
                        const void* A, int64_t a_batch_stride, int64_t a_row_stride, int64_t a_col_stride,
                        const void* B, int64_t b_batch_stride, int64_t b_row_stride, int64_t b_col_stride,
                        void* C, int64_t c_batch_stride, int64_t c_row_stride, int64_t c_col_stride,
                        int prologue, double prologue_arg, int epilogue, double epilogue_arg,
                        int variant, int k_splits, void* stream);
int acc950_gemm_batched_host(int in_type, int out_type, int batch, int M, int N, int K,
                             const void* A, int64_t a_batch_stride, int64_t a_row_stride, int64_t a_col_stride,
                             const void* B, int64_t b_batch_stride, int64_t b_row_stride, int64_t b_col_stride,
                             void* C, int64_t c_batch_stride, int64_t c_row_stride, int64_t c_col_stride,
                             int prologue, double prologue_arg, int epilogue, double epilogue_arg,
                             int variant, int k_splits);

/*
 * Bound call: validates the problem and chooses the kernel once, then acc950_launch(handle)
 * only launches (asynchronously on the stream given at bind time).  This is what a function
 * of a package is to its caller, a fixed kernel for fixed shapes, with the arrays fixed too;
 * it keeps per-launch host time at a few hundred nanoseconds, which matters for the
 * quick-start sized problems whose kernels run for a few microseconds
 * (hatlib times packages by calling the same function on the same arrays in a loop,
 * /root/reference/tools/benchmarkers/accera_gemm.py:640-648).  Arguments as acc950_gemm_batched.
 * The caller keeps A, B, C alive until acc950_unbind.
 */
int acc950_bind(int in_type, int out_type, int batch, int M, int N, int K,
                const void* A, int64_t a_batch_stride, int64_t a_row_stride, int64_t a_col_stride,
                const void* B, int64_t b_batch_stride, int64_t b_row_stride, int64_t b_col_stride,
                void* C, int64_t c_batch_stride, int64_t c_row_stride, int64_t c_col_stride,
                int prologue, double prologue_arg, int epilogue, double epilogue_arg,
                int variant, int k_splits, void* stream, int* handle);
int acc950_launch(int handle);
int acc950_unbind(int handle);

/*
 * Same computation on HOST pointers, synchronous: copies A, B (and C when it is
 * accumulated into) to the device, runs the kernel, copies C back.  This is the
 * calling convention of a HAT_DYNAMIC package function `void f(T* A, T* B, T* C)` as
 * hatlib calls it with NumPy arrays
 * (/root/reference/README.md:118-136; /root/reference/accera/python/accera/Package.py:776-784);
 * the per-function symbols of a package forward to this entry point.
 */
int acc950_gemm_relu_host(int in_type, int out_type, int M, int N, int K,
                          const void* A, int64_t a_row_stride, int64_t a_col_stride,
                          const void* B, int64_t b_row_stride, int64_t b_col_stride,
                          void* C, int64_t c_row_stride, int64_t c_col_stride,
                          int prologue, int epilogue);

/*
 * Launch record of the kernel acc950_gemm_relu_ex would run for this problem, without
 * running it: grid[3], block[3], dynamic LDS bytes, and the variant actually chosen.
 * The structural counterpart of the `launch_parameters` / `dynamic_shared_mem_bytes`
 * fields the reference regex-parses out of its generated source
 * (/root/reference/accera/python/accera/Package.py:25-28, 714-743).
 */
int acc950_launch_geometry(int in_type, int out_type, int M, int N, int K,
                           int64_t a_row_stride, int64_t a_col_stride,
                           int64_t b_row_stride, int64_t b_col_stride,
                           int64_t c_row_stride, int64_t c_col_stride,
                           int variant, int k_splits,
                           unsigned grid[3], unsigned block[3], unsigned* dynamic_lds_bytes, int* chosen_variant);

/* Number of MFMA table variants, and a human-readable description of any variant id
 * ("mfma 256x256 waves 2x2 B=row-major fill=direct", ...).  Returns ACC950_INVALID_ARGUMENT
 * for an unknown id. */
int acc950_num_variants(void);
int acc950_num_skinny_variants(void);
int acc950_variant_name(int variant, char* buf, size_t buf_len);

/* ---- bookkeeping of the library itself (for tests and long-running hosts; no counterpart in the reference) ---- */

/*
 * The K-split workspace the skinny kernels would use for a launch on `stream` of the current device
 * (partial sums and arrival counters; one workspace per device and stream, so that launches
 * on different streams never share one).  Allocates it at its smallest size if the stream has
 * none yet.  DEVICE addresses, for comparison only.
 */
int acc950_workspace_probe(void* stream, void** partial_sums, void** counters);

/* Number of device allocations (hipMalloc) the GEMM entry points of this process have made so far: K-split
 * workspaces and the device buffers of the host-pointer path.  A test of an entry point that must not allocate
 * reads it before and after. */
int acc950_allocation_probe(unsigned long long* count);

/*
 * Frees every K-split workspace the allocating entry points have made on the current device (all streams), the blocks
 * they have outgrown included, after waiting for the device to go idle, and the buffers the host-pointer entry points
 * keep between calls (per call that was ever in flight at once: device copies as large as the largest operands it
 * carried, 16 MiB of pinned staging, a stream).  The next launch that needs a workspace, the next call on host
 * pointers, allocates anew.  For programs that create and destroy streams or sweep over growing problems; a workspace
 * otherwise stays with its (device, stream) pair until the process ends (at least 4 MiB + 16 KiB per pair).  Must not
 * run while another thread launches on the device.  No counterpart in the reference, whose functions own no device state.
 */
int acc950_release_workspaces(void);

/*
 * What a bound call (acc950_bind) runs: the kernel variant chosen and the number of K slices (1: no split).  The
 * launch-geometry query above answers for the plain product; this answers for the call's own ops and pointers.
 */
int acc950_bound_choice(int handle, int* variant, int* k_splits);

/* Text of the last error on the calling thread ("" if none). */
const char* acc950_last_error(void);

#if defined(__cplusplus)
}
#endif
#endif /* ACCERA_MI355X_GEMM_H */
