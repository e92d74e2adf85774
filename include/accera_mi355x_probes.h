/*
 * accera_mi355x_probes.h -- measurement aids, exported by libaccera_mi355x_probes.so (a library of its own:
 * the product library libaccera_mi355x.so holds none of them, nor the timed kernel builds behind them).
 *
 * Not part of the product ABI (that is accera_mi355x_gemm.h): nothing here computes a result a
 * caller of the library needs.  The benchmark and the tests use these entry points to tell what
 * the GPU at hand sustains and to scale profiler byte counters.  None has a counterpart in the reference, whose harness times whole package
 * calls (/root/reference/tools/benchmarkers/accera_gemm.py:584-657).
 */
#ifndef ACCERA_MI355X_PROBES_H
#define ACCERA_MI355X_PROBES_H

#include <stddef.h>
#include <stdint.h>

#if defined(__cplusplus)
extern "C" {
#endif

/*
 * acc950_mfma_ceiling: runs a register-resident loop of independent MFMAs of `in_type`
 * (F16, BF16 or I8) on zero (data_mode 0), constant (1) or random (2) operands and
 * reports the achieved tera-ops per second and the shader clock sustained meanwhile.
 * The sustained clock under MFMA load depends on the operand data, so the random-data
 * figure is the practical compute roof for random GEMM inputs on the device at hand.
 *
 * acc950_mfma_traffic_probe: the same MFMAs, one wave per SIMD and 64 per step as in the four-wave GEMM loop, on random
 * operands, with that loop's traffic added piece by piece: traffic 0 none, 1 its 24 LDS reads per step, 2 also its
 * direct-to-LDS fills (32 KB per step and workgroup) from a buffer that stays in the caches, 3 the fills from a 1 GiB
 * buffer.  Shows which traffic the sustained clock follows.
 *
 * acc950_mfma_phase_probe: runs a build of the 256x256 MFMA kernel the automatic choice takes
 * for large aligned problems (four waves with the hand-laid K loop when K has at least four
 * K tiles of 64 bytes, else the eight-wave ping-pong form) that reads the shader-clock counter
 * and the constant 100 MHz counter at four points in every workgroup, on dense row-major
 * DEVICE operands (M, N multiples of 256, K a multiple of 64 bytes, 16-byte aligned pointers; SET-0 prologue, ReLU
 * epilogue), synchronously; anything else is refused with ACC950_UNSUPPORTED before anything is launched.
 * out[0..2] = average time of prologue / main loop / write-back in ns, out[3..5] = shader
 * clock in GHz during each phase, out[6] = first workgroup start to last workgroup end in
 * ns, out[7] = fraction of the main loop's cycles the MFMA pipe is busy (the cycles its
 * MFMAs occupy / shader cycles).  Tells a loop that keeps the matrix cores busy at a throttled
 * clock from one that stalls.
 *
 * acc950_copy_probe / acc950_stream_read_probe: a plain copy (reads and writes `bytes`)
 * and a plain streaming read of `bytes` on DEVICE pointers, asynchronous on `stream`;
 * `bytes` must be a multiple of 16.  Known-size reference points for scaling profiler
 * byte counters and for the achievable HBM rate.  `scratch4` is 4 bytes of device memory.
 */
int acc950_mfma_ceiling(int in_type, int data_mode, int iters, double* tera_ops, double* clock_ghz);
int acc950_mfma_traffic_probe(int in_type, int traffic, int iters, double* tera_ops, double* clock_ghz);
int acc950_mfma_phase_probe(int in_type, int out_type, int M, int N, int K, const void* A, const void* B, void* C, double out[8]);
int acc950_copy_probe(void* dst, const void* src, size_t bytes, void* stream);
int acc950_stream_read_probe(const void* src, size_t bytes, void* scratch4, void* stream);

/* Why acc950_mfma_phase_probe refused its last call on this thread (the product library's acc950_last_error knows nothing of it). */
const char* acc950_probes_last_error(void);

#if defined(__cplusplus)
}
#endif
#endif /* ACCERA_MI355X_PROBES_H */
