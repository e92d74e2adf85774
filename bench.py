#!/usr/bin/env python3
"""Benchmark of the matmul + fused-ReLU hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2] [--no-cpu] [--only]

A "step" is one GEMM+ReLU launch on device-resident synthetic inputs.  The default
workload is the configuration the headline metric is quoted on: fp16 inputs, fp32
accumulate / output, M=N=K=4096, C = max(A.B, 0).  The metric also names the int8 GEMM and
the skinny decode GEMM, and the benchmark has two more configurations (the fp32 quick-start
problem and the bf16 FFN GEMM), so the default run measures all four others as well, the same
way, and reports them under "other_configs", each with its own roofline block (`--only`
leaves them out).  Before the W untimed warm-up steps of a configuration its kernel is launched for
SETTLE_MS of wall time (reported as settle_ms): after idling the engine clock takes some tens
of milliseconds of load to settle, whatever W is.  One JSON line is printed with
  value         whole-job TFLOP/s (2*M*N*K per step, the formula of the reference's
                harness: /root/reference/tools/benchmarkers/accera_gemm.py:648-654)
  roofline      algorithmic FLOP (or bytes) per launch / average launch duration from
                HIP events on the launch stream, against the MI355X dense peak
  cpu_baseline  the CPU oracle (a restatement of the reference's HOST schedule, not an
                Accera-generated package) timed on this box's host cores

(`--all` is accepted and means the default: all five configurations.)
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"f16": 2500.0, "bf16": 2500.0, "i8": 5000.0, "f32": 157.3}  # dense MFMA TFLOP/s (TOP/s)
HBM_PEAK_GBS = 8000.0
SETTLE_MS = 150.0  # launches of the kernel under test before the counted warm-up, by wall time

CONFIGS = {
    # name: in, out, M, N, K, B layout, bound
    "c1": dict(in_type="f32", out_type="f32", M=512, N=512, K=512, b="row", bound="mfma",
               workload="fp32 matmul+ReLU 512x512x512 (README quickstart)"),
    "c2": dict(in_type="f16", out_type="f32", M=4096, N=4096, K=4096, b="row", bound="mfma",
               workload="fp16->fp32 matmul+ReLU 4096x4096x4096, row-major A,B"),
    "c3": dict(in_type="bf16", out_type="bf16", M=4096, N=3072, K=768, b="col", bound="mfma",
               workload="bf16 FFN GEMM+ReLU M4096 K768 N3072, B column-major, bf16 out"),
    "c4": dict(in_type="i8", out_type="i32", M=8192, N=8192, K=8192, b="row", bound="mfma",
               workload="int8->int32 GEMM+ReLU 8192x8192x8192"),
    "c5": dict(in_type="f16", out_type="f16", M=8, N=11008, K=4096, b="row", bound="hbm",
               workload="skinny decode GEMM+ReLU M8 K4096 N11008 fp16"),
}
ES = {"f32": 4, "f16": 2, "bf16": 2, "i8": 1, "i32": 4}


def algorithmic_bytes(c):
    """A + B read once, C written once (C starts at zero: SET prologue, not read)."""
    return c["M"] * c["K"] * ES[c["in_type"]] + c["K"] * c["N"] * ES[c["in_type"]] + c["M"] * c["N"] * ES[c["out_type"]]


def algorithmic_flops(c):
    return 2 * c["M"] * c["N"] * c["K"]


def make_inputs(c, n_sets, seed):
    """Device-resident inputs in the distributions BASELINE names; n_sets rotating copies."""
    import torch
    tt = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16, "i8": torch.int8, "i32": torch.int32}
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    M, N, K = c["M"], c["N"], c["K"]
    sets = []
    for _ in range(n_sets):
        if c["in_type"] == "i8":
            A = torch.randint(-128, 128, (M, K), device="cuda", dtype=torch.int8, generator=g)
            B = torch.randint(-128, 128, (K, N), device="cuda", dtype=torch.int8, generator=g)
        elif c["in_type"] == "f32":
            A = torch.rand((M, K), device="cuda", generator=g)
            B = torch.rand((K, N), device="cuda", generator=g)
        elif c["in_type"] == "f16" and c["bound"] == "mfma":
            A = (torch.rand((M, K), device="cuda", generator=g) * 2 - 1).to(torch.float16)
            B = (torch.rand((K, N), device="cuda", generator=g) * 2 - 1).to(torch.float16)
        else:  # N(0,1) activations, N(0, 0.02^2) weights
            A = torch.randn((M, K), device="cuda", generator=g).to(tt[c["in_type"]])
            B = (torch.randn((K, N), device="cuda", generator=g) * 0.02).to(tt[c["in_type"]])
        if c["b"] == "col":
            B = B.t().contiguous().t()  # same values, column-major storage
        C = torch.zeros((M, N), device="cuda", dtype=tt[c["out_type"]])
        sets.append((A, B, C))
    return sets


def run_gpu(c, steps, warmup, variant=-1, k_splits=0):
    import torch
    import accera_amd as acc
    # bandwidth-bound case: rotate over enough distinct buffers to exceed the 256 MB
    # last-level cache so that B really streams from HBM
    n_sets = 1 if c["bound"] == "mfma" else max(2, int(640e6 // algorithmic_bytes(c)) + 1)
    sets = make_inputs(c, n_sets, seed=1000)
    stream = torch.cuda.current_stream()

    # one bound call per input set: the timed loop only launches
    calls = [acc.GemmCall(A, B, C, prologue=acc.PROLOGUE_SET0, epilogue=acc.EPILOGUE_RELU, variant=variant, k_splits=k_splits)
             for A, B, C in sets]

    def step(i):
        calls[i % n_sets]()

    # clock settle by wall time, then the counted warm-up
    t_settle = time.perf_counter()
    n = 0
    while (time.perf_counter() - t_settle) * 1e3 < SETTLE_MS:
        for _ in range(32):
            step(n)
            n += 1
        torch.cuda.synchronize()
    run_gpu.settle_ms = round((time.perf_counter() - t_settle) * 1e3, 1)
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    run_gpu.rotating_sets = n_sets
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for i in range(steps):
        step(i)
    ev1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    launch_s = ev0.elapsed_time(ev1) * 1e-3 / steps
    run_gpu.asked = (calls[0].variant, calls[0].k_splits)  # a recorded per-shape choice, or what the caller passed
    return wall, launch_s, sets[0]


def cpu_baseline(c, threads, budget_rows=None):
    """Oracle (CPU restatement, 'transformed' 16x16 schedule) on a row block of the same
    problem; full N and K so that the access pattern is the workload's."""
    import oracle as ora
    rng = np.random.default_rng(1000)
    M = c["M"] if budget_rows is None else min(c["M"], budget_rows)
    N, K = c["N"], c["K"]
    t = c["in_type"]
    if t == "i8":
        A = rng.integers(-128, 128, (M, K), dtype=np.int8)
        B = rng.integers(-128, 128, (K, N), dtype=np.int8)
    else:
        A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
        if t == "f16":
            A, B = A.astype(np.float16), B.astype(np.float16)
        elif t == "bf16":
            A, B = ora.to_bf16(A), ora.to_bf16(B)
    if c["b"] == "col":
        B = np.asfortranarray(B)
    C = np.zeros((M, N), ora.NP_STORAGE[c["out_type"]])
    ora.gemm_relu(A[:16], B, C[:16], t, c["out_type"], threads=threads)  # warm-up (page faults, OpenMP pool)
    passes, dt = 3, float("inf")
    for _ in range(passes):
        t0 = time.perf_counter()
        ora.gemm_relu(A, B, C, t, c["out_type"], schedule=ora.SCHED_TRANSFORMED, threads=threads)
        dt = min(dt, time.perf_counter() - t0)
    return dict(value=round(2 * M * N * K / dt / 1e12, 5), unit="TFLOP/s" if t != "i8" else "TOP/s", cores=threads,
                kind="port", seconds=round(dt, 3),
                sample=f"rows 0..{M - 1} of A against all of B ({M}x{N}x{K}), best of {passes} passes, OpenMP over column tiles")


def vendor_library(c, first_set, steps):
    """The vendor GEMM library (torch.matmul -> hipBLASLt / rocBLAS, torch._int_mm for int8) on the same
    operands: a yardstick beside the reference's own rocBLAS benchmarker
    (/root/reference/tools/benchmarkers/rocblas/main.cpp).  It writes an output of the input type (int32 for
    int8) and has no fused epilogue; nothing in the product path calls it."""
    import torch
    A, B, _ = first_set
    try:
        if c["in_type"] == "i8":
            call = lambda: torch._int_mm(A, B)
        else:
            out = torch.empty((c["M"], c["N"]), dtype=A.dtype, device="cuda")
            call = lambda: torch.matmul(A, B, out=out)
        for _ in range(min(steps, 50)):
            call()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n = max(min(steps, 200), 10)
        e0.record()
        for _ in range(n):
            call()
        e1.record()
        torch.cuda.synchronize()
        dt = e0.elapsed_time(e1) * 1e-3 / n
    except RuntimeError as e:
        return {"error": str(e).splitlines()[0][:80]}
    if c["bound"] == "hbm":
        return {"value": round(algorithmic_bytes(c) / dt / 1e9, 1), "unit": "GB/s", "ms_per_step": round(dt * 1e3, 5),
                "call": "torch.matmul, output of the input type, no epilogue"}
    return {"value": round(algorithmic_flops(c) / dt / 1e12, 1), "unit": "TFLOP/s" if c["in_type"] != "i8" else "TOP/s",
            "ms_per_step": round(dt * 1e3, 5),
            "call": "torch._int_mm, int32 output, no epilogue" if c["in_type"] == "i8" else "torch.matmul, output of the input type, no epilogue"}


def traffic_bytes(name):
    """HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and scaled by the
    plain copy kernel of known size (written to profiles/traffic.json by accera_amd.profiling)."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        rec = json.load(f).get(name)
    return None if not rec else int(rec["hbm_bytes_per_launch"])


def machine_ceiling(c):
    """What this GPU sustains, measured now: pure-MFMA rate on random operands (the engine
    clock under MFMA load is data dependent) or a plain streaming read of the same size."""
    import torch
    from accera_amd import _lib
    if c["bound"] == "mfma" and c["in_type"] in ("f16", "bf16", "i8"):
        t = getattr(_lib, c["in_type"].upper())
        rnd, ghz = _lib.mfma_ceiling(t, 2, 20000)
        cool, ghz0 = _lib.mfma_ceiling(t, 0, 20000)
        out = {"mfma_only_random_operands": round(rnd, 1), "clock_ghz_random": round(ghz, 3),
               "mfma_only_zero_operands": round(cool, 1), "clock_ghz_zero": round(ghz0, 3), "unit": "TFLOP/s" if t != _lib.I8 else "TOP/s"}
        # the four-wave loop's MFMAs with its traffic added piece by piece: which traffic the sustained clock follows
        for key, traffic in (("four_wave_issue_no_traffic", 0), ("plus_lds_reads", 1), ("plus_fills_from_cache", 2), ("plus_fills_from_hbm", 3)):
            rate, clock = _lib.mfma_traffic_probe(t, traffic, 3000)
            out[key] = {"rate": round(rate, 1), "clock_ghz": round(clock, 3)}
        return out
    if c["bound"] == "hbm":
        nbytes = c["K"] * c["N"] * ES[c["in_type"]]
        bufs = [torch.empty(nbytes, dtype=torch.uint8, device="cuda").fill_(i + 1) for i in range(8)]
        out = torch.zeros(1, dtype=torch.int32, device="cuda")
        stream = torch.cuda.current_stream()
        L = _lib.probes()
        for i in range(8):
            _lib.check_probe(L.acc950_stream_read_probe(bufs[i].data_ptr(), nbytes, out.data_ptr(), stream.cuda_stream))
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(80):
            _lib.check_probe(L.acc950_stream_read_probe(bufs[i % 8].data_ptr(), nbytes, out.data_ptr(), stream.cuda_stream))
        e1.record(stream)
        torch.cuda.synchronize()
        return {"plain_streaming_read_same_bytes": round(nbytes / (e0.elapsed_time(e1) * 1e-3 / 80) / 1e9, 1), "unit": "GB/s"}
    return None


def measure(name, steps, warmup, variant=-1, k_splits=0):
    c = CONFIGS[name]
    wall, launch_s, first_set = run_gpu(c, steps, warmup, variant, k_splits)
    in_kernel = None
    if c["bound"] == "mfma" and c["in_type"] in ("f16", "bf16", "i8") and c["b"] == "row" and c["M"] % 256 == 0 and c["N"] % 256 == 0 \
            and variant < 0:
        # clock stamps inside the 256x256 kernel of the automatic choice on the same operands: phase times, the
        # engine clock in each phase, and how busy the MFMA pipe is at that clock
        from accera_amd import _lib
        A, B, C = first_set
        in_kernel = {k: round(v, 4) for k, v in _lib.mfma_phase_probe(
            getattr(_lib, c["in_type"].upper()), getattr(_lib, c["out_type"].upper()), c["M"], c["N"], c["K"],
            A.data_ptr(), B.data_ptr(), C.data_ptr()).items()}
    flops, nbytes = algorithmic_flops(c), algorithmic_bytes(c)
    if c["bound"] == "hbm":
        achieved, peak, unit = nbytes / launch_s / 1e9, HBM_PEAK_GBS, "GB/s"
        value, vunit = nbytes * steps / wall / 1e9, "GB/s"
    else:
        achieved, peak, unit = flops / launch_s / 1e12, PEAK[c["in_type"]], "TFLOP/s" if c["in_type"] != "i8" else "TOP/s"
        value, vunit = flops * steps / wall / 1e12, unit
    return dict(config=name, workload=c["workload"], value=round(value, 3), unit=vunit, ms_per_step=round(wall / steps * 1e3, 5),
                steps=steps, warmup=warmup, settle_ms=run_gpu.settle_ms, rotating_input_sets=run_gpu.rotating_sets,
                dtype={"f16": "f16", "bf16": "bf16", "i8": "int8", "f32": "f32"}[c["in_type"]],
                kernel=_kernel_record(c),
                roofline=dict(bound=c["bound"], achieved=round(achieved, 3), peak=peak, unit=unit,
                              frac=round(achieved / peak, 4), traffic=traffic_bytes(name)),
                flops_per_launch=flops, bytes_per_launch=nbytes, in_kernel=in_kernel,
                machine_ceiling=machine_ceiling(c),
                vendor_library=vendor_library(c, first_set, steps))


def _kernel_record(c):
    """Name and launch geometry of the kernel the timed calls ran."""
    from accera_amd import _lib
    grid, block, lds, chosen = _lib.launch_geometry(
        getattr(_lib, c["in_type"].upper()), getattr(_lib, c["out_type"].upper()), c["M"], c["N"], c["K"],
        (c["K"], 1), (c["N"], 1) if c["b"] == "row" else (1, c["K"]), (c["N"], 1), *run_gpu.asked)
    return {"name": _lib.variant_name(chosen), "grid": grid, "block": block, "dynamic_lds_bytes": lds}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50, help="untimed steps (after the time-based clock settle)")
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--variant", type=int, default=-1)
    ap.add_argument("--k-splits", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", action="store_true", help="measure --config alone (default: the four other configurations ride along)")
    ap.add_argument("--all", action="store_true", help="all five BASELINE configurations (the default)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP kernels have no CPU fallback", file=sys.stderr)
        sys.exit(3)
    from accera_amd import _lib
    _lib.check(_lib.lib().acc950_init(0))

    c = CONFIGS[args.config]
    # plain copy of known size: the reference point for scaling profiler byte counters
    probe = torch.empty(2, 64 << 20, dtype=torch.uint8, device="cuda")
    _lib.check_probe(_lib.probes().acc950_copy_probe(probe[1].data_ptr(), probe[0].data_ptr(), 64 << 20, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    del probe
    m = measure(args.config, args.steps, args.warmup, args.variant, args.k_splits)
    out = {
        "metric": "GEMM+ReLU TFLOP/s (TOPS int8) & % MFMA peak at 4096^3 fp16; skinny GEMM HBM GB/s",
        "value": m["value"], "unit": m["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_ms": m["settle_ms"],
        "ms_per_step": m["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": m["dtype"], "data": "synthetic",
        "config": {"workload": c["workload"], "M": c["M"], "N": c["N"], "K": c["K"], "kernel": m["kernel"]["name"],
                   "grid": m["kernel"]["grid"], "block": m["kernel"]["block"], "dynamic_lds_bytes": m["kernel"]["dynamic_lds_bytes"],
                   "device": torch.cuda.get_device_name(0),
                   "arch": torch.cuda.get_device_properties(0).gcnArchName,
                   "compute_units": torch.cuda.get_device_properties(0).multi_processor_count},
        "roofline": m["roofline"],
        "machine_ceiling": m["machine_ceiling"],
        "in_kernel": m["in_kernel"],
        "vendor_library": m["vendor_library"],
    }
    if not args.no_cpu:
        threads = min(16, os.cpu_count() or 1)
        # bounded sample: about 10-30 s of single-core work spread over the host cores
        rows = {"c2": None, "c4": 2048, "c3": None, "c1": None, "c5": None}[args.config]
        out["cpu_baseline"] = cpu_baseline(c, threads, rows)
    # the rest of the metric -- int8 GEMM (TOP/s against the int8 MFMA peak), skinny decode GEMM (HBM GB/s) -- and the two
    # remaining configurations of the benchmark (bf16 FFN GEMM, fp32 quick-start problem)
    others = [] if args.only or args.variant >= 0 or args.k_splits else [n for n in ("c4", "c5", "c3", "c1") if n != args.config]
    if others:
        out["other_configs"] = [measure(n, args.steps, args.warmup) for n in others]
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
