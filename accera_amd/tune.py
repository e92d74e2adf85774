"""Variant sweep over a list of GEMM shapes: the counterpart of the reference's benchmark driver
(/root/reference/tools/benchmarkers/accera_gemm.py:187-348 builds one package per point of its
tuning space, :584-657 checks each against NumPy and times it with hatlib's min-of-means).

Here the points of the space are the prebuilt kernel variants of libaccera_mi355x.so.  For every
row of a shape list (columns m,n,k,transA,transB,alpha,beta,lda,ldb,ldc as in the reference's
tools/benchmarkers/gemm_*.csv; transX = 1 means the operand is stored column-major) the tool

  * asks the library which variants can take the problem (acc950_launch_geometry),
  * runs each on device-resident random inputs, optionally checks it against a float64 / int64
    NumPy product on sampled rows (rtol 1e-2 as the reference's driver),
  * times it with HIP events (min over batches of the mean time per launch),
  * writes one CSV row per (shape, variant) and prints the best variant per shape,
  * with --save records the best variant per shape in the table the automatic choice consults
    (accera_amd/tuned.py),
  * with --baseline also times the vendor GEMM library on the same operands (torch.matmul, i.e.
    hipBLASLt / rocBLAS; torch._int_mm for int8), the counterpart of the reference's rocBLAS
    benchmarker (/root/reference/tools/benchmarkers/rocblas/main.cpp).  The vendor call writes an
    output of the input type and has no fused epilogue; it is a yardstick, never a code path.

    python -m accera_amd.tune --input accera_amd/shapes/transformer_gemm.csv --type f16 --check --relu

    python -m accera_amd.tune --audit sweep.csv

reads a csv that --output wrote and compares, row by row of the shape list, the kernel and K slices the library takes
by itself (its cost model; the table of recorded choices is left out) with the fastest (variant, slices) of the sweep:
the geometric mean of chosen / best and the rows furthest off.  Needs no GPU: calls are bound, never launched.

alpha / beta map to the fragment ops: beta 0 -> prologue SET 0, beta 1 -> none, else SCALE beta;
alpha != 1 -> epilogue SCALE alpha (a ReLU epilogue and alpha != 1 exclude each other, as in the
reference's table docs/Tutorials/GPU/Tensor_MatMul_ElementWiseOps_GPU.md:85-99).
"""
import argparse
import csv
import sys

import numpy as np

from . import _lib

_OUT_FOR = {"f32": "f32", "f16": "f32", "bf16": "bf16", "i8": "i32"}


def _torch_dtype(torch, t):
    return {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16, "i8": torch.int8, "i32": torch.int32, "i16": torch.int16}[t]


def _make(torch, rows, cols, t, col_major, gen):
    """Random (rows x cols) matrix on the device, stored row- or column-major."""
    shape = (cols, rows) if col_major else (rows, cols)
    if t == "i8":
        x = torch.randint(-128, 128, shape, device="cuda", dtype=torch.int8, generator=gen)
    else:
        x = (torch.rand(shape, device="cuda", generator=gen) * 2 - 1).to(_torch_dtype(torch, t))
    return x.t() if col_major else x


def candidates(in_id, out_id, M, N, K, sa, sb, sc, splits_for_skinny=(0, 2, 4, 8), splits_for_mfma=(0, 2, 4, 8, 16, 32)):
    """(variant, k_splits) pairs the library accepts for this problem.  MFMA variants are tried with K split over workgroups
    only when the output is small (at most 128 tiles of 128 x 128) or has few rows (at most 256: the partial sums are then
    small beside B): elsewhere the partial sums cost more than the idle compute units."""
    L = _lib.lib()
    ids = list(range(_lib.num_variants())) + [_lib.VARIANT_SKINNY_BASE + i for i in range(_lib.num_skinny_variants())]
    ids += [_lib.VARIANT_F32_MFMA, _lib.VARIANT_GENERIC]
    out = []
    for v in ids:
        if _lib.VARIANT_SKINNY_BASE <= v < _lib.VARIANT_GENERIC:
            sweep = splits_for_skinny
        elif v < _lib.num_variants() and (-(-M // 128) * -(-N // 128) <= 128 or M <= 256):
            sweep = splits_for_mfma
        else:
            sweep = (0,)
        for sp in sweep:
            try:
                _lib.launch_geometry(in_id, out_id, M, N, K, sa, sb, sc, v, sp)
            except _lib.Acc950Error:
                continue
            out.append((v, sp))
    return out


def time_call(torch, call, min_time_s=0.05, batches=5):
    """Min over batches of the mean time per launch, HIP events on the launch stream."""
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(); call(); e1.record(); torch.cuda.synchronize()
    one = max(e0.elapsed_time(e1) * 1e-3, 1e-6)
    n = int(min(max(min_time_s / batches / one, 5), 2000))
    best = float("inf")
    for _ in range(batches):
        e0.record()
        for _ in range(n):
            call()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e-3 / n)
    return best


def sweep(rows, in_type, relu, check, out_type=None, min_time_s=0.05, log=print, baseline=False):
    import torch
    from .gemm import GemmCall
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU visible; the HIP kernels have no CPU fallback")
    out_type = out_type or _OUT_FOR[in_type]
    in_id, out_id = getattr(_lib, in_type.upper()), getattr(_lib, out_type.upper())
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    results = []
    for r in rows:
        M, N, K = int(r["m"]), int(r["n"]), int(r["k"])
        ta, tb = bool(int(r.get("transA", 0))), bool(int(r.get("transB", 0)))
        alpha, beta = float(r.get("alpha", 1.0)), float(r.get("beta", 0.0))
        A, B = _make(torch, M, K, in_type, ta, gen), _make(torch, K, N, in_type, tb, gen)
        C0 = _make(torch, M, N, "i8" if out_type in ("i32", "i16", "i8") else out_type, False, gen).to(_torch_dtype(torch, out_type))
        pro, parg = (_lib.PROLOGUE_SET0, 0.0) if beta == 0 else (_lib.PROLOGUE_NONE, 0.0) if beta == 1 else (_lib.PROLOGUE_SCALE, beta)
        if alpha != 1 and relu:
            log(f"{M}x{N}x{K}: skipped (alpha != 1 and a fused ReLU are two epilogue ops; one kernel carries one)")
            continue
        epi, earg = (_lib.EPILOGUE_SCALE, alpha) if alpha != 1 else (_lib.EPILOGUE_RELU if relu else _lib.EPILOGUE_NONE, 0.0)
        want = sample = None
        if check:
            idx = np.arange(M) if M <= 64 else np.random.default_rng(M + N).choice(M, 32, replace=False)
            Ah, Bh = A[torch.as_tensor(idx, device="cuda")].double().cpu().numpy(), B.double().cpu().numpy()
            parg_c, earg_c = (int(parg), int(earg)) if in_type == "i8" else (np.float32(parg), np.float32(earg))
            want = Ah @ Bh + (0 if beta == 0 else C0[torch.as_tensor(idx, device="cuda")].double().cpu().numpy() * (1 if beta == 1 else parg_c))
            want = want * earg_c if alpha != 1 else (np.maximum(want, 0) if relu else want)
            if out_type in ("i16", "i8"):  # narrow integer outputs keep the low bits
                bits = 16 if out_type == "i16" else 8
                want = ((want.astype(np.int64) + 2 ** (bits - 1)) % 2 ** bits) - 2 ** (bits - 1)
            sample = torch.as_tensor(idx, device="cuda")
        sa, sb, sc = (A.stride(0), A.stride(1)), (B.stride(0), B.stride(1)), (N, 1)
        best = None
        for v, sp in candidates(in_id, out_id, M, N, K, sa, sb, sc):
            C = C0.clone()
            try:
                call = GemmCall(A, B, C, prologue=pro, epilogue=epi, variant=v, k_splits=sp, prologue_arg=parg, epilogue_arg=earg)
                call()
            except _lib.Acc950Error:
                continue  # refused with the actual pointers (alignment) or fragment ops (kernels that only take C = A*B)
            ok = ""
            if check:
                C.copy_(C0)
                call()
                torch.cuda.synchronize()
                got = C[sample].double().cpu().numpy()
                tol = 0 if out_type in ("i32", "i16", "i8") else 1e-2
                ok = bool(np.allclose(got, want, rtol=tol, atol=tol * max(1.0, float(np.abs(want).max())) * 1e-1))
            # (beta != 0: C keeps accumulating over the timed launches, which costs nothing.  Restoring C before every launch
            # and subtracting the time of the restore alone measured the host instead: both loops are bound by the host's
            # cost of a launch then, and short kernels -- a K split's two above all -- came out at 5 to 6 us whatever they took.)
            t = time_call(torch, call, min_time_s)
            row = dict(m=M, n=N, k=K, transA=int(ta), transB=int(tb), alpha=alpha, beta=beta, type=in_type, out_type=out_type,
                       variant=v, k_splits=sp, kernel=_lib.variant_name(v), time_ms=round(t * 1e3, 5),
                       TFlops=round(2.0 * M * N * K / t / 1e12, 3), correct=ok)
            results.append(row)
            if ok is not False and (best is None or row["time_ms"] < best["time_ms"]):
                best = row
        vendor = ""
        if baseline:
            try:
                if in_type == "i8":
                    tv = time_call(torch, lambda: torch._int_mm(A, B), min_time_s)
                else:
                    out = torch.empty((M, N), device="cuda", dtype=A.dtype)
                    tv = time_call(torch, lambda: torch.matmul(A, B, out=out), min_time_s)
                results.append(dict(m=M, n=N, k=K, transA=int(ta), transB=int(tb), alpha=1.0, beta=0.0, type=in_type,
                                    out_type="i32" if in_type == "i8" else in_type, variant=-2, k_splits=0, kernel="vendor library (torch.matmul)",
                                    time_ms=round(tv * 1e3, 5), TFlops=round(2.0 * M * N * K / tv / 1e12, 3), correct=""))
                vendor = f"  | vendor library {round(2.0 * M * N * K / tv / 1e12, 1)} TFlops {round(tv * 1e3, 4)} ms"
            except RuntimeError as e:  # shapes the vendor call does not take (e.g. _int_mm alignment)
                vendor = f"  | vendor library: {str(e).splitlines()[0][:60]}"
        if best:
            log(f"{M}x{N}x{K} tA={int(ta)} tB={int(tb)} a={alpha} b={beta}: best {best['TFlops']} TFlops {best['time_ms']} ms  "
                f"variant {best['variant']} splits {best['k_splits']} ({best['kernel']}){vendor}")
    return results


def own_choice(in_id, out_id, M, N, K, a_col_major, b_col_major, alpha, beta):
    """(variant, K slices) the library's cost model takes for dense operands, without the table of recorded choices.
    The call is bound with made-up 256-byte aligned addresses and unbound again: nothing is launched."""
    import ctypes
    L = _lib.lib()
    sa = (1, M) if a_col_major else (K, 1)
    sb = (1, K) if b_col_major else (N, 1)
    pro, parg = (_lib.PROLOGUE_SET0, 0.0) if beta == 0 else (_lib.PROLOGUE_NONE, 0.0) if beta == 1 else (_lib.PROLOGUE_SCALE, beta)
    epi, earg = (_lib.EPILOGUE_SCALE, alpha) if alpha != 1 else (_lib.EPILOGUE_RELU, 0.0)
    handle, v, ks = ctypes.c_int(-1), ctypes.c_int(), ctypes.c_int()
    P = ctypes.c_void_p
    _lib.check(L.acc950_bind(in_id, out_id, 1, M, N, K, P(1 << 32), 0, sa[0], sa[1], P(2 << 32), 0, sb[0], sb[1], P(3 << 32), 0, N, 1,
                             pro, float(parg), epi, float(earg), _lib.VARIANT_AUTO, 0, None, ctypes.byref(handle)))
    try:
        _lib.check(L.acc950_bound_choice(handle.value, ctypes.byref(v), ctypes.byref(ks)))
    finally:
        L.acc950_unbind(handle.value)
    return v.value, max(ks.value, 1)


def audit(path, worst=10, log=print):
    """The library's own choice against the fastest entry of a sweep csv, per problem.  A choice of K slices the sweep did
    not time (it tries 2, 4, 8, 16, 32) is read at the nearest count it did.  Returns (geometric mean of chosen / best,
    [(ratio, problem, chosen kernel, slices, its ms, best kernel, slices, its ms), ...] worst first)."""
    import math
    problems = {}
    with open(path) as f:
        for r in csv.DictReader(f):
            if int(r["variant"]) == -2:  # the vendor library's row
                continue
            key = (r["type"], r["out_type"], int(r["m"]), int(r["n"]), int(r["k"]), int(r["transA"]), int(r["transB"]), float(r["alpha"]), float(r["beta"]))
            problems.setdefault(key, {})[(r["kernel"], max(int(r["k_splits"]), 1))] = float(r["time_ms"])
    rows = []
    for key, timed in problems.items():
        t, ot, M, N, K, ta, tb, alpha, beta = key
        v, ks = own_choice(getattr(_lib, t.upper()), getattr(_lib, ot.upper()), M, N, K, ta, tb, alpha, beta)
        name = _lib.variant_name(v)
        same = sorted((abs(math.log2(s) - math.log2(ks)), ms) for (n, s), ms in timed.items() if n == name)
        if not same:
            log(f"{M}x{N}x{K} tA={ta} tB={tb}: the sweep has no row for the chosen kernel ({name})")
            continue
        (best_name, best_ks), best_ms = min(timed.items(), key=lambda x: x[1])
        rows.append((same[0][1] / best_ms, key, name, ks, same[0][1], best_name, best_ks, best_ms))
    rows.sort(key=lambda x: -x[0])
    if not rows:
        return float("nan"), rows
    geomean = math.exp(sum(math.log(r[0]) for r in rows) / len(rows))
    for ratio, key, name, ks, ms, best_name, best_ks, best_ms in rows[:worst]:
        log(f"{ratio:.2f}  {key[2]}x{key[3]}x{key[4]} tA={key[5]} tB={key[6]} a={key[7]} b={key[8]}: chosen {name} x{ks} {ms} ms | best {best_name} x{best_ks} {best_ms} ms")
    log(f"{len(rows)} problems: geometric mean of chosen / best {geomean:.4f}, {sum(r[0] > 1.10 for r in rows)} more than 10 % off, "
        f"{sum(r[0] > 1.25 for r in rows)} more than 25 % off")
    return geomean, rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--input", default=None, help="shape list (csv: m,n,k,transA,transB,alpha,beta,...)")
    ap.add_argument("--audit", default=None, metavar="CSV", help="compare the library's own choices with the best rows of a csv that --output wrote (no GPU needed)")
    ap.add_argument("--type", default="f16", choices=sorted(_OUT_FOR))
    ap.add_argument("--out-type", default=None, choices=["f32", "f16", "bf16", "i32", "i16", "i8"])
    ap.add_argument("--relu", action="store_true", help="fused ReLU epilogue (rows with alpha != 1 are rejected)")
    ap.add_argument("--check", action="store_true", help="verify every variant against a NumPy product on sampled rows")
    ap.add_argument("--output", default=None, help="csv of all (shape, variant) results")
    ap.add_argument("--min-time", type=float, default=0.05, help="seconds of timed launches per variant")
    ap.add_argument("--baseline", action="store_true", help="also time the vendor GEMM library (torch.matmul) on each shape")
    ap.add_argument("--save", nargs="?", const="", default=None, metavar="JSON",
                    help="record the best variant per shape in the table that automatic kernel choices consult "
                         "(default: accera_amd/shapes/tuned_gfx950.json)")
    args = ap.parse_args(argv)
    if args.audit:
        audit(args.audit)
        return 0
    if not args.input:
        ap.error("--input or --audit is required")
    with open(args.input) as f:
        rows = [r for r in csv.DictReader(f) if r.get("m")]
    _lib.check(_lib.lib().acc950_init(0))
    results = sweep(rows, args.type, args.relu, args.check, args.out_type, args.min_time, baseline=args.baseline)
    if args.output and results:
        with open(args.output, "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=list(results[0]))
            w.writeheader()
            w.writerows(results)
    if args.save is not None and results:
        from . import tuned
        n = tuned.save(results, args.save or tuned.DEFAULT_PATH)
        print(f"{n} shapes recorded in {args.save or tuned.DEFAULT_PATH}")
    bad = [r for r in results if r["correct"] is False]
    for r in bad:
        print(f"MISMATCH {r['m']}x{r['n']}x{r['k']} variant {r['variant']} ({r['kernel']})", file=sys.stderr)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
