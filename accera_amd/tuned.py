"""Persisted per-shape kernel choices: the table `python -m accera_amd.tune --save` writes and the
calls with an automatic kernel choice consult.

The reference's benchmark driver keeps the best variant per GEMM shape in its results database and
picks it up for later builds (/root/reference/tools/benchmarkers/accera_gemm.py:584-657, 676-709);
here the table is a JSON file next to the shape lists.  Entries name the kernel by its description
(`acc950_variant_name`), not by its index, so a table survives a change of the variant order; an
entry whose kernel the library no longer has, or no longer accepts for the problem, is ignored and
the library's own choice applies.
"""
import json
import os

from . import _lib

DEFAULT_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "shapes", "tuned_gfx950.json")
_table = None
_names = None


def ops_class(prologue, prologue_arg, epilogue):
    """Kernels differ in the prologue / epilogue ops they take, so a choice is recorded per class:
    "lean"  C = A*B or relu(A*B)          (SET 0 prologue: C is not read)
    "acc"   C += A*B, then ReLU or nothing (C read, no operand)
    "full"  everything else               (SCALE / SET with an operand, the other epilogue ops)"""
    plain = epilogue in (_lib.EPILOGUE_RELU, _lib.EPILOGUE_NONE)
    if plain and prologue == _lib.PROLOGUE_SET and float(prologue_arg) == 0.0:
        return "lean"
    if plain and prologue == _lib.PROLOGUE_NONE:
        return "acc"
    return "full"


def key(in_id, out_id, M, N, K, a_col_major, b_col_major, ops):
    """ops: a class of ops_class() (True / False are read as "lean" / "full")."""
    if isinstance(ops, bool):
        ops = "lean" if ops else "full"
    return f"{in_id}-{out_id}-{M}x{N}x{K}-{'c' if a_col_major else 'r'}{'c' if b_col_major else 'r'}-{ops}"


def _load():
    global _table
    if _table is None:
        path = os.environ.get("ACCERA_AMD_TUNED", DEFAULT_PATH)
        try:
            with open(path) as f:
                _table = json.load(f)
        except (OSError, ValueError):
            _table = {}
    return _table


def _variant_by_name(name):
    global _names
    if _names is None:
        ids = list(range(_lib.num_variants())) + [_lib.VARIANT_SKINNY_BASE + i for i in range(_lib.num_skinny_variants())]
        _names = {_lib.variant_name(v): v for v in ids}
    return _names.get(name)


def lookup(in_id, out_id, M, N, K, a_strides, b_strides, c_strides, ops):
    """(variant, k_splits) recorded for this problem and class of ops (ops_class), or None.  Only plain
    row- / column-major operands and a row-major C are looked up; the library still validates the choice
    when the call is bound, and callers fall back to its own choice if it refuses."""
    if tuple(c_strides) != (N, 1):
        return None
    a_col = tuple(a_strides) == (1, M) and M != 1
    b_col = tuple(b_strides) == (1, K) and K != 1
    if not a_col and tuple(a_strides) != (K, 1):
        return None
    if not b_col and tuple(b_strides) != (N, 1):
        return None
    rec = _load().get(key(in_id, out_id, M, N, K, a_col, b_col, ops))
    if not rec:
        return None
    v = _variant_by_name(rec.get("kernel", ""))
    if v is None:
        return None
    try:
        _lib.launch_geometry(in_id, out_id, M, N, K, a_strides, b_strides, c_strides, v, int(rec.get("k_splits", 0)))
    except _lib.Acc950Error:
        return None
    return v, int(rec.get("k_splits", 0))


def save(results, path=DEFAULT_PATH, merge=True):
    """Write the best verified row per problem of a sweep (rows of accera_amd.tune.sweep)."""
    table = {}
    if merge and os.path.exists(path):
        try:
            with open(path) as f:
                table = json.load(f)
        except ValueError:
            table = {}
    best = {}
    for r in results:
        if r["variant"] < 0 or r["correct"] is False:
            continue
        alpha, beta = float(r["alpha"]), float(r["beta"])
        ops = "lean" if (alpha == 1.0 and beta == 0.0) else "acc" if (alpha == 1.0 and beta == 1.0) else "full"
        k = key(getattr(_lib, r["type"].upper()), getattr(_lib, r["out_type"].upper()), r["m"], r["n"], r["k"],
                bool(r["transA"]), bool(r["transB"]), ops)
        if k not in best or r["time_ms"] < best[k]["time_ms"]:
            best[k] = r
    for k, r in best.items():
        table[k] = {"kernel": r["kernel"], "k_splits": r["k_splits"], "time_ms": r["time_ms"], "TFlops": r["TFlops"]}
    with open(path, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
    return len(best)


def reset():
    """Forget the loaded table (tests, or after `save`)."""
    global _table
    _table = None
