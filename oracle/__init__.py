"""CPU oracle for the matmul + fused-ReLU hot path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; the product (``accera_amd``) never does.

Two restatements of the reference's nest semantics live here:

* ``gemm_relu``        -- the C loop nests in ``gemm_relu_oracle.c`` (float
  accumulate in sequential k order, both README schedules), called via ctypes.
* ``gemm_relu_exact``  -- NumPy: float64 (or int64) matmul of the exactly
  widened inputs, i.e. the mathematically exact sum up to float64 rounding;
  used where the sequential C nest would take too long and as an independent
  cross-check of it.

Reference semantics followed: /root/reference/README.md:52-92 (quickstart
nests and schedules), /root/reference/accera/python/accera/test/mfma_tests.py:58-101,380-432
(GPU matmul / matmul+ReLU plans, expected value alpha*(A@B)+beta*C),
/root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:95-118,630-655
(bf16 casts, relu / relu_no_conditional).

Parity unpinned: the exact float summation order of an Accera-generated HOST package
(fast-math, not reproducible from the tree); everything else is pinned by tests/test_oracle.py.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F32, F16, BF16, I8, I32, I16 = 0, 1, 2, 3, 4, 5
TYPE_IDS = {"f32": F32, "f16": F16, "bf16": BF16, "i8": I8, "i32": I32, "i16": I16}
NP_STORAGE = {"f32": np.float32, "f16": np.float16, "bf16": np.uint16, "i8": np.int8, "i32": np.int32, "i16": np.int16}
PRO_NONE, PRO_SET0, PRO_SET, PRO_SCALE = 0, 1, 1, 2
EPI_NONE, EPI_RELU, EPI_RELU_NOCOND, EPI_SCALE, EPI_SET = 0, 1, 2, 3, 4
SCHED_NAIVE, SCHED_TRANSFORMED = 0, 1

_lib = None


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        L.oracle_gemm_relu.restype = ci
        L.oracle_gemm_relu.argtypes = [ci, ci, ci, ci, ci, vp, i64, i64, vp, i64, i64, vp, i64, i64, ci, ci, ci]
        L.oracle_set_threads.argtypes = [ci]
        L.oracle_max_threads.restype = ci
        for n in ("half_to_float", "float_to_half", "bf16_to_float", "float_to_bf16"):
            getattr(L, f"oracle_{n}_n").argtypes = [vp, vp, i64]
        _lib = L
    return _lib


# ---- bf16 helpers (NumPy has no bfloat16: arrays travel as uint16 bit patterns) ----

def to_bf16(x):
    """float32 -> bfloat16 bit patterns (uint16), round to nearest even, NaN kept quiet."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def from_bf16(b):
    """bfloat16 bit patterns (uint16) -> float32, exact."""
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def widen(x, type_name):
    """Array of a storage type -> float64 (float family) or int64 (int family), exactly."""
    if type_name == "bf16":
        return from_bf16(x).astype(np.float64)
    if type_name in ("i8", "i16", "i32"):
        return np.asarray(x).astype(np.int64)
    return np.asarray(x).astype(np.float64)


def narrow(x, type_name):
    """float32 / int64 values -> storage type with the oracle's rounding."""
    if type_name == "bf16":
        return to_bf16(x.astype(np.float32))
    if type_name == "f16":
        return x.astype(np.float32).astype(np.float16)
    if type_name == "f32":
        return x.astype(np.float32)
    # integer outputs keep the low bits of the int32 sum, like the plain C conversion in the
    # reference's accumulator store (/root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:289-293)
    bits = {"i32": 32, "i16": 16, "i8": 8}[type_name]
    x = x.astype(np.int64)
    return (((x + 2 ** (bits - 1)) % 2 ** bits) - 2 ** (bits - 1)).astype(NP_STORAGE[type_name])


def _strides_elems(a):
    assert a.ndim == 2
    return a.strides[0] // a.itemsize, a.strides[1] // a.itemsize


def gemm_relu(A, B, C, in_type, out_type, prologue=PRO_SET0, epilogue=EPI_RELU,
              schedule=SCHED_TRANSFORMED, threads=1):
    """C = epilogue((prologue==SET0 ? 0 : C) + A @ B) in place, through the C nests.

    A (M,K), B (K,N), C (M,N) are NumPy arrays of the storage dtype of
    ``in_type`` / ``out_type`` ("bf16" travels as uint16); any 2-D strides are
    honoured, so a column-major B is simply an ``order="F"`` array.
    """
    L = lib()
    M, K = A.shape
    K2, N = B.shape
    assert K2 == K and C.shape == (M, N)
    assert A.dtype == NP_STORAGE[in_type] and B.dtype == NP_STORAGE[in_type] and C.dtype == NP_STORAGE[out_type]
    L.oracle_set_threads(int(threads))
    ars, acs = _strides_elems(A)
    brs, bcs = _strides_elems(B)
    crs, ccs = _strides_elems(C)
    rc = L.oracle_gemm_relu(TYPE_IDS[in_type], TYPE_IDS[out_type], M, N, K,
                            A.ctypes.data, ars, acs, B.ctypes.data, brs, bcs, C.ctypes.data, crs, ccs,
                            prologue, epilogue, schedule)
    if rc != 0:
        raise ValueError(f"oracle_gemm_relu failed with code {rc}")
    return C


def _op_arg(arg, in_type):
    """Operand of a SET / SCALE fragment op cast to the accumulator type, as the reference's
    helpers do (`const _Ty arg`, /root/reference/accera/acc-translate/src/Target/Cpp/CppPrinterUtils.h:644-655)."""
    return int(arg) if in_type == "i8" else float(np.float32(arg))


def gemm_relu_exact(A, B, C0, in_type, out_type, prologue=PRO_SET0, epilogue=EPI_RELU, narrow_out=True,
                    prologue_arg=0.0, epilogue_arg=0.0):
    """NumPy restatement: exact widened product summed in float64 / int64.

    prologue: NONE keeps C0, SET replaces it by ``prologue_arg``, SCALE multiplies it by
    ``prologue_arg``; epilogue: NONE, RELU, RELU_NOCOND, SCALE by ``epilogue_arg``, SET
    (/root/reference/docs/Tutorials/GPU/Tensor_MatMul_ElementWiseOps_GPU.md:85-99).  The C
    nests in gemm_relu_oracle.c cover NONE / SET 0 and the two ReLUs only.

    Returns the result narrowed to ``out_type`` storage (or the float64 / int64
    pre-narrowing values when ``narrow_out`` is False).
    """
    Aw, Bw = widen(A, in_type), widen(B, in_type)
    if in_type == "i8" and Aw.shape[1] * 2 ** 14 < 2 ** 52:
        # int8 products are at most 2^14 in size, so every partial sum is an integer below 2^52 and the float64 product
        # (a BLAS call, much faster than NumPy's int64 loop) is exact in whatever order it adds
        S = (Aw.astype(np.float64) @ Bw.astype(np.float64)).astype(np.int64)
    else:
        S = Aw @ Bw
    if prologue == PRO_SET:
        S = S + _op_arg(prologue_arg, in_type)
    elif prologue == PRO_SCALE:
        S = S + widen(C0, out_type) * _op_arg(prologue_arg, in_type)
    else:
        S = S + widen(C0, out_type)
    wrap = (lambda x: ((x + 2**31) % 2**32) - 2**31) if in_type == "i8" else (lambda x: x)
    S = wrap(S)
    if epilogue == EPI_RELU:
        S = np.maximum(S, 0) if in_type == "i8" else np.where(S > 0, S, 0.0)
    elif epilogue == EPI_RELU_NOCOND:
        S = np.maximum(S, 0) if in_type == "i8" else S * (S > 0)
    elif epilogue == EPI_SCALE:
        S = wrap(S * _op_arg(epilogue_arg, in_type))
    elif epilogue == EPI_SET:
        S = np.full_like(S, _op_arg(epilogue_arg, in_type))
    return narrow(S, out_type) if narrow_out else S
