"""Device-tensor front end of the C ABI: torch supplies device memory and streams,
every computation happens in the HIP kernels of libaccera_mi355x.so."""
import ctypes

import torch

from . import _lib

_TORCH_TYPES = {
    torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16,
    torch.int8: _lib.I8, torch.int32: _lib.I32, torch.int16: _lib.I16,
}


def _mat(t, name):
    if t.dim() not in (2, 3):
        raise ValueError(f"{name} must be 2-D, or 3-D for a batch")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (there is no CPU path)")
    if t.dim() == 3:
        return t.data_ptr(), t.stride(0), t.stride(1), t.stride(2)
    return t.data_ptr(), 0, t.stride(0), t.stride(1)


def _problem(A, B, C):
    """(in type, out type, batch, M, N, K, A ptr + strides, B ..., C ...) of a 2-D call or of a batch
    (3-D tensors (batch, rows, cols); a 2-D A or B is shared by every problem of the batch)."""
    batch = C.shape[0] if C.dim() == 3 else 1
    if C.dim() == 2 and (A.dim() == 3 or B.dim() == 3):
        raise ValueError("a batched A or B needs a 3-D C")
    for t, name in ((A, "A"), (B, "B")):
        if t.dim() == 3 and t.shape[0] != batch:
            raise ValueError(f"{name} has {t.shape[0]} matrices, C has {batch}")
    M, K = A.shape[-2:]
    K2, N = B.shape[-2:]
    if K2 != K or tuple(C.shape[-2:]) != (M, N):
        raise ValueError(f"shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, C {tuple(C.shape)}")
    if A.dtype != B.dtype or A.dtype not in _TORCH_TYPES or C.dtype not in _TORCH_TYPES:
        raise ValueError(f"unsupported dtypes {A.dtype}, {B.dtype}, {C.dtype}")
    return (_TORCH_TYPES[A.dtype], _TORCH_TYPES[C.dtype], batch, M, N, K, *_mat(A, "A"), *_mat(B, "B"), *_mat(C, "C"))


class GemmCall:
    """One matmul+epilogue bound to its tensors, like one function of a package bound to
    its arrays: everything about the call is fixed at construction, calling it only
    launches.  Keeps the tensors alive; `stream` is a raw hipStream_t (int) or None for the
    stream that is current when the object is built."""

    def __init__(self, A, B, C, prologue=_lib.PROLOGUE_SET0, epilogue=_lib.EPILOGUE_RELU, variant=_lib.VARIANT_AUTO,
                 k_splits=0, stream=None, prologue_arg=0.0, epilogue_arg=0.0):
        problem = _problem(A, B, C)
        hit = None
        if variant == _lib.VARIANT_AUTO and k_splits == 0 and problem[2] == 1:
            # a recorded choice for this very shape (accera_amd.tune --save) goes before the library's cost model
            from . import tuned
            hit = tuned.lookup(problem[0], problem[1], problem[3], problem[4], problem[5], problem[8:10], problem[12:14], problem[16:18],
                               tuned.ops_class(prologue, prologue_arg, epilogue))
            if hit:
                variant, k_splits = hit
        if stream is None:
            stream = torch.cuda.current_stream(C.device).cuda_stream
        self.variant, self.k_splits = variant, k_splits  # as asked of the library (after the table look-up)
        self.tensors = (A, B, C)
        L = _lib.lib()
        handle = ctypes.c_int(-1)
        rc = L.acc950_bind(*problem, prologue, float(prologue_arg), epilogue, float(epilogue_arg), variant, k_splits, stream,
                           ctypes.byref(handle))
        if rc and hit:
            # the recorded kernel does not take this call after all (pointer alignment, ops): the library chooses
            self.variant, self.k_splits = _lib.VARIANT_AUTO, 0
            rc = L.acc950_bind(*problem, prologue, float(prologue_arg), epilogue, float(epilogue_arg), _lib.VARIANT_AUTO, 0, stream,
                               ctypes.byref(handle))
        _lib.check(rc)
        self._handle = handle.value
        self._launch, self._unbind = L.acc950_launch, L.acc950_unbind
        # what the library bound for this very call (its ops and pointers): kernel variant and number of K slices
        v, ks = ctypes.c_int(), ctypes.c_int()
        _lib.check(L.acc950_bound_choice(self._handle, ctypes.byref(v), ctypes.byref(ks)))
        self.chosen = (v.value, ks.value)

    def __call__(self):
        rc = self._launch(self._handle)
        if rc:
            _lib.check(rc)
        return self.tensors[2]

    def __del__(self):
        if getattr(self, "_handle", -1) >= 0:
            self._unbind(self._handle)
            self._handle = -1


def gemm_relu(A, B, C, prologue=_lib.PROLOGUE_SET0, epilogue=_lib.EPILOGUE_RELU, variant=_lib.VARIANT_AUTO,
              k_splits=0, stream=None, prologue_arg=0.0, epilogue_arg=0.0):
    """C = epilogue(prologue(C) + A @ B), in place on C, asynchronously.

    prologue: NONE keeps C, SET replaces it by ``prologue_arg`` (0: the fused matmul+ReLU),
    SCALE multiplies it by ``prologue_arg`` (GEMM beta); epilogue: NONE, RELU, RELU_NOCOND,
    SCALE by ``epilogue_arg`` (GEMM alpha), SET
    (/root/reference/docs/Tutorials/GPU/Tensor_MatMul_ElementWiseOps_GPU.md:85-99).

    A (M,K), B (K,N), C (M,N) are CUDA/HIP tensors; strides are honoured (a
    column-major B is ``B_storage.t()`` of an (N,K) tensor).  With a 3-D C (batch, M, N) the
    call is a batch of independent problems in one launch (the reference's batch matmul nest,
    /root/reference/accera/python/accera/test/mfma_tests.py:435-549); A and B are 3-D, or 2-D to be
    shared by the whole batch.  Types: fp16/bf16 in -> fp32/fp16/bf16 out, int8 -> int32/int16/int8,
    fp32 -> fp32.  Mirrors calling one function of an Accera package on (A, B, C)
    (/root/reference/README.md:124-130), on device memory.
    """
    GemmCall(A, B, C, prologue, epilogue, variant, k_splits, stream, prologue_arg, epilogue_arg)()
    return C
