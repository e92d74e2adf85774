"""Device-tensor front end of the C ABI: torch supplies device memory and streams,
every computation happens in the HIP kernels of libaccera_mi355x.so."""
import torch

from . import _lib

_TORCH_TYPES = {
    torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16,
    torch.int8: _lib.I8, torch.int32: _lib.I32,
}


def _mat(t, name):
    if t.dim() != 2:
        raise ValueError(f"{name} must be 2-D")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (there is no CPU path)")
    return t.data_ptr(), t.stride(0), t.stride(1)


class GemmCall:
    """One matmul+epilogue bound to its tensors, like one function of a package bound to
    its arrays: everything about the call is fixed at construction, calling it only
    launches.  Keeps the tensors alive; `stream` is a raw hipStream_t (int) or None for the
    stream that is current when the object is built."""

    def __init__(self, A, B, C, prologue=_lib.PROLOGUE_SET0, epilogue=_lib.EPILOGUE_RELU, variant=_lib.VARIANT_AUTO,
                 k_splits=0, stream=None, prologue_arg=0.0, epilogue_arg=0.0):
        M, K = A.shape
        K2, N = B.shape
        if K2 != K or tuple(C.shape) != (M, N):
            raise ValueError(f"shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, C {tuple(C.shape)}")
        if A.dtype != B.dtype or A.dtype not in _TORCH_TYPES or C.dtype not in _TORCH_TYPES:
            raise ValueError(f"unsupported dtypes {A.dtype}, {B.dtype}, {C.dtype}")
        if stream is None:
            stream = torch.cuda.current_stream(C.device).cuda_stream
        self.tensors = (A, B, C)
        self._fn = _lib.lib().acc950_gemm_ops
        self._args = (_TORCH_TYPES[A.dtype], _TORCH_TYPES[C.dtype], M, N, K, *_mat(A, "A"), *_mat(B, "B"), *_mat(C, "C"),
                      prologue, float(prologue_arg), epilogue, float(epilogue_arg), variant, k_splits, stream)

    def __call__(self):
        rc = self._fn(*self._args)
        if rc:
            _lib.check(rc)
        return self.tensors[2]


def gemm_relu(A, B, C, prologue=_lib.PROLOGUE_SET0, epilogue=_lib.EPILOGUE_RELU, variant=_lib.VARIANT_AUTO,
              k_splits=0, stream=None, prologue_arg=0.0, epilogue_arg=0.0):
    """C = epilogue(prologue(C) + A @ B), in place on C, asynchronously.

    prologue: NONE keeps C, SET replaces it by ``prologue_arg`` (0: the fused matmul+ReLU),
    SCALE multiplies it by ``prologue_arg`` (GEMM beta); epilogue: NONE, RELU, RELU_NOCOND,
    SCALE by ``epilogue_arg`` (GEMM alpha), SET
    (/root/reference/docs/Tutorials/GPU/Tensor_MatMul_ElementWiseOps_GPU.md:85-99).

    A (M,K), B (K,N), C (M,N) are CUDA/HIP tensors; strides are honoured (a
    column-major B is ``B_storage.t()`` of an (N,K) tensor).  Types: fp16/bf16 in ->
    fp32/fp16/bf16 out, int8 -> int32, fp32 -> fp32.  Mirrors calling one function of
    an Accera package on (A, B, C) (/root/reference/README.md:124-130), on device memory.
    """
    M, K = A.shape
    K2, N = B.shape
    if K2 != K or tuple(C.shape) != (M, N):
        raise ValueError(f"shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, C {tuple(C.shape)}")
    if A.dtype != B.dtype or A.dtype not in _TORCH_TYPES or C.dtype not in _TORCH_TYPES:
        raise ValueError(f"unsupported dtypes {A.dtype}, {B.dtype}, {C.dtype}")
    if stream is None:
        stream = torch.cuda.current_stream(C.device).cuda_stream
    rc = _lib.lib().acc950_gemm_ops(_TORCH_TYPES[A.dtype], _TORCH_TYPES[C.dtype], M, N, K,
                                    *_mat(A, "A"), *_mat(B, "B"), *_mat(C, "C"),
                                    prologue, float(prologue_arg), epilogue, float(epilogue_arg), variant, k_splits, stream)
    _lib.check(rc)
    return C
