"""Shared helpers of the parity tests: seeded inputs in the reference's conventions,
host<->device plumbing through torch, and comparison against the CPU oracle."""
import numpy as np

import oracle as ora

TORCH_OF = None


def _torch():
    import torch
    return torch


def make_input(rng, shape, t, dist="uniform"):
    """Random matrix in storage dtype (bf16 as uint16).  float: U[-1,1) or N(0,1);
    int8: full range (the reference draws randint(-2,2), mfma_tests.py:141-145; the
    full range is the harder superset)."""
    if t == "i8":
        return rng.integers(-128, 128, shape, dtype=np.int8)
    x = rng.uniform(-1, 1, shape) if dist == "uniform" else rng.standard_normal(shape)
    x = x.astype(np.float32)
    if t == "f32":
        return x
    if t == "f16":
        return x.astype(np.float16)
    return ora.to_bf16(x)


INT_OUT = ("i32", "i16", "i8")


def make_c0(rng, shape, out_type, dist="uniform", scale=1000):
    """Initial C of an accumulating call.  int32: int8 draws times ``scale``; int16 / int8: the
    full range of the type (so that widening must honour the sign); float: like the inputs."""
    if out_type == "i32":
        return make_input(rng, shape, "i8", dist).astype(np.int32) * scale
    if out_type == "i16":
        return rng.integers(-2**15, 2**15, shape, dtype=np.int16)
    return make_input(rng, shape, out_type, dist)


def to_device(x, t):
    torch = _torch()
    x = np.ascontiguousarray(x) if not (x.flags.c_contiguous or x.flags.f_contiguous) else x
    if x.flags.f_contiguous and not x.flags.c_contiguous:
        # keep the column-major layout: upload the transpose, hand back a transposed view
        return to_device(np.ascontiguousarray(x.T), t).t()
    if t == "bf16":
        return torch.from_numpy(x.view(np.int16).copy()).view(torch.bfloat16).cuda()
    return torch.from_numpy(x.copy()).cuda()


def to_host(x, t):
    torch = _torch()
    if t == "bf16":
        return x.cpu().view(torch.int16).numpy().view(np.uint16)
    return x.cpu().numpy()


def out_zeros(M, N, t, order="C"):
    return np.zeros((M, N), ora.NP_STORAGE[t], order=order)


def assert_matches(got, want, out_type, K, exact=False, rtol=None):
    """got/want in storage dtype.  Integer: bit-exact.  Float: rtol by type
    (1e-3 for fp32 output of an fp32-accumulated sum, 1e-2 for fp16/bf16 output) plus an
    absolute term for near-cancelling sums that scales with sqrt(K)."""
    if out_type in INT_OUT or exact:
        assert np.array_equal(got, want), f"{(got != want).sum()} of {got.size} elements differ"
        return
    g, w = ora.widen(got, out_type), ora.widen(want, out_type)
    if rtol is None:
        rtol = {"f32": 1e-3, "f16": 1e-2, "bf16": 1e-2}[out_type]
    atol = 1e-5 * np.sqrt(max(K, 1)) * max(1.0, float(np.abs(w).max()) / 8)
    np.testing.assert_allclose(g, w, rtol=rtol, atol=atol)
