"""Frozen vectors (tests/golden/gemm_relu_vectors.npz, written by tests/golden/make_vectors.py):
the oracle must still reproduce them bit for bit, and the kernels must match them."""
import os

import numpy as np
import pytest

import oracle as ora
from tests.golden.make_vectors import CASES, build

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemm_relu_vectors.npz")


def test_oracle_reproduces_the_frozen_vectors():
    frozen = np.load(PATH)
    now = build()
    assert set(frozen.files) == set(now)
    for k in frozen.files:
        assert frozen[k].dtype == now[k].dtype and np.array_equal(frozen[k], now[k], equal_nan=True), k
    # the reference's constant-fill known answers: 6K + 0.42
    assert np.allclose(frozen["kat_256.C"], 1536.42) and np.allclose(frozen["kat_128.C"], 768.42)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES + [("kat_256", "f32", "f32", 16, 16, 256, "row", ora.PRO_NONE, 0.0, ora.EPI_NONE, 0.0),
                                          ("kat_128", "f32", "f32", 16, 16, 128, "row", ora.PRO_NONE, 0.0, ora.EPI_NONE, 0.0)],
                         ids=lambda c: c[0])
def test_kernels_match_the_frozen_vectors(case):
    import accera_amd as acc
    import torch
    from tests.util import assert_matches, to_device, to_host
    name, it, ot, M, N, K, bl, pro, pa, epi, ea = case
    z = np.load(PATH)
    A, B, C0, want = z[f"{name}.A"], z[f"{name}.B"], z[f"{name}.C0"], z[f"{name}.C"]
    dC = to_device(C0, ot)
    acc.gemm_relu(to_device(A, it), to_device(np.asfortranarray(B) if bl == "col" else B, it), dC, prologue=pro, prologue_arg=pa,
                  epilogue=epi, epilogue_arg=ea)
    torch.cuda.synchronize()
    assert_matches(to_host(dC, ot), want, ot, K)
