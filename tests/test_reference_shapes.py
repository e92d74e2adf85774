"""Every shape the reference's GEMM benchmark driver sweeps (tools/benchmarkers/gemm_*.csv: BERT, ResNet / Inception,
square, rectangular and "big" lists; 339 distinct rows with their transA / transB / beta flags, kept as
tests/golden/reference_sweep_shapes.csv) through the library's own kernel choice, checked on sampled rows against the
oracle's exact product.  A third of them have a K, an N or a leading dimension that is not a multiple of the 16-byte
vector; none may fall to the thread-bound kernel, and the small outputs with a long K run split over K."""
import csv
import os

import numpy as np
import pytest

import oracle as ora
from util import assert_matches

HERE = os.path.dirname(os.path.abspath(__file__))


def _rows():
    with open(os.path.join(HERE, "golden", "reference_sweep_shapes.csv")) as f:
        return [(int(r["m"]), int(r["n"]), int(r["k"]), int(r["transA"]), int(r["transB"]), float(r["alpha"]), float(r["beta"]))
                for r in csv.DictReader(f)]


def test_shape_list_fixture():
    rows = _rows()
    assert len(rows) == len(set(rows)) == 339
    assert (768, 320, 30522, 0, 0, 1.0, 1.0) in rows and (8192, 8192, 8192, 1, 1, 1.0, 1.0) in rows
    assert all(a == 1.0 and b in (0.0, 1.0) for *_, a, b in rows)


@pytest.mark.gpu
@pytest.mark.parametrize("in_type,out_type", [("f16", "f16"), ("bf16", "f32"), ("i8", "i32"), ("f32", "f32")])
def test_every_shape_of_the_reference_sweep_lists(in_type, out_type):
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    tdt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "i8": torch.int8, "i32": torch.int32}
    gen = torch.Generator(device="cuda")
    gen.manual_seed(339)
    kinds = {}
    for n, (M, N, K, ta, tb, alpha, beta) in enumerate(_rows()):
        def draw(r, c, t, col_major):
            shape = (c, r) if col_major else (r, c)
            if t == "i8":
                x = torch.randint(-128, 128, shape, device="cuda", dtype=torch.int8, generator=gen)
            else:
                x = (torch.rand(shape, device="cuda", generator=gen) * 2 - 1).to(tdt[t])
            return x.t() if col_major else x
        A, B = draw(M, K, in_type, ta), draw(K, N, in_type, tb)
        C0 = draw(M, N, "i8" if out_type == "i32" else out_type, False).to(tdt[out_type])
        C = C0.clone()
        prologue = ora.PRO_SET0 if beta == 0 else ora.PRO_NONE
        # the kernel and the K slices bound for this very call: its prologue (beta = 1 reads C) and its pointers
        call = acc.GemmCall(A, B, C, prologue=prologue, epilogue=ora.EPI_RELU)
        v, slices = call.chosen
        name = _lib.variant_name(v)
        assert v != _lib.VARIANT_GENERIC, (M, N, K, ta, tb, name)
        split = slices > 1 and "skinny" not in name
        kind = "fp32 32x32 blocks" if v == _lib.VARIANT_F32_MFMA else "skinny" if "skinny" in name else ("any-alignment" if "any-alignment" in name else "mfma") + (", K split" if split else "")
        kinds[kind] = kinds.get(kind, 0) + 1
        print(n, (M, N, K, ta, tb, beta), name, "slices", slices, flush=True)
        call()
        idx = np.arange(M) if M <= 48 else np.random.default_rng(n).choice(M, 24, replace=False)
        sel = torch.as_tensor(idx, device="cuda")
        torch.cuda.synchronize()
        host = lambda x, t: x.cpu().view(torch.int16).numpy().view(np.uint16) if t == "bf16" else x.cpu().numpy()  # (bf16 travels as its bits)
        want = ora.gemm_relu_exact(host(A[sel], in_type), host(B, in_type), host(C0[sel], out_type), in_type, out_type, prologue, ora.EPI_RELU)
        assert_matches(host(C[sel], out_type), want, out_type, K)
    print(kinds)
    if in_type != "f32":  # (small fp32 problems stay with the kernel of 32 x 32 blocks, which takes any size)
        assert kinds.get("any-alignment", 0) + kinds.get("any-alignment, K split", 0) >= 90
    assert sum(c for k, c in kinds.items() if "K split" in k) >= 10
