"""Writes tests/golden/gemm_relu_vectors.npz: small seeded problems with the results of the CPU
oracle (C nests for the SET-0 / accumulate + ReLU forms, NumPy restatement for the SET / SCALE
operands), so that a later change to the oracle or to a kernel shows up against frozen numbers.

The reference holds no stored vectors for this path (its tests draw unseeded random data and
compare with NumPy); its two constant-fill known answers (A = 2, B = 3, C = 0.42 -> 6K + 0.42:
/root/reference/docs/Tutorials/Hello_MatMul.md:165-237, Optimized_MatMul.md:204-280) are included as cases
`kat_256` and `kat_128`.

    python tests/golden/make_vectors.py        # regenerates the file (run from the repository root)
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
import oracle as ora  # noqa: E402
from tests.util import make_input  # noqa: E402

CASES = [  # name, in, out, M, N, K, B layout, prologue, prologue_arg, epilogue, epilogue_arg
    ("f16_f32_relu", "f16", "f32", 48, 64, 80, "row", ora.PRO_SET0, 0.0, ora.EPI_RELU, 0.0),
    ("f16_f16_acc_relu", "f16", "f16", 40, 56, 96, "col", ora.PRO_NONE, 0.0, ora.EPI_RELU, 0.0),
    ("bf16_bf16_relu", "bf16", "bf16", 64, 48, 64, "col", ora.PRO_SET0, 0.0, ora.EPI_RELU, 0.0),
    ("bf16_f32_nocond", "bf16", "f32", 32, 40, 48, "row", ora.PRO_NONE, 0.0, ora.EPI_RELU_NOCOND, 0.0),
    ("i8_i32_relu", "i8", "i32", 64, 64, 128, "row", ora.PRO_SET0, 0.0, ora.EPI_RELU, 0.0),
    ("i8_i32_acc", "i8", "i32", 33, 47, 29, "row", ora.PRO_NONE, 0.0, ora.EPI_NONE, 0.0),
    ("f32_f32_relu", "f32", "f32", 64, 32, 40, "row", ora.PRO_SET0, 0.0, ora.EPI_RELU, 0.0),
    ("f16_f16_skinny", "f16", "f16", 8, 128, 256, "row", ora.PRO_SET0, 0.0, ora.EPI_RELU, 0.0),
    ("f16_f32_alpha_beta", "f16", "f32", 48, 64, 64, "row", ora.PRO_SCALE, 0.5, ora.EPI_SCALE, -3.0),
    ("i8_i32_set_scale", "i8", "i32", 32, 32, 64, "row", ora.PRO_SET, 11.0, ora.EPI_SCALE, 3.0),
]


def build():
    out = {}
    for n, (name, it, ot, M, N, K, bl, pro, pa, epi, ea) in enumerate(CASES):
        rng = np.random.default_rng(9000 + n)
        A, B = make_input(rng, (M, K), it), make_input(rng, (K, N), it)
        C0 = make_input(rng, (M, N), "i8").astype(np.int32) * 100 if ot == "i32" else make_input(rng, (M, N), ot)
        if pa == 0.0 and ea == 0.0:
            Bl = np.asfortranarray(B) if bl == "col" else B
            C = ora.gemm_relu(A, Bl, C0.copy(), it, ot, prologue=pro, epilogue=epi)
        else:
            C = ora.gemm_relu_exact(A, B, C0, it, ot, pro, epi, prologue_arg=pa, epilogue_arg=ea)
        out.update({f"{name}.A": A, f"{name}.B": B, f"{name}.C0": C0, f"{name}.C": C})
    for K in (256, 128):
        A, B, C0 = np.full((16, K), 2, np.float32), np.full((K, 16), 3, np.float32), np.full((16, 16), 0.42, np.float32)
        C = ora.gemm_relu(A, B, C0.copy(), "f32", "f32", prologue=ora.PRO_NONE, epilogue=ora.EPI_NONE)
        out.update({f"kat_{K}.A": A, f"kat_{K}.B": B, f"kat_{K}.C0": C0, f"kat_{K}.C": C})
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_relu_vectors.npz")
    np.savez_compressed(path, **build())
    print(path, os.path.getsize(path), "bytes")
