"""GPU parity tests: every kernel family of libaccera_mi355x.so, called through the C
ABI on device memory, against the CPU oracle on the same seeded inputs.

Integer results must be bit-exact; float results are held to the tolerances the
reference's own tests use (rtol 1e-3 for fp32 output of fp16/bf16 inputs, 1e-2 for
fp16/bf16 output: mfma_tests.py:2047,2083,2553-2577), with signed data so that ReLU
really clips (the reference's ReLU tests use non-negative inputs only).
"""
import re

import numpy as np
import pytest

import oracle as ora
from tests.util import INT_OUT, assert_matches, make_c0, make_input, out_zeros, to_device, to_host

pytestmark = pytest.mark.gpu

PAIRS = [("f16", "f32"), ("f16", "f16"), ("bf16", "f32"), ("bf16", "bf16"), ("i8", "i32"), ("i8", "i16"), ("i8", "i8")]


def run_case(in_type, out_type, M, N, K, b_layout="row", c_layout="row", variant=-1, splits=0,
             prologue=ora.PRO_SET0, epilogue=ora.EPI_RELU, seed=0, dist="uniform", expect_variant=None, a_layout="row"):
    import accera_amd as acc
    import torch
    rng = np.random.default_rng(seed)
    A = make_input(rng, (M, K), in_type, dist)
    B = make_input(rng, (K, N), in_type, dist)
    if b_layout == "col":
        B = np.asfortranarray(B)
    if a_layout == "col":
        A = np.asfortranarray(A)
    if prologue == ora.PRO_NONE:
        C0 = make_c0(rng, (M, N), out_type, dist)
    else:
        # poison C so that a kernel that wrongly reads it cannot pass
        C0 = np.full((M, N), 77, ora.NP_STORAGE[out_type]) if out_type in INT_OUT else make_input(rng, (M, N), out_type, dist)
    if c_layout == "col":
        C0 = np.asfortranarray(C0)
    dA, dB, dC = to_device(A, in_type), to_device(B, in_type), to_device(C0, out_type)
    assert dB.stride() == ((1, K) if b_layout == "col" else (N, 1))
    acc.gemm_relu(dA, dB, dC, prologue=prologue, epilogue=epilogue, variant=variant, k_splits=splits)
    torch.cuda.synchronize()
    got = to_host(dC, out_type)
    want = ora.gemm_relu_exact(A, B, C0, in_type, out_type, prologue, epilogue)
    assert_matches(got, want, out_type, K)
    if epilogue == ora.EPI_RELU and M * N >= 64:
        w = ora.widen(want, out_type)
        assert (w == 0).any() and (w > 0).any(), "test data must exercise both ReLU branches"
    return got


def _variants(b_layout):
    from accera_amd import _lib
    names = [(v, _lib.variant_name(v)) for v in range(_lib.num_variants())]
    key = " B=col-major" if b_layout == "col" else " B=row-major"
    return [(v, n) for v, n in names if key in n]


# ---- every MFMA variant, every input type, both B layouts --------------------------------
@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("bf16", "bf16"), ("i8", "i32")])
@pytest.mark.parametrize("b_layout", ["row", "col"])
def test_mfma_all_variants(in_type, out_type, b_layout):
    for v, name in _variants(b_layout):
        print("variant", v, name, in_type, b_layout, flush=True)
        # two tiles in each direction; K tile counts below, at and above the pipeline depth
        kb = int(re.search(r"kb(\d+)", name).group(1)) // (1 if in_type == "i8" else 2)
        a_layout = "col" if "A=col-major" in name else "row"
        bm, bn = map(int, re.search(r"mfma (\d+)x(\d+)", name).groups())
        M, N = max(512, 2 * bm), (max(512, 2 * bn) if 512 % bn == 0 else 3 * bn)
        # (the hand-laid loop takes at least four K tiles, the depth of its pipeline; every remainder modulo four enters
        # its four-step body at another position)
        for k_tiles in ((4, 5, 6, 7, 8, 9, 20) if "hand-laid" in name else (1, 2, 3, 7)):
            run_case(in_type, out_type, M, N, k_tiles * kb, b_layout=b_layout, variant=v, seed=v + k_tiles, a_layout=a_layout)
        if "edge" in name:
            # ragged M, N (multiple of the 16-byte vector only) and a K tail
            run_case(in_type, out_type, 208 if a_layout == "col" else 200, 144, 336 if in_type == "i8" else 176, b_layout=b_layout,
                     variant=v, seed=100 + v, a_layout=a_layout)


@pytest.mark.parametrize("out_type", ["i16", "i8"])
def test_mfma_all_variants_narrow_integer_outputs(out_type):
    """int8 -> int16 / int8 (pairs of the reference's tensor-core table, Targets.py:814-821; its tests
    mfma_tests.py:2117-2141): every tile geometry's write-back, overwriting and accumulating, with
    full-range data so that the kept low bits differ from the int32 sums."""
    for b_layout in ("row", "col"):
        for v, name in _variants(b_layout):
            print("variant", v, name, out_type, b_layout, flush=True)
            kb = int(re.search(r"kb(\d+)", name).group(1))
            a_layout = "col" if "A=col-major" in name else "row"
            bm, bn = map(int, re.search(r"mfma (\d+)x(\d+)", name).groups())
            M, N = max(512, 2 * bm), (max(512, 2 * bn) if 512 % bn == 0 else 3 * bn)
            if "hand-laid" in name:  # C = A*B and relu(A*B) only, K in steps of four tiles
                run_case("i8", out_type, M, N, 4 * kb, b_layout=b_layout, variant=v, seed=v, a_layout=a_layout)
                run_case("i8", out_type, M, N, 12 * kb, b_layout=b_layout, variant=v, seed=v + 1, epilogue=ora.EPI_NONE, a_layout=a_layout)
                continue
            run_case("i8", out_type, M, N, 2 * kb, b_layout=b_layout, variant=v, seed=v, a_layout=a_layout)
            run_case("i8", out_type, M, N, 3 * kb, b_layout=b_layout, variant=v, seed=v + 1, a_layout=a_layout, prologue=ora.PRO_NONE)
            if "edge" in name:
                run_case("i8", out_type, 208 if a_layout == "col" else 200, 144, 336, b_layout=b_layout, variant=v, seed=50 + v,
                         a_layout=a_layout, prologue=ora.PRO_NONE)


def test_narrow_integer_outputs_known_answers():
    """Closed forms: sums past the output range keep their low bits; C widens with its sign."""
    import accera_amd as acc
    import torch
    M = N = 256
    K = 512
    ones = np.ones((M, K), np.int8)
    for out_type, np_t, bits in (("i16", np.int16, 16), ("i8", np.int8, 8)):
        # K * 127 = 65024: 0xFE00 -> -512 as int16, 0x00 -> 0 as int8
        dC = to_device(np.zeros((M, N), np_t), out_type)
        acc.gemm_relu(to_device(ones, "i8"), to_device(np.full((K, N), 127, np.int8), "i8"), dC, epilogue=acc.EPILOGUE_NONE)
        torch.cuda.synchronize()
        want = ((K * 127 + 2 ** (bits - 1)) % 2 ** bits) - 2 ** (bits - 1)
        assert np.all(to_host(dC, out_type) == want), (out_type, want)
        # C = -1 everywhere (all bits set) must count as -1, not 255 / 65535: -1 + K*1 = 511
        dC = to_device(np.full((M, N), -1, np_t), out_type)
        acc.gemm_relu(to_device(ones, "i8"), to_device(np.ones((K, N), np.int8), "i8"), dC, prologue=acc.PROLOGUE_NONE)
        torch.cuda.synchronize()
        want = ((511 + 2 ** (bits - 1)) % 2 ** bits) - 2 ** (bits - 1)
        assert np.all(to_host(dC, out_type) == want), (out_type, want)


@pytest.mark.parametrize("in_type,out_type", PAIRS)
def test_mfma_auto_output_types(in_type, out_type):
    run_case(in_type, out_type, 256, 384, 512, seed=3)
    run_case(in_type, out_type, 256, 384, 512, seed=4, prologue=ora.PRO_NONE)
    run_case(in_type, out_type, 256, 384, 512, seed=5, epilogue=ora.EPI_RELU_NOCOND, b_layout="col")
    run_case(in_type, out_type, 256, 384, 512, seed=6, epilogue=ora.EPI_NONE, prologue=ora.PRO_NONE)


def test_column_major_a_takes_the_mfma_kernels():
    """Column-major A (the transA rows of the reference's sweep lists, tools/benchmarkers/gemm_*.csv)
    is chosen automatically and matches; so is a transposed view of a row-major tensor."""
    from accera_amd import _lib
    for in_type, out_type in [("f16", "f32"), ("bf16", "bf16"), ("i8", "i32")]:
        for b_layout in ("row", "col"):
            run_case(in_type, out_type, 512, 768, 1024, a_layout="col", b_layout=b_layout, seed=11)
            run_case(in_type, out_type, 384, 128, 256, a_layout="col", b_layout=b_layout, seed=12, prologue=ora.PRO_NONE)
    g, b, lds, v = _lib.launch_geometry(_lib.F16, _lib.F32, 4096, 4096, 4096, (1, 4096), (4096, 1), (4096, 1))
    assert "A=col-major" in _lib.variant_name(v) and "hand-laid" in _lib.variant_name(v)


@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("f16", "f16"), ("bf16", "bf16"), ("i8", "i32"), ("i8", "i8")])
@pytest.mark.parametrize("b_layout", ["row", "col"])
def test_four_wave_kernel_column_major_a(in_type, out_type, b_layout):
    """The hand-laid kernel's form for a column-major A (staged as it lies in memory, read with the transposing LDS
    loads), named explicitly: every position the K loop can be entered at, both wave rows and columns, C overwritten
    and accumulated into, ragged M and N, and views of larger matrices (fill strides that differ from the extents)."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    kb = 64 if in_type == "i8" else 32
    vec = 16 if in_type == "i8" else 8
    variants = [v for v, n in _variants(b_layout) if "hand-laid" in n and "A=col-major" in n]
    assert len(variants) == 2  # one tile per workgroup, and the form that walks several tiles
    for v in variants:
        _column_major_a_cases(v, in_type, out_type, b_layout, kb, vec)


def _column_major_a_cases(v, in_type, out_type, b_layout, kb, vec):
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    for k_tiles, epi in ((4, ora.EPI_RELU), (5, ora.EPI_NONE), (6, ora.EPI_RELU), (7, ora.EPI_RELU), (8, ora.EPI_NONE), (21, ora.EPI_RELU)):
        print("variant", v, in_type, out_type, b_layout, "k tiles", k_tiles, flush=True)
        run_case(in_type, out_type, 512, 768, k_tiles * kb, a_layout="col", b_layout=b_layout, variant=v, seed=900 + k_tiles, epilogue=epi)
    if out_type != "i8":
        print("variant", v, in_type, out_type, b_layout, "accumulating", flush=True)
        run_case(in_type, out_type, 512, 512, 6 * kb, a_layout="col", b_layout=b_layout, variant=v, seed=931, prologue=ora.PRO_NONE)
    # ragged M (a multiple of the 16-byte vector: the last row of tiles starts at M - 256) and ragged N
    print("variant", v, in_type, out_type, b_layout, "ragged", flush=True)
    run_case(in_type, out_type, 256 + 5 * vec, 512 + 3 * 16, 8 * kb, a_layout="col", b_layout=b_layout, variant=v, seed=932)
    with pytest.raises(_lib.Acc950Error):  # the last row of tiles would start in the middle of a 16-byte piece of A's columns
        run_case(in_type, out_type, 256 + vec // 2, 512, 8 * kb, a_layout="col", b_layout=b_layout, variant=v, seed=933)
    # views: A is the transpose of the first M columns of a wider K x (M + pad) array
    rng = np.random.default_rng(934)
    M, N, K = 512, 512, 6 * kb
    Abig = make_input(rng, (K, M + 3 * vec), in_type)
    Bbig = make_input(rng, (N, K + vec) if b_layout == "col" else (K, N + 2 * vec), in_type)
    Bview = Bbig[:, :K].T if b_layout == "col" else Bbig[:, :N]
    Cbig = make_c0(rng, (M, N + 16), out_type)
    dA, dB, dC = to_device(Abig, in_type), to_device(Bbig, in_type), to_device(Cbig, out_type)
    print("variant", v, in_type, out_type, b_layout, "views", flush=True)
    acc.gemm_relu(dA[:, :M].t(), dB[:, :K].t() if b_layout == "col" else dB[:, :N], dC[:, :N], variant=v)
    torch.cuda.synchronize()
    got = to_host(dC, out_type)
    want = ora.gemm_relu_exact(np.ascontiguousarray(Abig[:, :M].T), np.ascontiguousarray(Bview), None, in_type, out_type)
    assert_matches(got[:, :N], want, out_type, K)
    assert np.array_equal(got[:, N:], Cbig[:, N:]), "columns beside the view were written"


def test_mfma_single_k_tile_and_many_tiles():
    run_case("f16", "f32", 128, 128, 64, seed=7)          # K loop runs once (no prefetch)
    run_case("f16", "f32", 1024, 1536, 128, seed=8)       # many tiles: exercises the XCD / group remap
    run_case("i8", "i32", 768, 1280, 256, seed=9, variant=5)  # tile count not a multiple of 8 XCDs
    run_case("bf16", "f32", 1280, 768, 1024, seed=10)     # reference size 1280x768x1024 (mfma_tests.py:2007-2272)


def test_mfma_tile_map_covers_every_tile_once():
    """Identity-like check of the workgroup -> tile map: C = A @ I must reproduce A in
    every tile, for tile grids that are / are not multiples of the XCD count and group size."""
    import accera_amd as acc
    import torch
    for (M, N) in [(256, 128), (640, 384), (1152, 1664), (2048, 2048)]:
        K = N
        rng = np.random.default_rng(M + N)
        A = make_input(rng, (M, K), "f16")
        I = np.eye(K, N, dtype=np.float16)
        dC = to_device(out_zeros(M, N, "f32"), "f32")
        acc.gemm_relu(to_device(A, "f16"), to_device(I, "f16"), dC, epilogue=acc.EPILOGUE_NONE)
        torch.cuda.synchronize()
        assert np.array_equal(to_host(dC, "f32"), A.astype(np.float32)), (M, N)


# ---- edge kernel and generic kernel: sizes of the reference's boundary tests ---------------
@pytest.mark.parametrize("shape", [(16, 16, 1264), (64, 64, 96), (960, 1024, 1024), (100, 72, 40), (16, 16, 16), (128, 16, 16)])
@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("bf16", "f32"), ("i8", "i32")])
def test_boundary_shapes(shape, in_type, out_type):
    M, N, K = shape  # 16x16x1264: mfma_tests.py:2242-2272; 16/128 x K=16: :2579-2602
    run_case(in_type, out_type, M, N, K, seed=sum(shape))


@pytest.mark.parametrize("in_type,out_type", PAIRS + [("f32", "f32")])
@pytest.mark.parametrize("shape", [(33, 47, 29), (1, 1, 1), (65, 130, 7), (64, 93, 64)])
def test_generic_kernel_any_shape(in_type, out_type, shape):
    M, N, K = shape
    run_case(in_type, out_type, M, N, K, variant=200, seed=sum(shape))
    run_case(in_type, out_type, M, N, K, variant=200, seed=sum(shape) + 1, b_layout="col", c_layout="col", prologue=ora.PRO_NONE)


def test_column_major_c_uses_transposed_product():
    run_case("f16", "f32", 256, 384, 256, c_layout="col", seed=21)
    run_case("i8", "i32", 256, 384, 256, c_layout="col", b_layout="col", seed=22)
    run_case("bf16", "bf16", 384, 256, 192, c_layout="col", seed=23, prologue=ora.PRO_NONE)


def test_strided_views_with_padding():
    """Leading dimensions larger than the logical width (sub-matrix views)."""
    import accera_amd as acc
    import torch
    rng = np.random.default_rng(31)
    M, N, K = 256, 256, 192
    Abig = make_input(rng, (M, K + 64), "f16")
    Bbig = make_input(rng, (K, N + 128), "f16")
    Cbig = np.full((M, N + 8), -5.0, np.float32)
    dA, dB, dC = to_device(Abig, "f16"), to_device(Bbig, "f16"), to_device(Cbig, "f32")
    acc.gemm_relu(dA[:, :K], dB[:, :N], dC[:, :N])
    torch.cuda.synchronize()
    got = to_host(dC, "f32")
    want = ora.gemm_relu_exact(Abig[:, :K], Bbig[:, :N], None, "f16", "f32")
    assert_matches(got[:, :N], want, "f32", K)
    assert np.all(got[:, N:] == -5.0)  # padding untouched


@pytest.mark.parametrize("in_type,out_type,pad", [("f16", "f32", 3), ("f16", "f16", 8), ("f16", "f16", 3), ("bf16", "bf16", 5),
                                                  ("i8", "i32", 1), ("i8", "i16", 3), ("i8", "i16", 8), ("i8", "i8", 16),
                                                  pytest.param("i8", "i8", 7, marks=pytest.mark.skip(
                                                      reason="byte-wise stores to rows at odd distances faulted the GPU in the large-tile kernel; cause "
                                                             "not found, path switched off: the library now refuses the variant for such a C"))])
def test_large_tile_kernels_on_padded_output_rows(in_type, out_type, pad):
    """Every store path of the 16x16-shape kernels: rows of C that are / are not 16-byte multiples apart
    (whole-row pieces through LDS, or single elements), overwriting and accumulating, padding untouched."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    mi16 = [v for v in range(_lib.num_variants()) if "mi16" in _lib.variant_name(v) and "256x256 kb64" in _lib.variant_name(v)
            and "B=row-major" in _lib.variant_name(v) and "A=col" not in _lib.variant_name(v)]
    assert mi16
    M, N, K = 512, 256, 256
    rng = np.random.default_rng(500 + pad)
    A, B = make_input(rng, (M, K), in_type), make_input(rng, (K, N), in_type)
    fill = 77 if out_type in INT_OUT else None
    for prologue in (ora.PRO_SET0, ora.PRO_NONE):
        Cbig = make_c0(rng, (M, N + pad), out_type)
        dC = to_device(Cbig, out_type)
        acc.gemm_relu(to_device(A, in_type), to_device(B, in_type), dC[:, :N], prologue=prologue, variant=mi16[0])
        torch.cuda.synchronize()
        got = to_host(dC, out_type)
        want = ora.gemm_relu_exact(A, B, np.ascontiguousarray(Cbig[:, :N]), in_type, out_type, prologue, ora.EPI_RELU)
        assert_matches(got[:, :N], want, out_type, K)
        assert np.array_equal(got[:, N:], Cbig[:, N:]), "padding columns were written"


def _hand_laid(b_layout):
    from accera_amd import _lib
    return next(v for v, n in _variants(b_layout) if "hand-laid" in n and "A=col-major" not in n)


@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("f16", "f16"), ("bf16", "bf16"), ("bf16", "f32"),
                                              ("i8", "i32"), ("i8", "i16"), ("i8", "i8")])
@pytest.mark.parametrize("b_layout", ["row", "col"])
def test_four_wave_kernel_every_output_type(in_type, out_type, b_layout):
    """The kernel with the hand-laid K loop (accumulators pinned in the AGPR file): both epilogues it
    takes, every store path (32-bit straight from the accumulator registers, narrow types through
    LDS), 6 output tiles so that the tile map and both wave rows / columns are exercised, K at one,
    two and five rounds of the four LDS stages."""
    kb = 64 if in_type == "i8" else 32
    for v in [v for v, n in _variants(b_layout) if "hand-laid" in n and "A=col-major" not in n]:  # 256x256, and 256x192 for column-major B
        for k_tiles, epi in ((4, ora.EPI_RELU), (8, ora.EPI_NONE), (20, ora.EPI_RELU)):
            print("variant", v, in_type, out_type, b_layout, "k tiles", k_tiles, flush=True)
            run_case(in_type, out_type, 512, 768, k_tiles * kb, b_layout=b_layout, variant=v, seed=700 + k_tiles, epilogue=epi)
        if out_type != "i8":
            # C += A*B: the tile of C is loaded (16-bit types: widened) into the accumulator registers before the loop
            for k_tiles, epi in ((4, ora.EPI_NONE), (12, ora.EPI_RELU)):
                print("variant", v, in_type, out_type, b_layout, "accumulating, k tiles", k_tiles, flush=True)
                run_case(in_type, out_type, 512, 768, k_tiles * kb, b_layout=b_layout, variant=v, seed=720 + k_tiles, epilogue=epi,
                         prologue=ora.PRO_NONE)


@pytest.mark.parametrize("in_type,out_type,b_layout", [("f16", "f32", "row"), ("bf16", "bf16", "col"), ("i8", "i32", "row"), ("i8", "i8", "col")])
def test_four_wave_kernel_on_views_of_larger_matrices(in_type, out_type, b_layout):
    """Leading dimensions larger than the logical widths (every fill stride and the row stride of C differ from
    the tile's extent), overwriting and accumulating; what lies beside the views stays as it was."""
    import accera_amd as acc
    import torch
    rng = np.random.default_rng(41)
    M, N, K = 512, 768, 256 if in_type == "i8" else 384
    esz = 1 if in_type == "i8" else 2
    for v in [v for v, n in _variants(b_layout) if "hand-laid" in n and "A=col-major" not in n]:
        Abig = make_input(rng, (M, K + 128 // esz), in_type)
        Bbig = make_input(rng, (N, K + 64 // esz) if b_layout == "col" else (K, N + 256 // esz), in_type)
        Bview = Bbig[:, :K].T if b_layout == "col" else Bbig[:, :N]
        pad_c = 16 if out_type == "i8" else 8
        for prologue in ((ora.PRO_SET0, ora.PRO_NONE) if out_type != "i8" else (ora.PRO_SET0,)):
            Cbig = make_c0(rng, (M, N + pad_c), out_type)
            dA, dB, dC = to_device(Abig, in_type), to_device(Bbig, in_type), to_device(Cbig, out_type)
            dBv = dB[:, :K].t() if b_layout == "col" else dB[:, :N]
            print("variant", v, in_type, out_type, b_layout, "prologue", prologue, flush=True)
            acc.gemm_relu(dA[:, :K], dBv, dC[:, :N], prologue=prologue, variant=v)
            torch.cuda.synchronize()
            got = to_host(dC, out_type)
            want = ora.gemm_relu_exact(np.ascontiguousarray(Abig[:, :K]), np.ascontiguousarray(Bview), np.ascontiguousarray(Cbig[:, :N]),
                                       in_type, out_type, prologue, ora.EPI_RELU)
            assert_matches(got[:, :N], want, out_type, K)
            assert np.array_equal(got[:, N:], Cbig[:, N:]), "columns beside the view were written"


@pytest.mark.parametrize("in_type,out_type,M", [("f16", "f32", 600), ("bf16", "bf16", 1000), ("i8", "i32", 257), ("f16", "f16", 511)])
def test_four_wave_kernel_any_number_of_rows(in_type, out_type, M):
    """M and N that are not multiples of the tile: the last row / column of tiles ends at M / N and overlaps the
    one before it, overwriting C and accumulating into it."""
    import accera_amd as acc
    from accera_amd import _lib
    kb = 64 if in_type == "i8" else 32
    for b_layout in ("row", "col"):
        for v in [v for v, n in _variants(b_layout) if "hand-laid" in n and "A=col-major" not in n]:
            print("variant", v, in_type, out_type, b_layout, "M", M, flush=True)
            run_case(in_type, out_type, M, 768, 8 * kb, b_layout=b_layout, variant=v, seed=M)
            run_case(in_type, out_type, M, 768 + 16 + 64 * (M % 3), 4 * kb, b_layout=b_layout, variant=v, seed=M + 1)  # N ragged too
            # C += A*B with such sizes: the moved tiles leave what they share with their neighbours to the neighbours
            run_case(in_type, out_type, M, 768, 8 * kb, b_layout=b_layout, variant=v, seed=M + 2, prologue=ora.PRO_NONE)
            run_case(in_type, out_type, M, 768 + 16 + 64 * (M % 3), 5 * kb, b_layout=b_layout, variant=v, seed=M + 3, prologue=ora.PRO_NONE,
                     epilogue=ora.EPI_NONE)
    with pytest.raises(_lib.Acc950Error):  # fewer rows than one tile
        run_case(in_type, out_type, 200, 768, 8 * kb, variant=_hand_laid("row"))


def test_four_wave_kernel_is_refused_for_what_it_does_not_take():
    """Reading an int8 C (accumulating into it, scaling it) and a K of fewer than four tiles go to the other
    kernels: naming the variant for them is an error, never a wrong result."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    v = _hand_laid("row")
    rng = np.random.default_rng(5)
    A, B = make_input(rng, (256, 96), "f16"), make_input(rng, (96, 256), "f16")
    dC = to_device(np.zeros((256, 256), np.float32), "f32")
    with pytest.raises(_lib.Acc950Error):
        acc.gemm_relu(to_device(A, "f16"), to_device(B, "f16"), dC, variant=v)  # K = 3 tiles: fewer than the pipeline is deep
    A, B = make_input(rng, (256, 128), "f16"), make_input(rng, (128, 256), "f16")
    for kw in (dict(prologue=acc.PROLOGUE_NONE), dict(prologue=acc.PROLOGUE_SCALE, prologue_arg=2.0)):  # reading an int8 C
        with pytest.raises(_lib.Acc950Error):
            acc.gemm_relu(to_device(np.ones((256, 256), np.int8), "i8"), to_device(np.ones((256, 256), np.int8), "i8"),
                          to_device(np.zeros((256, 256), np.int8), "i8"), variant=v, **kw)
    acc.gemm_relu(to_device(A, "f16"), to_device(B, "f16"), dC, variant=v)  # and what it does take still runs
    torch.cuda.synchronize()
    assert_matches(to_host(dC, "f32"), ora.gemm_relu_exact(A, B, np.zeros((256, 256), np.float32), "f16", "f32", ora.PRO_SET0, ora.EPI_RELU), "f32", 128)


def test_int8_output_rows_at_odd_distances_take_the_thread_bound_kernel():
    """int8 C whose rows are not 16 bytes apart: every MFMA variant refuses, the automatic choice falls back."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    M, N, K, pad = 512, 256, 256, 7
    g, b, lds, v = _lib.launch_geometry(_lib.I8, _lib.I8, M, N, K, (K, 1), (N, 1), (N + pad, 1))
    assert v == _lib.VARIANT_GENERIC
    with pytest.raises(_lib.Acc950Error):
        _lib.launch_geometry(_lib.I8, _lib.I8, M, N, K, (K, 1), (N, 1), (N + pad, 1), 0, 0)
    rng = np.random.default_rng(507)
    A, B = make_input(rng, (M, K), "i8"), make_input(rng, (K, N), "i8")
    Cbig = make_c0(rng, (M, N + pad), "i8")
    dC = to_device(Cbig, "i8")
    acc.gemm_relu(to_device(A, "i8"), to_device(B, "i8"), dC[:, :N], prologue=acc.PROLOGUE_NONE)
    torch.cuda.synchronize()
    got = to_host(dC, "i8")
    assert_matches(got[:, :N], ora.gemm_relu_exact(A, B, np.ascontiguousarray(Cbig[:, :N]), "i8", "i8", ora.PRO_NONE, ora.EPI_RELU), "i8", K)
    assert np.array_equal(got[:, N:], Cbig[:, N:])


# ---- fp32 kernel ------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(512, 512, 512), (64, 32, 8), (100, 70, 52), (33, 47, 29), (256, 256, 1000)])
@pytest.mark.parametrize("b_layout", ["row", "col"])
def test_f32_mfma_kernel(shape, b_layout):
    M, N, K = shape
    got = run_case("f32", "f32", M, N, K, b_layout=b_layout, seed=41)
    # fp32 products: must be far better than a reduced-precision input path could give
    rng = np.random.default_rng(41)
    A, B = make_input(rng, (M, K), "f32"), make_input(rng, (K, N), "f32")
    want = np.maximum(A.astype(np.float64) @ B.astype(np.float64), 0)
    assert np.abs(got - want).max() < 1e-4 * max(1, np.sqrt(K) / 8)
    run_case("f32", "f32", M, N, K, b_layout=b_layout, seed=42, prologue=ora.PRO_NONE, epilogue=ora.EPI_RELU_NOCOND)


def test_readme_quickstart_shape_and_data():
    """README.md:118-136: A,B ~ U[0,1) 512x512 fp32, C zeros, atol 1e-3."""
    import accera_amd as acc
    import torch
    rng = np.random.default_rng(1001)
    A = rng.random((512, 512), dtype=np.float32)
    B = rng.random((512, 512), dtype=np.float32)
    C = np.zeros((512, 512), np.float32)
    dC = to_device(C, "f32")
    acc.gemm_relu(to_device(A, "f32"), to_device(B, "f32"), dC, prologue=acc.PROLOGUE_NONE)
    torch.cuda.synchronize()
    np.testing.assert_allclose(to_host(dC, "f32"), np.maximum(C + A @ B, 0.0), atol=1e-3)


# ---- skinny streaming kernel -----------------------------------------------------------------
@pytest.mark.parametrize("in_type,out_type", [("f16", "f16"), ("f16", "f32"), ("bf16", "bf16")])
def test_skinny_all_variants_and_splits(in_type, out_type):
    from accera_amd import _lib
    names = [_lib.variant_name(100 + sv) for sv in range(_lib.num_skinny_variants())]
    for sv, name in enumerate(names):
        for splits in (1, 3, 8):
            print("skinny", sv, name, "splits", splits, flush=True)
            run_case(in_type, out_type, 8, 1024 + 64, 1024, variant=100 + sv, splits=splits, seed=sv * 10 + splits, dist="normal")
    mfma = 100 + next(i for i, n in enumerate(names) if "mfma" in n)
    dot2 = 100 + next(i for i, n in enumerate(names) if "dot2" in n)
    # matrix-core family: up to 32 rows of A; ragged M, N not a multiple of the column block,
    # fewer k steps than waves, more splits than steps allow
    run_case(in_type, out_type, 32, 1024 + 64, 1024, variant=mfma, splits=2, seed=70, dist="normal")
    run_case(in_type, out_type, 17, 1000, 1008, variant=mfma, splits=4, seed=71, dist="normal")
    run_case(in_type, out_type, 1, 8, 16, variant=mfma, splits=1, seed=72, dist="normal", epilogue=ora.EPI_NONE)
    run_case(in_type, out_type, 3, 72, 48, variant=mfma, splits=8, seed=73, dist="normal")
    # dot-product family: M < 8, K not a multiple of the k step
    run_case(in_type, out_type, 5, 1000, 998, variant=dot2, splits=4, seed=77, dist="normal")
    run_case(in_type, out_type, 1, 8, 2, variant=dot2, splits=1, seed=78, dist="normal", epilogue=ora.EPI_NONE)
    # automatic choice: K % 16 != 0 falls to the dot-product family; accumulate into C
    run_case(in_type, out_type, 5, 1000, 998, seed=74, dist="normal")
    run_case(in_type, out_type, 8, 2048, 512, seed=79, dist="normal", prologue=ora.PRO_NONE)
    run_case(in_type, out_type, 24, 2048, 512, seed=80, dist="normal", prologue=ora.PRO_NONE, epilogue=ora.EPI_RELU_NOCOND)


@pytest.mark.parametrize("in_type,out_type,M,N,K,cols,splits,prologue", [
    ("f16", "f16", 8, 22016, 4096, 256, 2, ora.PRO_SET0),     # 86 wide blocks in two slices: 172 workgroups
    ("bf16", "f32", 16, 16384, 16384, 256, 4, ora.PRO_NONE),  # accumulates into C
    ("f16", "f32", 5, 40960 + 72, 1024, 256, 1, ora.PRO_SET0),  # enough wide blocks without a split; the last block is ragged
    ("i8", "i32", 8, 12288, 8192, 256, 4, ora.PRO_SET0),
    ("i8", "i16", 32, 8192, 16384, 256, 4, ora.PRO_SET0),
    ("f16", "f16", 8, 16384, 4096, 64, 1, ora.PRO_SET0),      # two slices would fill half the chip: the default form
])
def test_decode_shapes_take_the_wide_blocks_of_the_streaming_kernel(in_type, out_type, M, N, K, cols, splits, prologue):
    """Few rows of A against a large B: the library by itself takes the streaming kernel's 256-column blocks, with the K split
    that fills the chip in one round, where they measured ahead of the 64-column default; results against the oracle."""
    from accera_amd import _lib, tune
    n_in, n_out = {"f16": _lib.F16, "bf16": _lib.BF16, "i8": _lib.I8}[in_type], {"f16": _lib.F16, "f32": _lib.F32, "i32": _lib.I32, "i16": _lib.I16}[out_type]
    variant, slices = tune.own_choice(n_in, n_out, M, N, K, False, False, 1.0, 1.0 if prologue == ora.PRO_NONE else 0.0)
    assert f"skinny mfma cols/wg={cols} " in _lib.variant_name(variant) and slices == splits, (_lib.variant_name(variant), slices)
    run_case(in_type, out_type, M, N, K, seed=N % 97 + K % 89, dist="normal", prologue=prologue)


@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("bf16", "bf16"), ("i8", "i32"), ("i8", "i8"), ("f32", "f32")])
def test_small_tiles_with_direct_fills_take_fewer_rows_than_a_tile(in_type, out_type):
    """The tiles with direct fills (32x32 instruction shapes) on fewer rows of a row-major A than they have: the fills of the missing rows fetch A's last row, and
    what comes of them is dropped by the range check on C.  Both layouts of B, C written and accumulated into; the rows of C
    behind the last one (a larger allocation, poisoned) must stay as they are."""
    import torch
    from accera_amd import _lib
    small = [(v, _lib.variant_name(v)) for v in range(_lib.num_variants())]
    small = [(v, n) for v, n in small if "fill=direct" in n and "A=col-major" not in n and "mi16" not in n and "edge" not in n]
    assert len(small) >= 10
    for v, name in small:
        b_layout = "col" if "B=col-major" in name else "row"
        bm, bn = map(int, re.search(r"mfma (\d+)x(\d+)", name).groups())
        for M in ((1, 8, 33, 63) if bm == 64 else (5, 65, 127) if bm == 128 else (3, 129, 255)):
            for pro, epi in ((ora.PRO_SET0, ora.EPI_RELU), (ora.PRO_NONE, ora.EPI_NONE)):
                if out_type == "i8" and pro == ora.PRO_NONE:
                    continue
                print(name, in_type, out_type, M, pro, flush=True)
                run_case(in_type, out_type, M, 3 * bn, 512, b_layout=b_layout, variant=v, prologue=pro, epilogue=epi, seed=M + v, dist="normal")
    # C as the first rows of a taller matrix: nothing behind row M may change
    v = next(v for v, n in small if "mfma 64x64" in n)
    rng = np.random.default_rng(9)
    M, N, K = 5, 128, 256
    A, B = make_input(rng, (M, K), in_type, "normal"), make_input(rng, (K, N), in_type, "normal")
    full = to_device(np.full((64, N), 3, ora.NP_STORAGE[out_type]), out_type)
    import accera_amd as acc
    acc.gemm_relu(to_device(A, in_type), to_device(B, in_type), full[:M], variant=v)
    torch.cuda.synchronize()
    got = to_host(full, out_type)
    assert (got[M:] == np.full((64 - M, N), 3, ora.NP_STORAGE[out_type])).all()
    assert_matches(got[:M], ora.gemm_relu_exact(A, B, out_zeros(M, N, out_type), in_type, out_type, ora.PRO_SET0, ora.EPI_RELU), out_type, K)
    # A and C as the left columns of wider matrices (rows further apart than they are long), and a batch of such problems
    batch, pad = 3, 64
    As = np.stack([make_input(rng, (M, K + pad), in_type, "normal") for _ in range(batch)])
    Bs = np.stack([make_input(rng, (K, N), in_type, "normal") for _ in range(batch)])
    dA = torch.stack([to_device(a, in_type) for a in As])[:, :, :K]
    dB = torch.stack([to_device(b, in_type) for b in Bs])
    dC = torch.stack([to_device(np.full((M, N + 16), 3, ora.NP_STORAGE[out_type]), out_type) for _ in range(batch)])
    assert dA.stride(1) == K + pad and dC.stride(1) == N + 16
    acc.gemm_relu(dA, dB, dC[:, :, :N], variant=v)
    torch.cuda.synchronize()
    for b in range(batch):
        got = to_host(dC[b], out_type)
        assert (got[:, N:] == 3).all()
        want = ora.gemm_relu_exact(np.ascontiguousarray(As[b][:, :K]), Bs[b], out_zeros(M, N, out_type), in_type, out_type, ora.PRO_SET0, ora.EPI_RELU)
        assert_matches(got[:, :N], want, out_type, K)


@pytest.mark.parametrize("in_type,out_type,M,N,K,b_layout,tile,splits,prologue", [
    ("f16", "f16", 33, 8192, 12288, "row", "64x64", 4, ora.PRO_SET0),       # fewer rows than the 64-row tile has: direct fills all the same
    ("f16", "f16", 100, 8192, 12288, "row", "128x128", 4, ora.PRO_SET0),    # 128-row tiles on 100 rows, direct fills: 64 of them in four slices
    ("f16", "f16", 8, 11008, 4096, "col", "64x64", 1, ora.PRO_SET0),        # a decode step against a K-contiguous B (the streaming kernels want a row-major one)
    ("bf16", "bf16", 1, 8192, 12288, "col", "64x64", 4, ora.PRO_NONE),      # one row
    ("bf16", "f32", 128, 12288, 8192, "row", "128x128", 2, ora.PRO_NONE),   # 96 tiles with direct fills in two slices, accumulating into C
    ("f16", "f16", 64, 8192, 12288, "col", "64x64", 4, ora.PRO_SET0),
    ("i8", "i32", 256, 16384, 12288, "row", "256x256", 2, ora.PRO_SET0),    # the four-wave kernel, K split
    ("f16", "f32", 200, 12288, 8192, "row", "128x128", 1, ora.PRO_SET0),    # two rows of 128 x 128 tiles: 192 tiles stream by themselves
    ("f16", "f16", 48, 11008, 4096, "row", "64x64", 1, ora.PRO_SET0),       # 86 MB: the general rule's tiles (172 of them stream by themselves)
])
def test_many_column_problems_with_few_rows_stream_b_once(in_type, out_type, M, N, K, b_layout, tile, splits, prologue):
    """A few dozen to a few hundred rows of A against a B beyond the caches: the library takes a tile as tall as A and the
    K slices that give the memory system enough workgroups; results against the oracle."""
    from accera_amd import _lib, tune
    ids = {"f16": _lib.F16, "bf16": _lib.BF16, "i8": _lib.I8, "f32": _lib.F32, "i32": _lib.I32}
    variant, slices = tune.own_choice(ids[in_type], ids[out_type], M, N, K, False, b_layout == "col", 1.0, 1.0 if prologue == ora.PRO_NONE else 0.0)
    name = _lib.variant_name(variant)
    assert f"mfma {tile} " in name and slices == splits, (name, slices)
    run_case(in_type, out_type, M, N, K, b_layout=b_layout, seed=M + N % 91, dist="normal", prologue=prologue)


@pytest.mark.parametrize("out_type", ["i32", "i16", "i8"])
def test_skinny_int8_streaming_kernels(out_type):
    """int8 rows of A against a large row-major int8 B on the streaming kernels of the matrix-core family
    (v_mfma_i32_32x32x32_i8, 32 k rows per step), bit-exact against the oracle: every variant x K splits, ragged M / N, a K of
    one step, accumulation into C, and the automatic choice for the decode shape."""
    from accera_amd import _lib
    names = [_lib.variant_name(100 + sv) for sv in range(_lib.num_skinny_variants())]
    mfma = [100 + i for i, n in enumerate(names) if "mfma" in n]
    for v in mfma:
        for splits in (1, 3, 8):
            print("skinny int8", v, names[v - 100], "splits", splits, flush=True)
            run_case("i8", out_type, 8, 1024 + 64, 1024, variant=v, splits=splits, seed=v * 10 + splits)
    run_case("i8", out_type, 32, 1024 + 64, 2048, variant=mfma[0], splits=2, seed=170)
    run_case("i8", out_type, 17, 1008, 992, variant=mfma[0], splits=4, seed=171)
    run_case("i8", out_type, 1, 16, 32, variant=mfma[0], splits=1, seed=172, epilogue=ora.EPI_NONE)
    run_case("i8", out_type, 3, 80, 96, variant=mfma[0], splits=8, seed=173)
    if out_type != "i8":  # (an int8 C is only written)
        run_case("i8", out_type, 8, 2048, 512, seed=179, prologue=ora.PRO_NONE)
        run_case("i8", out_type, 24, 2048, 512, seed=180, prologue=ora.PRO_NONE, epilogue=ora.EPI_RELU_NOCOND)
    # the dot-product family has no int8 form
    dot2 = 100 + next(i for i, n in enumerate(names) if "dot2" in n)
    with pytest.raises(_lib.Acc950Error) as e:
        _lib.launch_geometry(_lib.I8, _lib.I32, 8, 1024, 1024, (1024, 1), (1024, 1), (1024, 1), variant=dot2)
    assert e.value.code == _lib.UNSUPPORTED
    # automatic choice: the decode shape in int8 streams on the matrix-core family
    grid, block, lds, v = _lib.launch_geometry(_lib.I8, getattr(_lib, out_type.upper()), 8, 11008, 4096, (4096, 1), (11008, 1), (11008, 1))
    assert "skinny mfma" in _lib.variant_name(v)
    run_case("i8", out_type, 8, 11008, 4096, seed=181)


def test_skinny_repeated_launches_reuse_counters():
    """The K-split arrival counters must return to zero after every launch."""
    for rep in range(3):
        run_case("f16", "f16", 8, 4096, 2048, variant=100, splits=8, seed=90 + rep, dist="normal")
    run_case("f16", "f16", 8, 512, 2048, variant=103, splits=5, seed=95, dist="normal")
    run_case("f16", "f16", 8, 11008, 4096, splits=7, seed=96, dist="normal")  # the decode shape itself


# ---- closed forms: bit-exact expectations ------------------------------------------------------
@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("bf16", "f32"), ("i8", "i32"), ("f32", "f32")])
def test_permutation_matrix_is_bit_exact(in_type, out_type):
    import accera_amd as acc
    import torch
    rng = np.random.default_rng(51)
    M, K = 256, 256
    A = make_input(rng, (M, K), in_type)
    perm = rng.permutation(K)
    P = np.zeros((K, K), np.float32)
    P[perm, np.arange(K)] = 1
    Pm = {"f32": P, "f16": P.astype(np.float16), "bf16": ora.to_bf16(P), "i8": P.astype(np.int8)}[in_type]
    dC = to_device(out_zeros(M, K, out_type), out_type)
    acc.gemm_relu(to_device(A, in_type), to_device(Pm, in_type), dC)
    torch.cuda.synchronize()
    want = np.maximum(ora.widen(A, in_type)[:, perm], 0)
    assert np.array_equal(ora.widen(to_host(dC, out_type), out_type), want)


def test_reference_constant_fill_known_answers():
    """A=2, B=3, C=0.42 -> 6K + 0.42 (docs/Tutorials/Hello_MatMul.md:165-237, K=256;
    docs/Tutorials/Optimized_MatMul.md:204-280, K=128)."""
    import accera_amd as acc
    import torch
    for K, expected in [(256, 1536.42), (128, 768.42)]:
        for t in ("f32", "f16"):
            A = np.full((128, K), 2.0, ora.NP_STORAGE[t])
            B = np.full((K, 256), 3.0, ora.NP_STORAGE[t])
            dC = to_device(np.full((128, 256), 0.42, np.float32), "f32")
            acc.gemm_relu(to_device(A, t), to_device(B, t), dC, prologue=acc.PROLOGUE_NONE)
            torch.cuda.synchronize()
            np.testing.assert_allclose(to_host(dC, "f32"), expected, rtol=1e-6)


def test_int8_extremes_are_exact():
    import accera_amd as acc
    import torch
    M = N = 256
    K = 1024
    A = np.full((M, K), -128, np.int8)
    B = np.full((K, N), -128, np.int8)
    dC = to_device(out_zeros(M, N, "i32"), "i32")
    acc.gemm_relu(to_device(A, "i8"), to_device(B, "i8"), dC)
    torch.cuda.synchronize()
    assert np.all(to_host(dC, "i32") == K * 16384)
    B[:] = 127
    dC = to_device(out_zeros(M, N, "i32"), "i32")
    acc.gemm_relu(to_device(A, "i8"), to_device(B, "i8"), dC, epilogue=acc.EPILOGUE_NONE)
    torch.cuda.synchronize()
    assert np.all(to_host(dC, "i32") == -K * 128 * 127)


@pytest.mark.parametrize("variant", [-1, 200])
@pytest.mark.parametrize("epi", [ora.EPI_RELU, ora.EPI_RELU_NOCOND])
def test_relu_special_values(variant, epi):
    """epilogue(C0 + 0): relu maps NaN, -0, -inf to +0; relu_no_conditional keeps NaN and
    turns -inf into NaN (-inf * 0).  CppPrinterUtils.h:630-643."""
    import accera_amd as acc
    import torch
    M, N, K = 128, 128, 64
    vals = np.array([-0.0, np.nan, np.inf, -np.inf, -3.5, 2.25, 0.0, 1e-38], np.float32)
    C0 = np.tile(vals, (M, N // len(vals)))
    A = np.zeros((M, K), np.float16)
    B = np.zeros((K, N), np.float16)
    dC = to_device(C0, "f32")
    acc.gemm_relu(to_device(A, "f16"), to_device(B, "f16"), dC, prologue=acc.PROLOGUE_NONE, epilogue=epi, variant=variant)
    torch.cuda.synchronize()
    got = to_host(dC, "f32")
    want = C0.copy()
    ora.gemm_relu(A, B, want, "f16", "f32", prologue=ora.PRO_NONE, epilogue=epi)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok])
    assert np.array_equal(np.signbit(got[ok]), np.signbit(want[ok]))


@pytest.mark.parametrize("out_type", ["bf16", "f16"])
@pytest.mark.parametrize("variant,prologue", [(-1, ora.PRO_SET0), (-1, ora.PRO_NONE), (200, ora.PRO_SET0)])
def test_narrowing_store_rounds_to_nearest_even(out_type, variant, prologue):
    """x + y is exact in the float accumulator and lands on / next to a rounding tie of the
    16-bit output type: the store must round to nearest even, overflow to inf and keep NaN
    (the widen-accumulate-narrow rule, CppPrinterUtils.h:95-118 with LLVM's host rounding).
    Covers the packed (SET prologue) and the element-wise (accumulating, generic) stores."""
    import accera_amd as acc
    import torch
    in_type = "bf16" if out_type == "bf16" else "f16"
    mant = 7 if out_type == "bf16" else 10
    u = 2.0 ** -mant                       # ulp of the output type at 1.0
    big = (2 - u) * (2.0 ** 127 if out_type == "bf16" else 2.0 ** 15)   # largest finite
    pairs = [(1.0, u / 2), (1.0 + u, u / 2), (1.0, u / 2 * (1 + u)), (1.0 + u, u / 4), (-1.0, -u / 2), (-1.0 - u, -u / 2),
             (big, big * u / 4), (big, big), (-big, -big * u / 4), (np.inf, 1.0), (np.nan, 1.0), (3.0, -3.0), (0.375, u * 0.375 / 2),
             (1024.0, 1024 * 3 * u / 2), (1.0, 0.0), (-2.5, 0.0)]
    M, N, K = 128, 128, 32
    x = np.array([p[0] for p in pairs] * (M // len(pairs)), np.float32)
    y = np.array([p[1] for p in pairs] * (M // len(pairs)), np.float32)
    Af = np.zeros((M, K), np.float32)
    Af[:, 3], Af[:, 17] = x, y
    Bf = np.zeros((K, N), np.float32)
    Bf[3, :], Bf[17, :] = 1.0, 1.0
    A, B = ora.narrow(Af, in_type), ora.narrow(Bf, in_type)
    assert np.array_equal(ora.widen(A, in_type)[:, 3][~np.isnan(x)], x[~np.isnan(x)].astype(np.float64)), "inputs must be exact"
    C0 = ora.narrow(np.zeros((M, N), np.float32), out_type)
    dC = to_device(C0, out_type)
    acc.gemm_relu(to_device(A, in_type), to_device(B, in_type), dC, prologue=prologue, epilogue=acc.EPILOGUE_NONE, variant=variant)
    torch.cuda.synchronize()
    got = ora.widen(to_host(dC, out_type), out_type)
    want = ora.widen(ora.narrow(x + y, out_type), out_type)[:, None].repeat(N, 1)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok]), (got[:16, 0], want[:16, 0])


# ---- SET / SCALE fragment ops (GEMM alpha / beta table) through every kernel family ---------------------
OPS = [(ora.PRO_SET, 0.0, ora.EPI_SCALE, 5.0), (ora.PRO_SCALE, 0.5, ora.EPI_NONE, 0.0), (ora.PRO_SCALE, -2.0, ora.EPI_SCALE, 3.0),
       (ora.PRO_SET, -7.0, ora.EPI_RELU, 0.0), (ora.PRO_SET, 3.0, ora.EPI_RELU_NOCOND, 0.0), (ora.PRO_NONE, 0.0, ora.EPI_SET, 1.25),
       (ora.PRO_SCALE, 2.9, ora.EPI_SCALE, -3.7)]


@pytest.mark.parametrize("case", [("f16", "f32", 256, 512, 256, -1), ("bf16", "bf16", 256, 384, 128, -1), ("i8", "i32", 256, 256, 512, -1),
                                  ("i8", "i16", 256, 256, 512, -1), ("i8", "i8", 256, 512, 256, -1), ("i8", "i8", 33, 47, 29, -1),
                                  ("f16", "f16", 200, 144, 176, -1), ("f32", "f32", 96, 80, 72, -1), ("f16", "f32", 33, 47, 29, 200),
                                  ("f16", "f16", 8, 1088, 512, -1), ("bf16", "f32", 24, 1024, 256, -1), ("f16", "f16", 5, 1000, 998, -1),
                                  ("f16", "f32", 256, 512, 256, "mi16"), ("bf16", "bf16", 512, 256, 128, "mi16"), ("f16", "f16", 256, 256, 192, "mi16"),
                                  ("i8", "i32", 256, 256, 512, "mi16"), ("i8", "i16", 256, 256, 256, "mi16"), ("i8", "i8", 256, 512, 256, "mi16"),
                                  ("f16", "f32", 512, 768, 256, "w4"), ("bf16", "bf16", 512, 768, 128, "w4"), ("f16", "f16", 256, 256, 192, "w4"),
                                  ("i8", "i32", 256, 512, 512, "w4"), ("i8", "i16", 256, 256, 256, "w4"), ("i8", "i8", 256, 512, 256, "w4")])
def test_fragment_ops_alpha_beta(case):
    """C = epilogue(prologue(C) + A@B) for the SET / SCALE ops of the reference's tensorized plan
    (Tensor_MatMul_ElementWiseOps_GPU.md:85-99; helpers CppPrinterUtils.h:630-655), on the MFMA,
    edge, fp32, generic and both skinny kernels."""
    import accera_amd as acc
    import torch
    in_type, out_type, M, N, K, variant = case
    if variant == "mi16":  # the full build of the 16x16-shape kernel (the automatic choice keeps it for C = A*B and relu(A*B))
        from accera_amd import _lib
        variant = next(v for v in range(_lib.num_variants()) if "mi16" in _lib.variant_name(v) and "256x256 kb64" in _lib.variant_name(v)
                       and "B=row-major" in _lib.variant_name(v) and "A=col" not in _lib.variant_name(v))
    w4 = variant == "w4"  # the four-wave kernel: the accumulators start from the prologue'd C; an int8 C is only written
    if w4:
        variant = _hand_laid("row")
    for n, (pro, pa, epi, ea) in enumerate(OPS):
        if w4 and out_type == "i8" and pro != ora.PRO_SET:
            continue
        rng = np.random.default_rng(300 + n)
        A, B = make_input(rng, (M, K), in_type), make_input(rng, (K, N), in_type)
        C0 = make_c0(rng, (M, N), out_type)
        dC = to_device(C0, out_type)
        acc.gemm_relu(to_device(A, in_type), to_device(B, in_type), dC, prologue=pro, prologue_arg=pa, epilogue=epi, epilogue_arg=ea,
                      variant=variant)
        torch.cuda.synchronize()
        want = ora.gemm_relu_exact(A, B, C0, in_type, out_type, pro, epi, prologue_arg=pa, epilogue_arg=ea)
        assert_matches(to_host(dC, out_type), want, out_type, K)


def test_linearity_and_k_split_invariance_full_size_int8():
    """Size-independent property at a large size: for int8, A@[B1|B2] computed as one
    N=2048 problem equals the two N=1024 problems, and equals int64 NumPy on sampled rows."""
    import accera_amd as acc
    import torch
    rng = np.random.default_rng(61)
    M, N, K = 2048, 2048, 4096
    A, B = make_input(rng, (M, K), "i8"), make_input(rng, (K, N), "i8")
    dA, dB = to_device(A, "i8"), to_device(B, "i8")
    dC = to_device(out_zeros(M, N, "i32"), "i32")
    acc.gemm_relu(dA, dB, dC, epilogue=acc.EPILOGUE_NONE)
    dC1 = to_device(out_zeros(M, N // 2, "i32"), "i32")
    acc.gemm_relu(dA, dB[:, : N // 2], dC1, epilogue=acc.EPILOGUE_NONE)
    torch.cuda.synchronize()
    C = to_host(dC, "i32")
    assert np.array_equal(C[:, : N // 2], to_host(dC1, "i32"))
    rows = rng.choice(M, 16, replace=False)
    assert np.array_equal(C[rows], (A[rows].astype(np.int64) @ B.astype(np.int64)).astype(np.int32))
    # checksum of checksums: sum_j C[i,j] = A[i,:] . (B 1)
    assert np.array_equal(C.astype(np.int64).sum(axis=1), A.astype(np.int64) @ B.astype(np.int64).sum(axis=1))


# ---- the benchmark configurations at their full sizes --------------------------------------------------
@pytest.mark.parametrize("cfg", [("f16", "f32", 4096, 4096, 4096, "row", "uniform"), ("bf16", "bf16", 4096, 3072, 768, "col", "normal"),
                                 ("i8", "i32", 8192, 8192, 8192, "row", "uniform"), ("f16", "f16", 8, 11008, 4096, "row", "normal")])
def test_benchmark_configurations_at_full_size(cfg):
    """Automatic kernel choice at the sizes the benchmark quotes: sampled rows and columns of the
    result against the exact restatement (float64 matmul of the exactly widened inputs; for int8 every
    partial sum stays below 2^53, so float64 BLAS is exact there too), plus the row-checksum identity
    sum_j (A@B)[i,j] = A[i,:] . (B 1) on the pre-ReLU product for the integer case."""
    import accera_amd as acc
    import torch
    in_type, out_type, M, N, K, b_layout, dist = cfg
    rng = np.random.default_rng(M + N + K)
    A, B = make_input(rng, (M, K), in_type, dist), make_input(rng, (K, N), in_type, dist)
    if b_layout == "col":
        B = np.asfortranarray(B)
    dA, dB = to_device(A, in_type), to_device(B, in_type)
    dC = to_device(out_zeros(M, N, out_type) + (1 if out_type == "i32" else 0), out_type)  # poisoned: SET must overwrite
    acc.gemm_relu(dA, dB, dC)
    torch.cuda.synchronize()
    got = ora.widen(to_host(dC, out_type), out_type)
    Aw, Bw = ora.widen(A, in_type).astype(np.float64), ora.widen(B, in_type).astype(np.float64)
    rows = np.arange(M) if M <= 64 else rng.choice(M, 48, replace=False)
    cols = rng.choice(N, 48, replace=False)
    want_rows = np.maximum(Aw[rows] @ Bw, 0)
    want_cols = np.maximum(Aw @ Bw[:, cols], 0)
    if out_type == "i32":
        assert np.array_equal(got[rows], want_rows) and np.array_equal(got[:, cols], want_cols)
        dC2 = to_device(out_zeros(M, N, out_type), out_type)
        acc.gemm_relu(dA, dB, dC2, epilogue=acc.EPILOGUE_NONE)
        torch.cuda.synchronize()
        assert np.array_equal(to_host(dC2, "i32").astype(np.int64).sum(axis=1), (Aw @ Bw.sum(axis=1)).astype(np.int64))
    else:
        assert_matches(ora.narrow(got[rows], out_type), ora.narrow(want_rows, out_type), out_type, K)
        assert_matches(ora.narrow(got[:, cols], out_type), ora.narrow(want_cols, out_type), out_type, K)
    assert (got[rows] == 0).any() and (got[rows] > 0).any()


@pytest.mark.parametrize("case", [("f16", "f32", 3, 1280, 768, 1024, -1), ("bf16", "bf16", 8, 256, 384, 128, -1), ("i8", "i32", 4, 256, 256, 512, -1),
                                  ("i8", "i16", 3, 256, 256, 512, -1), ("i8", "i8", 5, 128, 384, 256, -1),
                                  ("f32", "f32", 32, 128, 128, 128, -1), ("f16", "f16", 5, 100, 72, 40, -1), ("f16", "f16", 6, 8, 1088, 512, -1),
                                  ("f16", "f16", 3, 8, 1088, 512, 100), ("bf16", "f32", 2, 5, 1000, 998, -1), ("f16", "f32", 1, 64, 64, 64, -1),
                                  ("f16", "f32", 3, 512, 768, 512, "hand-laid"), ("i8", "i32", 2, 256, 512, 1024, "hand-laid"),
                                  # a decode step's attention, P x V per head: few rows, a narrow B, many problems -- the 64 x 64 tiles with direct
                                  # fills on fewer rows than they have (the streaming kernels read such short rows slowly)
                                  ("f16", "f16", 80, 8, 128, 512, -1), ("i8", "i32", 70, 1, 256, 256, -1), ("bf16", "f32", 140, 20, 64, 192, -1)])
def test_batched_gemm(case):
    """C[b] = relu(A[b] @ B[b]) in one launch: the reference's batch matmul nest
    (mfma_tests.py:435-549; shapes 3 x 1280x768x1024, 8 x ..., 32 x 128^3, 1 x 64^3 from :2519-2549) on
    every kernel family; then with one B shared by the batch (batch stride 0) and accumulation into C."""
    import accera_amd as acc
    import torch
    in_type, out_type, batch, M, N, K, variant = case
    if variant == "hand-laid":  # the four-wave kernel, named (it also accumulates into a 32-bit C)
        variant = _hand_laid("row")
    rng = np.random.default_rng(batch * 1000 + M)
    A = np.stack([make_input(rng, (M, K), in_type, "normal") for _ in range(batch)])
    B = np.stack([make_input(rng, (K, N), in_type, "normal") for _ in range(batch)])
    C0 = np.stack([make_c0(rng, (M, N), out_type, scale=1) for _ in range(batch)])
    up = lambda x, t: torch.stack([to_device(m, t) for m in x])
    dA, dB, dC = up(A, in_type), up(B, in_type), up(C0, out_type)
    if batch >= 64:
        from accera_amd.gemm import GemmCall
        from accera_amd import _lib
        name = _lib.variant_name(GemmCall(dA, dB, dC).chosen[0])
        assert "mfma 64x64" in name and "fill=direct" in name, name
    acc.gemm_relu(dA, dB, dC, variant=variant, k_splits=3 if variant >= 100 else 0)
    torch.cuda.synchronize()
    got = [to_host(dC[b], out_type) for b in range(batch)]
    for b in range(batch):
        assert_matches(got[b], ora.gemm_relu_exact(A[b], B[b], None, in_type, out_type), out_type, K)
    # shared B (2-D) and accumulate
    dC = up(C0, out_type)
    acc.gemm_relu(dA, dB[0], dC, prologue=acc.PROLOGUE_NONE, epilogue=acc.EPILOGUE_NONE, variant=variant)
    torch.cuda.synchronize()
    for b in range(batch):
        want = ora.gemm_relu_exact(A[b], B[0], C0[b], in_type, out_type, ora.PRO_NONE, ora.EPI_NONE)
        assert_matches(to_host(dC[b], out_type), want, out_type, K)


def test_sweep_tool_checks_and_times_every_variant():
    """accera_amd.tune on two small rows (one with alpha / beta, one transposed): every variant the
    library accepts must pass the NumPy check (rtol 1e-2 as accera_gemm.py:632)."""
    from accera_amd import tune
    rows = [dict(m=512, n=768, k=256, transA=0, transB=1, alpha=1.0, beta=0.0), dict(m=256, n=256, k=512, transA=1, transB=0, alpha=2.0, beta=0.5),
            dict(m=8, n=1088, k=512, transA=0, transB=0, alpha=1.0, beta=1.0)]
    res = tune.sweep(rows, "f16", relu=False, check=True, min_time_s=0.002, log=lambda *_: None)
    assert len(res) >= 8 and all(r["correct"] is True for r in res), [r for r in res if r["correct"] is not True]
    res = tune.sweep(rows[:1], "i8", relu=True, check=True, min_time_s=0.002, log=lambda *_: None)
    assert res and all(r["correct"] is True for r in res)
    res = tune.sweep(rows[:1], "i8", relu=True, check=True, out_type="i16", min_time_s=0.002, log=lambda *_: None)
    assert res and all(r["correct"] is True for r in res)
    # the vendor-library yardstick adds one row per shape and does not touch the checks
    lines = []
    res = tune.sweep(rows[:2], "f16", relu=False, check=True, min_time_s=0.002, log=lines.append, baseline=True)
    assert sum(r["variant"] == -2 for r in res) == 2 and all("vendor library" in l for l in lines)
    assert all(r["correct"] is True for r in res if r["variant"] != -2)


# ---- error behaviour of the C ABI ---------------------------------------------------------------
def test_errors_are_reported_not_thrown():
    import accera_amd as acc
    import torch
    A = torch.zeros((64, 64), dtype=torch.int8, device="cuda")
    Cf = torch.zeros((64, 64), dtype=torch.float32, device="cuda")
    with pytest.raises(acc.Acc950Error) as e:
        acc.gemm_relu(A, A, Cf)  # int8 -> fp32 is not a supported pair
    assert e.value.code == 1
    Ah = torch.zeros((100, 72), dtype=torch.float16, device="cuda")
    Ch = torch.zeros((100, 100), dtype=torch.float32, device="cuda")
    with pytest.raises(acc.Acc950Error) as e:
        acc.gemm_relu(Ah, Ah.t(), Ch, variant=0)  # 256x256 tile variant cannot take 100x100
    assert e.value.code == 2
    with pytest.raises(acc.Acc950Error):
        acc.gemm_relu(Ah, Ah.t(), Ch, variant=57)
    with pytest.raises(ValueError):
        acc.gemm_relu(Ah.cpu(), Ah.t(), Ch)  # no CPU path


def test_random_problems_through_the_automatic_choice():
    """Seeded random shapes, types, layouts and ops through the automatic kernel choice (MFMA tiles of
    every size, edge and thread-bound kernels, skinny kernels), each checked against the oracle."""
    import accera_amd as acc
    import torch
    rng = np.random.default_rng(2024)
    pairs = [("f16", "f32"), ("f16", "f16"), ("bf16", "f32"), ("bf16", "bf16"), ("i8", "i32"), ("i8", "i16"), ("i8", "i8"), ("f32", "f32")]
    ops = [(ora.PRO_SET0, 0.0, ora.EPI_RELU, 0.0), (ora.PRO_SET0, 0.0, ora.EPI_NONE, 0.0), (ora.PRO_NONE, 0.0, ora.EPI_RELU, 0.0),
           (ora.PRO_SCALE, 0.5, ora.EPI_SCALE, 2.0), (ora.PRO_SET, 3.0, ora.EPI_RELU_NOCOND, 0.0), (ora.PRO_NONE, 0.0, ora.EPI_SET, 1.0)]
    sizes_m = [1, 5, 8, 16, 31, 64, 100, 128, 200, 256, 384, 512, 768, 1024]
    sizes_n = [8, 16, 40, 64, 72, 128, 192, 256, 384, 512, 768, 1000, 1024, 1088, 2048]
    sizes_k = [16, 32, 64, 96, 128, 176, 256, 336, 512, 998, 1024, 2048]
    for case in range(60):
        in_type, out_type = pairs[rng.integers(len(pairs))]
        M, N, K = (int(s[rng.integers(len(s))]) for s in (sizes_m, sizes_n, sizes_k))
        pro, pa, epi, ea = ops[rng.integers(len(ops))]
        a_col, b_col = bool(rng.integers(2)) and in_type != "f32", bool(rng.integers(2))
        print("case", case, in_type, out_type, M, N, K, "A col" if a_col else "A row", "B col" if b_col else "B row", pro, pa, epi, ea, flush=True)
        A, B = make_input(rng, (M, K), in_type), make_input(rng, (K, N), in_type)
        if a_col:
            A = np.asfortranarray(A)
        if b_col:
            B = np.asfortranarray(B)
        C0 = make_c0(rng, (M, N), out_type, scale=100)
        dC = to_device(C0, out_type)
        acc.gemm_relu(to_device(A, in_type), to_device(B, in_type), dC, prologue=pro, prologue_arg=pa, epilogue=epi, epilogue_arg=ea)
        torch.cuda.synchronize()
        want = ora.gemm_relu_exact(A, B, C0, in_type, out_type, pro, epi, prologue_arg=pa, epilogue_arg=ea)
        assert_matches(to_host(dC, out_type), want, out_type, K)


def test_random_problems_on_the_four_wave_kernel():
    """Seeded random sizes (M and N ragged or whole tiles, every K remainder modulo four k-steps), types, B layouts
    and ops on the kernels with the hand-laid loop, named explicitly; what a kernel refuses is skipped, never wrong."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    rng = np.random.default_rng(950)
    pairs = [("f16", "f32"), ("f16", "f16"), ("bf16", "f32"), ("bf16", "bf16"), ("i8", "i32"), ("i8", "i16"), ("i8", "i8")]
    ops = [(ora.PRO_SET0, 0.0, ora.EPI_RELU, 0.0), (ora.PRO_SET0, 0.0, ora.EPI_NONE, 0.0), (ora.PRO_NONE, 0.0, ora.EPI_RELU, 0.0),
           (ora.PRO_SCALE, 0.5, ora.EPI_SCALE, 2.0), (ora.PRO_SET, 3.0, ora.EPI_RELU_NOCOND, 0.0), (ora.PRO_NONE, 0.0, ora.EPI_SET, 1.0),
           (ora.PRO_SCALE, -1.5, ora.EPI_RELU, 0.0)]
    ran = 0
    for case in range(48):
        in_type, out_type = pairs[rng.integers(len(pairs))]
        b_layout = ("row", "col")[rng.integers(2)]
        variants = [v for v, n in _variants(b_layout) if "hand-laid" in n and "A=col-major" not in n]
        v = variants[rng.integers(len(variants))]
        kb = 64 if in_type == "i8" else 32
        pro, pa, epi, ea = ops[rng.integers(len(ops))]
        whole = rng.integers(2) == 0
        tile_n = 192 if "256x192" in _lib.variant_name(v) else 256
        M = int(rng.integers(1, 5)) * 256 if whole else int(rng.integers(256, 1100))
        N = int(rng.integers(1, 5)) * tile_n if whole else int(rng.integers(tile_n // 16, 70)) * 16
        K = int(rng.integers(4, 14)) * kb
        print("case", case, "variant", v, in_type, out_type, M, N, K, b_layout, pro, pa, epi, ea, flush=True)
        A, B = make_input(rng, (M, K), in_type), make_input(rng, (K, N), in_type)
        if b_layout == "col":
            B = np.asfortranarray(B)
        C0 = make_c0(rng, (M, N), out_type, scale=100)
        dC = to_device(C0, out_type)
        try:
            acc.gemm_relu(to_device(A, in_type), to_device(B, in_type), dC, prologue=pro, prologue_arg=pa, epilogue=epi, epilogue_arg=ea,
                          variant=v)
        except _lib.Acc950Error as err:
            # the only refusal these kernels may make here: an int8 C that would be read
            assert err.code == _lib.UNSUPPORTED and out_type == "i8" and pro != ora.PRO_SET, (case, str(err))
            continue
        torch.cuda.synchronize()
        want = ora.gemm_relu_exact(A, B, C0, in_type, out_type, pro, epi, prologue_arg=pa, epilogue_arg=ea)
        assert_matches(to_host(dC, out_type), want, out_type, K)
        ran += 1
    assert ran >= 30, ran


@pytest.mark.parametrize("in_type,out_type,b_layout,M,N,K,pro,epi", [
    # 17 x 16 = 272 tiles of 256 x 256 over 256 workgroups: sixteen of them walk two tiles; K a multiple of four k-steps, so
    # the closing steps of a tile fetch for the next one and (32-bit C) its first k-steps run with the stores in flight
    ("i8", "i32", "row", 4352, 4096, 512, "set0", "relu"),
    ("f16", "f32", "row", 4352, 4096, 256, "set0", "relu"),
    ("bf16", "f32", "col", 4352, 4096, 384, "set0", "none"),
    # narrow outputs: the slabs of the write-back live in the stage the next tile's fills leave alone
    ("f16", "f16", "row", 4352, 4096, 256, "set0", "relu"),
    ("i8", "i8", "row", 4352, 4096, 512, "set0", "relu"),
    # a number of k-steps that is not a multiple of four: the next tile is fetched after the write-back
    ("i8", "i32", "row", 4352, 4096, 448, "set0", "relu"),
    ("bf16", "bf16", "row", 4352, 4096, 288, "set0", "relu"),
    # ragged M and N, 18 x 17 = 306 tiles (not a multiple of the eight XCDs either)
    ("f16", "f32", "row", 4400, 4112, 256, "set0", "relu"),
    ("i8", "i32", "col", 4400, 4112, 512, "set0", "relu"),
    # C is read: C += A*B straight into the accumulators (32-bit C), and widened / scaled by ordinary code
    ("i8", "i32", "row", 4352, 4096, 512, "none", "relu"),
    ("f16", "f16", "row", 4352, 4096, 256, "scale", "scale"),
    # ragged sizes and C read: moved tiles do not store what their neighbours own
    ("f16", "f32", "row", 4400, 4112, 256, "none", "relu"),
    ("bf16", "bf16", "col", 4400, 4112, 384, "scale", "none"),
    # three rounds over the workgroups
    ("i8", "i32", "row", 8192, 6144, 256, "set0", "relu"),
])
def test_four_wave_kernel_walking_several_tiles(in_type, out_type, b_layout, M, N, K, pro, epi):
    """More tiles than compute units on the multi-tile form of the hand-laid kernel, named explicitly, and the automatic
    choice takes it when the tiles make whole rounds over the compute units."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    v = [v for v, n in _variants(b_layout) if "multi-tile" in n and "A=col-major" not in n]
    assert len(v) == 1
    pro_op, pa = {"set0": (ora.PRO_SET0, 0.0), "none": (ora.PRO_NONE, 0.0), "scale": (ora.PRO_SCALE, 0.5)}[pro]
    epi_op, ea = {"relu": (ora.EPI_RELU, 0.0), "none": (ora.EPI_NONE, 0.0), "scale": (ora.EPI_SCALE, 2.0)}[epi]
    rng = np.random.default_rng(M + N + K)
    A, B = make_input(rng, (M, K), in_type), make_input(rng, (K, N), in_type)
    if b_layout == "col":
        B = np.asfortranarray(B)
    C0 = make_c0(rng, (M, N), out_type, scale=100)
    dA, dB = to_device(A, in_type), to_device(B, in_type)
    want = ora.gemm_relu_exact(A, B, C0, in_type, out_type, pro_op, epi_op, prologue_arg=pa, epilogue_arg=ea)
    for variant in (v[0], -1):
        dC = to_device(C0, out_type)
        call = acc.GemmCall(dA, dB, dC, prologue=pro_op, prologue_arg=pa, epilogue=epi_op, epilogue_arg=ea, variant=variant)
        call()
        torch.cuda.synchronize()
        assert_matches(to_host(dC, out_type), want, out_type, K)
    grid, block, lds, chosen = _lib.launch_geometry(getattr(_lib, in_type.upper()), getattr(_lib, out_type.upper()), M, N, K, (K, 1),
                                                    (N, 1) if b_layout == "row" else (1, K), (N, 1))
    if (M // 256) * (N // 256) % 256 == 0 and M % 256 == 0 and N % 256 == 0:
        # whole rounds of tiles over the compute units (with a nearly empty last round the cost model prefers smaller tiles)
        assert "multi-tile" in _lib.variant_name(chosen) and grid == [256, 1, 1]


@pytest.mark.parametrize("in_type,out_type,b_layout,M,N,K,pro,epi", [
    # two rounds over the workgroups, K of 8 and 12 k-steps (closing steps fetch the next tile)
    ("f16", "f32", "row", 4096, 8192, 256, "set0", "relu"),
    ("bf16", "bf16", "col", 4096, 8192, 384, "set0", "relu"),
    ("i8", "i32", "row", 8192, 4096, 512, "set0", "relu"),
    ("i8", "i8", "col", 4096, 8192, 768, "set0", "none"),
    # a K that enters the loop in the middle (9 k-steps: no fetching ahead), ragged M and N, C read
    ("f16", "f16", "row", 4112, 4400, 288, "set0", "relu"),
    ("i8", "i32", "col", 4352, 4096, 512, "none", "relu"),
    ("f16", "f32", "col", 4400, 4112, 256, "none", "relu"),
])
def test_four_wave_kernel_walking_several_tiles_with_a_column_major_a(in_type, out_type, b_layout, M, N, K, pro, epi):
    """The multi-tile form for a column-major A (the transA rows of the reference's sweep lists,
    /root/reference/tools/benchmarkers/accera_gemm.py:310-311), named explicitly and through the automatic choice."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    v = [v for v, n in _variants(b_layout) if "multi-tile" in n and "A=col-major" in n]
    assert len(v) == 1
    pro_op, pa = {"set0": (ora.PRO_SET0, 0.0), "none": (ora.PRO_NONE, 0.0)}[pro]
    epi_op, ea = {"relu": (ora.EPI_RELU, 0.0), "none": (ora.EPI_NONE, 0.0)}[epi]
    rng = np.random.default_rng(M + N + K + 1)
    A, B = np.asfortranarray(make_input(rng, (M, K), in_type)), make_input(rng, (K, N), in_type)
    if b_layout == "col":
        B = np.asfortranarray(B)
    C0 = make_c0(rng, (M, N), out_type, scale=100)
    dA, dB = to_device(A, in_type), to_device(B, in_type)
    assert dA.stride() == (1, M)
    want = ora.gemm_relu_exact(A, B, C0, in_type, out_type, pro_op, epi_op, prologue_arg=pa, epilogue_arg=ea)
    for variant in (v[0], -1):
        dC = to_device(C0, out_type)
        call = acc.GemmCall(dA, dB, dC, prologue=pro_op, prologue_arg=pa, epilogue=epi_op, epilogue_arg=ea, variant=variant)
        call()
        torch.cuda.synchronize()
        assert_matches(to_host(dC, out_type), want, out_type, K)
    name = _lib.variant_name(acc.GemmCall(dA, dB, to_device(C0, out_type), prologue=pro_op, epilogue=epi_op, variant=-1).chosen[0])
    assert "A=col-major" in name, name


def test_skinny_workspaces_are_per_stream():
    """Launches on different streams may overlap, so each stream has its own K-split partial sums and arrival
    counters; the decode shape (whose slow-phase column blocks are shared by two workgroups each) runs on two streams
    at once and both results match the oracle."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    w1, w2, w1b = _lib.workspace_probe(s1.cuda_stream), _lib.workspace_probe(s2.cuda_stream), _lib.workspace_probe(s1.cuda_stream)
    assert w1 == w1b and w1[0] != w2[0] and w1[1] != w2[1] and all(w1) and all(w2)
    rng = np.random.default_rng(77)
    M, N, K = 8, 11008, 4096
    A = make_input(rng, (M, K), "f16", "normal")
    Bs = [(make_input(rng, (K, N), "f16", "normal").astype(np.float32) * 0.05).astype(np.float16) for _ in range(2)]
    dA = to_device(A, "f16")
    dBs = [to_device(B, "f16") for B in Bs]
    dCs = [to_device(out_zeros(M, N, "f16"), "f16") for _ in range(2)]
    torch.cuda.synchronize()
    calls = [acc.GemmCall(dA, dBs[i], dCs[i], stream=s.cuda_stream) for i, s in enumerate((s1, s2))]
    for _ in range(20):
        for c in calls:
            c()
    torch.cuda.synchronize()
    for i in range(2):
        want = ora.gemm_relu_exact(A, Bs[i], out_zeros(M, N, "f16"), "f16", "f16", ora.PRO_SET0, ora.EPI_RELU)
        assert_matches(to_host(dCs[i], "f16"), want, "f16", K)
    # the workspaces can be handed back (a host that creates and destroys streams): the next launches make new ones
    before = _lib.allocation_probe()
    _lib.release_workspaces()
    for d in dCs:
        d.fill_(5)
    for c in calls:
        c()
    torch.cuda.synchronize()
    assert _lib.allocation_probe() >= before + 2
    for i in range(2):
        want = ora.gemm_relu_exact(A, Bs[i], out_zeros(M, N, "f16"), "f16", "f16", ora.PRO_SET0, ora.EPI_RELU)
        assert_matches(to_host(dCs[i], "f16"), want, "f16", K)


@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("f16", "f16"), ("bf16", "bf16"), ("i8", "i32"), ("i8", "i16")])
@pytest.mark.parametrize("a_layout,b_layout", [("row", "row"), ("row", "col"), ("col", "row"), ("col", "col")])
def test_any_alignment_mfma_kernel(in_type, out_type, a_layout, b_layout):
    """Sizes, leading dimensions and pointers that are not multiples of the 16-byte vector (the odd shapes of the
    reference's sweep lists, tools/benchmarkers/gemm_resnet_inception.csv: K = 1225, 3025, 5329, M = 27, 147, 363 ...):
    the edge kernel whose fill takes unaligned chunks, named explicitly; C overwritten and read; then operands that are
    views into larger arrays starting at an odd element."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    key = " B=col-major" if b_layout == "col" else " B=row-major"
    variants = [v for v in range(_lib.num_variants()) if "any-alignment" in _lib.variant_name(v) and key in _lib.variant_name(v)
                and ("A=col-major" in _lib.variant_name(v)) == (a_layout == "col")]
    # 128 x 128 and 64 x 64 tiles, and 256 x 256 ones for a row-major A
    assert len(variants) == (2 if a_layout == "col" else 3), [_lib.variant_name(v) for v in variants]
    for v in variants:
        _any_alignment_cases(v, in_type, out_type, a_layout, b_layout)


def _any_alignment_cases(v, in_type, out_type, a_layout, b_layout):
    import accera_amd as acc
    import torch
    for n, (M, N, K) in enumerate([(363, 64, 3025), (192, 48, 1225), (27, 32, 2201), (196, 600, 64), (100, 72, 41), (129, 257, 131), (1, 1, 1), (5, 300, 7)]):
        print("variant", v, in_type, out_type, a_layout, b_layout, M, N, K, flush=True)
        run_case(in_type, out_type, M, N, K, a_layout=a_layout, b_layout=b_layout, variant=v, seed=1200 + n)
        run_case(in_type, out_type, M, N, K, a_layout=a_layout, b_layout=b_layout, variant=v, seed=1300 + n, prologue=ora.PRO_NONE,
                 epilogue=ora.EPI_NONE)
    # views that start at an odd element of larger arrays (pointers aligned to the element only, odd leading dimensions)
    rng = np.random.default_rng(1400)
    M, N, K = 150, 203, 333
    Abig = make_input(rng, (K + 3, M + 5) if a_layout == "col" else (M + 3, K + 5), in_type)
    Bbig = make_input(rng, (N + 3, K + 7) if b_layout == "col" else (K + 3, N + 7), in_type)
    Cbig = make_c0(rng, (M + 2, N + 3), out_type)
    dA, dB, dC = to_device(Abig, in_type), to_device(Bbig, in_type), to_device(Cbig, out_type)
    Av = Abig[1:K + 1, 3:M + 3].T if a_layout == "col" else Abig[1:M + 1, 3:K + 3]
    Bv = Bbig[1:N + 1, 5:K + 5].T if b_layout == "col" else Bbig[1:K + 1, 5:N + 5]
    dAv = dA[1:K + 1, 3:M + 3].t() if a_layout == "col" else dA[1:M + 1, 3:K + 3]
    dBv = dB[1:N + 1, 5:K + 5].t() if b_layout == "col" else dB[1:K + 1, 5:N + 5]
    for prologue in (ora.PRO_SET0, ora.PRO_NONE):
        dC.copy_(to_device(Cbig, out_type))
        print("variant", v, in_type, out_type, a_layout, b_layout, "views, prologue", prologue, flush=True)
        acc.gemm_relu(dAv, dBv, dC[1:M + 1, 1:N + 1], prologue=prologue, variant=v)
        torch.cuda.synchronize()
        got = to_host(dC, out_type)
        want = ora.gemm_relu_exact(np.ascontiguousarray(Av), np.ascontiguousarray(Bv), np.ascontiguousarray(Cbig[1:M + 1, 1:N + 1]),
                                   in_type, out_type, prologue, ora.EPI_RELU)
        assert_matches(got[1:M + 1, 1:N + 1], want, out_type, K)
        rest = np.ones(Cbig.shape, bool)
        rest[1:M + 1, 1:N + 1] = False
        assert np.array_equal(got[rest], Cbig[rest]), "elements around the view were written"


def test_odd_sizes_take_an_mfma_kernel_automatically():
    """K, N or leading dimensions that are not multiples of the 16-byte vector no longer fall to the thread-bound kernel."""
    from accera_amd import _lib
    for in_t, out_t, M, N, K in ((_lib.I8, _lib.I32, 1000, 1000, 1000), (_lib.F16, _lib.F32, 363, 64, 3025), (_lib.BF16, _lib.BF16, 289, 384, 2593)):
        g, b, lds, v = _lib.launch_geometry(in_t, out_t, M, N, K, (K, 1), (N, 1), (N, 1))
        assert "any-alignment" in _lib.variant_name(v), _lib.variant_name(v)
    run_case("i8", "i32", 1000, 1000, 1000, seed=77, expect_variant=None)
    run_case("f16", "f16", 289, 384, 2593, seed=78, a_layout="col")


def _named(*keys, b_layout="row"):
    """The first variant whose description holds every key."""
    return next(v for v, n in _variants(b_layout) if all(k in n for k in keys))


@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("f16", "f16"), ("bf16", "bf16"), ("i8", "i32"), ("i8", "i8")])
def test_k_split_of_the_mfma_kernels(in_type, out_type):
    """K split over workgroups: the kernel runs as a batch of partial products into a workspace, a second kernel adds the
    slices in slice order and applies the ops (the ReLU after the whole sum).  Per kernel family and split count, slices
    of equal and unequal length, C overwritten and read, every op; integer results bit-exact; two runs give the same bits."""
    import accera_amd as acc
    import torch
    from accera_amd import _lib
    kb = 64 if in_type == "i8" else 32
    families = [("hand-laid", "row", "row", ("mfma 256x256", "hand-laid loop")), ("hand-laid, B col-major", "row", "col", ("mfma 256x256", "hand-laid loop")),
                ("hand-laid, A col-major", "col", "row", ("A=col-major", "hand-laid loop")),
                ("ping-pong 16x16", "row", "row", ("mfma 256x256 kb64", "pingpong mi16")), ("128x128 direct", "row", "row", ("mfma 128x128 kb64", "fill=direct")),
                ("any alignment", "row", "row", ("mfma 128x128", "any-alignment")),
                ("64x64 direct", "row", "row", ("mfma 64x64", "fill=direct")), ("64x64 direct, A and B col-major", "col", "col", ("mfma 64x64", "fill=direct")),
                ("128x64 direct", "row", "col", ("mfma 128x64", "fill=direct")), ("64x64 any alignment", "col", "row", ("mfma 64x64", "any-alignment"))]
    for label, a_layout, b_layout, keys in families:
        v = next(v for v, n in _variants(b_layout) if all(k in n for k in keys) and ("A=col-major" in n) == (a_layout == "col")
                 and "multi-tile" not in n)
        kb = int(re.search(r"kb(\d+)", _lib.variant_name(v)).group(1)) // (1 if in_type == "i8" else 2) if "64 " in label or "128x64" in label else kb
        for splits, k_tiles in ((2, 8), (3, 40), (5, 21), (8, 40)):
            print(label, "variant", v, in_type, out_type, "splits", splits, "k tiles", k_tiles, flush=True)
            g = _lib.launch_geometry(ora.TYPE_IDS[in_type], ora.TYPE_IDS[out_type], 256, 512, k_tiles * kb,
                                     (1, 256) if a_layout == "col" else (k_tiles * kb, 1), (1, k_tiles * kb) if b_layout == "col" else (512, 1), (512, 1), v, splits)[0]
            assert 1 < g[2] <= splits, g
            run_case(in_type, out_type, 256, 512, k_tiles * kb, a_layout=a_layout, b_layout=b_layout, variant=v, splits=splits, seed=1500 + splits)
            if out_type != "i8" or "hand-laid" not in label:
                run_case(in_type, out_type, 256, 512, k_tiles * kb, a_layout=a_layout, b_layout=b_layout, variant=v, splits=splits, seed=1510 + splits,
                         prologue=ora.PRO_NONE, epilogue=ora.EPI_RELU_NOCOND)
    # odd sizes on the any-alignment kernel; SCALE / SET ops with their operands; the same bits on a second run
    v = _named("any-alignment")
    rng = np.random.default_rng(1520)
    M, N, K = 147, 64 if out_type == "i8" else 65, 3025   # (rows of an int8 C must be 16 bytes apart for the MFMA kernels)
    A, B = make_input(rng, (M, K), in_type), make_input(rng, (K, N), in_type)
    C0 = make_c0(rng, (M, N), out_type, scale=100)
    for pro, pa, epi, ea in ((ora.PRO_SCALE, 0.5, ora.EPI_SCALE, 2.0), (ora.PRO_SET, 3.0, ora.EPI_RELU, 0.0), (ora.PRO_NONE, 0.0, ora.EPI_SET, 1.0)):
        outs = []
        for _ in range(2):
            dC = to_device(C0, out_type)
            acc.gemm_relu(to_device(A, in_type), to_device(B, in_type), dC, prologue=pro, prologue_arg=pa, epilogue=epi, epilogue_arg=ea,
                          variant=v, k_splits=4)
            torch.cuda.synchronize()
            outs.append(to_host(dC, out_type))
        assert np.array_equal(outs[0].view(np.uint8), outs[1].view(np.uint8)), "a K split must add its slices in a fixed order"
        want = ora.gemm_relu_exact(A, B, C0, in_type, out_type, pro, epi, prologue_arg=pa, epilogue_arg=ea)
        assert_matches(outs[0], want, out_type, K)


def test_k_split_is_chosen_for_small_outputs_with_a_long_k_and_refused_where_it_cannot_run():
    """Shapes of the reference's sweep lists that leave most compute units idle (gemm_bert_assorted.csv: 768 x 320 x 30522;
    gemm_resnet_inception.csv: 288 x 64 x 21609) are split by the library itself; the benchmark configurations are not."""
    import accera_amd as acc
    from accera_amd import _lib
    g, b, lds, v = _lib.launch_geometry(_lib.F16, _lib.F32, 768, 320, 30522, (30522, 1), (320, 1), (320, 1))
    assert "mfma" in _lib.variant_name(v) and g[2] > 1, (g, _lib.variant_name(v))
    run_case("f16", "f32", 768, 320, 30522, seed=1530, dist="normal")
    run_case("i8", "i32", 288, 64, 21609, seed=1531)
    run_case("bf16", "bf16", 512, 256, 8192, seed=1532, prologue=ora.PRO_NONE)
    for M, N, K, sa, sb, sc, t_in, t_out in ((4096, 4096, 4096, (4096, 1), (4096, 1), (4096, 1), _lib.F16, _lib.F32),
                                             (4096, 3072, 768, (768, 1), (1, 768), (3072, 1), _lib.BF16, _lib.BF16),
                                             (8192, 8192, 8192, (8192, 1), (8192, 1), (8192, 1), _lib.I8, _lib.I32)):
        assert _lib.launch_geometry(t_in, t_out, M, N, K, sa, sb, sc)[0][2] == 1
    with pytest.raises(_lib.Acc950Error):  # three K tiles cannot be split for a kernel whose slices need four each
        _lib.launch_geometry(_lib.F16, _lib.F32, 256, 256, 224, (224, 1), (256, 1), (256, 1), _hand_laid("row"), 2)


@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("bf16", "bf16"), ("i8", "i32")])
def test_full_tile_kernels_on_sizes_that_are_not_tile_multiples(in_type, out_type):
    """The direct-fill kernels on the 32x32 instruction shapes take any M, N of at least one tile when C is only written:
    the last row / column of tiles is moved to end at M / N.  Every such variant, both layouts of B, column-major A;
    reading C with such sizes is refused (the edge kernels take it), and so is less than one tile of rows of a column-major A."""
    from accera_amd import _lib
    vec = 16 if in_type == "i8" else 8
    seen = 0
    for b_layout in ("row", "col"):
        for v, name in _variants(b_layout):
            if "fill=direct" not in name or "mi16" in name:
                continue
            bm, bn = map(int, re.search(r"mfma (\d+)x(\d+)", name).groups())
            kb = int(re.search(r"kb(\d+)", name).group(1)) // (1 if in_type == "i8" else 2)
            a_layout = "col" if "A=col-major" in name else "row"
            M, N = 2 * bm + 5 * vec, bn + 3 * 16
            print("variant", v, name, in_type, M, N, flush=True)
            run_case(in_type, out_type, M, N, 5 * kb, a_layout=a_layout, b_layout=b_layout, variant=v, seed=1600 + v)
            run_case(in_type, out_type, bm, N, 3 * kb, a_layout=a_layout, b_layout=b_layout, variant=v, seed=1700 + v, epilogue=ora.EPI_NONE)
            with pytest.raises(_lib.Acc950Error):
                run_case(in_type, out_type, M, N, 5 * kb, a_layout=a_layout, b_layout=b_layout, variant=v, seed=1, prologue=ora.PRO_NONE)
            if a_layout == "row":   # less than one tile: taken when A is row-major
                run_case(in_type, out_type, bm - vec, N, 5 * kb, a_layout=a_layout, b_layout=b_layout, variant=v, seed=1)
            else:
                with pytest.raises(_lib.Acc950Error):
                    run_case(in_type, out_type, bm - vec, N, 5 * kb, a_layout=a_layout, b_layout=b_layout, variant=v, seed=1)
            seen += 1
    assert seen >= 20


@pytest.mark.parametrize("in_type,out_type", [("f16", "f16"), ("f16", "f32"), ("bf16", "bf16"), ("i8", "i32"), ("i8", "i16"), ("f32", "f32")])
def test_direct_fill_kernels_take_any_n_with_a_k_contiguous_b(in_type, out_type):
    """A column-major (K-contiguous) B has no row that a moved last tile's first column could split: the direct-fill kernels
    on the 32x32 instruction shapes take any N of at least one tile with it when C is only written -- odd vocabulary sizes
    of language-model heads.  C's rows are then not 16 bytes apart and are stored element by element; every such variant."""
    from accera_amd import _lib
    seen = 0
    for v, name in _variants("col"):
        if "fill=direct" not in name or "mi16" in name or "edge" in name:
            continue
        bm, bn = map(int, re.search(r"mfma (\d+)x(\d+)", name).groups())
        kb = int(re.search(r"kb(\d+)", name).group(1)) // {"f16": 2, "bf16": 2, "i8": 1, "f32": 4}[in_type]
        a_layout = "col" if "A=col-major" in name else "row"
        for N in (2 * bn + 37, bn + 1):
            print("variant", v, name, in_type, out_type, N, flush=True)
            run_case(in_type, out_type, 2 * bm, N, 3 * kb, a_layout=a_layout, b_layout="col", variant=v, seed=N + v, dist="normal")
        seen += 1
    assert seen >= 8
    if out_type == "f16":   # the library by itself: a prefill step's language-model head with GPT-2's vocabulary, scaled down in M and K
        from accera_amd import tune
        name = _lib.variant_name(tune.own_choice(_lib.F16, _lib.F16, 4096, 50257, 4096, False, True, 1.0, 0.0)[0])
        assert "fill=direct" in name and "edge" not in name, name
        run_case("f16", "f16", 300, 50257, 256, b_layout="col", seed=3, dist="normal")
    if out_type == "i16":   # an int8 C keeps its rule: rows 16 bytes apart, or the thread-bound kernel
        with pytest.raises(_lib.Acc950Error):
            run_case("i8", "i8", 256, 293, 256, b_layout="col", variant=next(v for v, n in _variants("col") if "mfma 128x128" in n and "fill=direct" in n and "mi16" not in n), seed=1)


@pytest.mark.parametrize("b_layout", ["row", "col"])
def test_fp32_on_the_tiled_mfma_kernels(b_layout):
    """fp32 inputs on the LDS-tiled kernels (v_mfma_f32_32x32x2_f32; four instructions per 32-byte k-step): every variant
    that has a launcher for fp32 -- the 32x32-shape ones; the 16x16-shape places of the table refuse -- at K tile counts
    below, at and above the pipeline depth, column-major A, edges, odd sizes, C read, and a K split."""
    from accera_amd import _lib
    seen = 0
    for v, name in _variants(b_layout):
        kb = int(re.search(r"kb(\d+)", name).group(1)) // 4
        a_layout = "col" if "A=col-major" in name else "row"
        bm, bn = map(int, re.search(r"mfma (\d+)x(\d+)", name).groups())
        M, N = max(512, 2 * bm), (max(512, 2 * bn) if 512 % bn == 0 else 3 * bn)
        if "mi16" in name:
            with pytest.raises(_lib.Acc950Error):
                run_case("f32", "f32", M, N, 4 * kb, a_layout=a_layout, b_layout=b_layout, variant=v, seed=v)
            continue
        print("variant", v, name, flush=True)
        for k_tiles in (1, 2, 3, 7):
            run_case("f32", "f32", M, N, k_tiles * kb, a_layout=a_layout, b_layout=b_layout, variant=v, seed=1800 + v + k_tiles)
        run_case("f32", "f32", M, N, 5 * kb, a_layout=a_layout, b_layout=b_layout, variant=v, seed=1900 + v, prologue=ora.PRO_NONE,
                 epilogue=ora.EPI_RELU_NOCOND)
        if "edge" in name:
            odd = "any-alignment" in name
            run_case("f32", "f32", 204 if a_layout == "col" and not odd else 203 if odd else 200, 145 if odd else 144, 171 if odd else 172,
                     a_layout=a_layout, b_layout=b_layout, variant=v, seed=2000 + v)
        if "fill=direct" in name and "pingpong" not in name:
            run_case("f32", "f32", M, N, 12 * kb, a_layout=a_layout, b_layout=b_layout, variant=v, splits=3, seed=2100 + v)
        seen += 1
    assert seen >= 12


def test_fp32_automatic_choice():
    """Small fp32 problems stay with the kernel of 32 x 32 blocks; large ones take the tiled kernels -- 64 x 64 tiles while
    larger ones would leave compute units idle -- split over K where the tiles alone would not fill the chip."""
    from accera_amd import _lib
    g, b, lds, v = _lib.launch_geometry(_lib.F32, _lib.F32, 512, 512, 512, (512, 1), (512, 1), (512, 1))
    assert v == _lib.VARIANT_F32_MFMA
    g, b, lds, v = _lib.launch_geometry(_lib.F32, _lib.F32, 1024, 1024, 1024, (1024, 1), (1024, 1), (1024, 1))
    assert "mfma 64x64" in _lib.variant_name(v) and g[2] == 1, (g, _lib.variant_name(v))   # one small tile per compute unit
    g, b, lds, v = _lib.launch_geometry(_lib.F32, _lib.F32, 256, 256, 4096, (4096, 1), (256, 1), (256, 1))
    assert "mfma 64x64" in _lib.variant_name(v) and g[2] > 1, (g, _lib.variant_name(v))    # 16 tiles: split over K
    g, b, lds, v = _lib.launch_geometry(_lib.F32, _lib.F32, 4096, 4096, 4096, (4096, 1), (4096, 1), (4096, 1))
    assert "mfma" in _lib.variant_name(v) and "thread-bound" not in _lib.variant_name(v) and g[2] == 1
    run_case("f32", "f32", 1024, 1024, 1024, seed=2200)
    run_case("f32", "f32", 2048, 1536, 1000, seed=2201, b_layout="col", prologue=ora.PRO_NONE)
    run_case("f32", "f32", 363, 64, 3025, seed=2202, a_layout="col")


@pytest.mark.gpu
@pytest.mark.parametrize("in_type,out_type", [("f16", "f32"), ("bf16", "bf16"), ("i8", "i32")])
def test_measurement_aids_of_the_benchmark(in_type, out_type):
    """The in-kernel phase times and the MFMA ceilings that bench.py reports beside every figure: the calls succeed on a
    small problem and what they return is plausible (positive times that add up to less than the kernel's span, a clock
    between 0.5 and 3 GHz, a pipe occupancy between 0 and 1, a rate below the nominal peak)."""
    import torch
    from accera_amd import _lib
    _lib.check(_lib.lib().acc950_init(0))
    tin = {"f16": torch.float16, "bf16": torch.bfloat16, "i8": torch.int8}[in_type]
    tout = {"f32": torch.float32, "bf16": torch.bfloat16, "i32": torch.int32}[out_type]
    M, N, K = 512, 768, 1024
    if in_type == "i8":
        A = torch.randint(-128, 128, (M, K), device="cuda", dtype=tin)
        B = torch.randint(-128, 128, (K, N), device="cuda", dtype=tin)
    else:
        A = torch.randn((M, K), device="cuda").to(tin)
        B = torch.randn((K, N), device="cuda").to(tin)
    C = torch.zeros((M, N), device="cuda", dtype=tout)
    lid = {"f16": _lib.F16, "bf16": _lib.BF16, "i8": _lib.I8, "f32": _lib.F32, "i32": _lib.I32}
    r = _lib.mfma_phase_probe(lid[in_type], lid[out_type], M, N, K, A.data_ptr(), B.data_ptr(), C.data_ptr())
    torch.cuda.synchronize()
    assert r["prologue_us"] > 0 and r["main_loop_us"] > 0 and r["write_back_us"] > 0
    assert r["prologue_us"] + r["main_loop_us"] + r["write_back_us"] <= r["kernel_span_us"] * 1.001
    assert 0.5 < r["clock_ghz_main_loop"] < 3.0 and 0.0 < r["mfma_pipe_busy_main_loop"] <= 1.0
    peak = 5000.0 if in_type == "i8" else 2500.0
    rate, clock = _lib.mfma_ceiling(lid[in_type], 2, 2000)
    assert 0.2 * peak < rate < peak * 1.02 and 0.5 < clock < 3.0
    for traffic in range(4):
        rate, clock = _lib.mfma_traffic_probe(lid[in_type], traffic, 300)
        assert 0.1 * peak < rate < peak * 1.02 and 0.5 < clock < 3.0


@pytest.mark.parametrize("in_type,out_type,M,N,K,a_col,b_col,kernel", [
    ("f16", "f16", 1049600, 2048, 2048, False, False, "hand-laid loop"),   # A and C beyond 4 GiB on the four-wave kernel (multi-tile form)
    ("i8", "i32", 33024, 33024, 256, False, False, "hand-laid loop"),      # C beyond 4 GiB
    ("f16", "f32", 1100003, 72, 2049, False, False, "any-alignment"),      # A beyond 4 GiB, register-staged fills
    ("bf16", "bf16", 2200000, 64, 1024, True, False, "A=col-major"),       # a column-major A beyond 4 GiB
    ("f32", "f32", 600000, 128, 2048, False, False, "mfma"),               # fp32
    ("f16", "f16", 8, 32776, 65536, False, False, "skinny mfma"),          # few rows, B beyond 4 GiB on the streaming kernel
    ("f16", "f32", 512, 1100000, 2048, False, True, "B=col-major"),        # a column-major B beyond 4 GiB
])
def test_operands_beyond_four_gib(in_type, out_type, M, N, K, a_col, b_col, kernel):
    """Maximum sizes: an A, B or C larger than 4 GiB on every kernel family (64-bit tile bases, 32-bit offsets only inside a
    tile or a step).  B has one +-1 per column, which makes the expected C a gather of A's columns: compared exactly, on the
    GPU, in slabs of rows.  Inputs are small integers, so every type holds the results exactly."""
    import torch
    from accera_amd import _lib
    from accera_amd.gemm import GemmCall
    tt = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "i8": torch.int8, "i32": torch.int32}
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(M % 1000 + N + K)
    lo, hi = (-128, 128) if in_type == "i8" else (-4, 5)
    if a_col:
        A = torch.randint(lo, hi, (K, M), device=dev, generator=g, dtype=torch.int8).to(tt[in_type]).t()
    else:
        A = torch.randint(lo, hi, (M, K), device=dev, generator=g, dtype=torch.int8).to(tt[in_type])
    cols = torch.arange(N, device=dev)
    src = (cols * 7 + 3) % K                      # column n of B has its one entry in row src[n]
    sign = torch.where(cols % 3 == 0, -1, 1)
    if b_col:
        B = torch.zeros((N, K), device=dev, dtype=tt[in_type])
        B[cols, src] = sign.to(tt[in_type])
        B = B.t()
    else:
        B = torch.zeros((K, N), device=dev, dtype=tt[in_type])
        B[src, cols] = sign.to(tt[in_type])
    C = torch.full((M, N), 7, device=dev, dtype=tt[out_type])
    assert max(t.numel() * t.element_size() for t in (A, B, C)) > 1 << 32
    call = GemmCall(A, B, C, variant=_lib.VARIANT_AUTO)   # (the library's own choice, not a recorded one: these shapes are in no table)
    name = _lib.variant_name(call.chosen[0])
    print(in_type, out_type, M, N, K, name, call.chosen[1], flush=True)
    assert kernel in name, name
    call()
    torch.cuda.synchronize()
    step = max(1, (1 << 28) // N)
    for r0 in range(0, M, step):
        want = torch.relu(A[r0:r0 + step][:, src].to(torch.float32) * sign.to(torch.float32)).to(tt[out_type])
        assert torch.equal(C[r0:r0 + step], want), (r0, name)
        del want
    del A, B, C, call
    torch.cuda.empty_cache()


@pytest.mark.gpu
def test_small_tiles_are_chosen_for_problems_that_would_not_fill_the_chip():
    """64 x 64 tiles (a wave has one 32 x 32 block) while 128 x 128 tiles would leave most compute units idle; the larger
    tiles again once a compute unit would get more than two of the small ones (8- and 16-bit inputs)."""
    from accera_amd import _lib
    for t, o in ((_lib.F16, _lib.F16), (_lib.BF16, _lib.F32), (_lib.I8, _lib.I32)):
        for (M, N, K), want in (((1024, 1024, 1024), "mfma 64x64"), ((1536, 1152, 2048), "mfma 64x64"), ((512, 512, 512), "mfma 64x64"),
                                ((2048, 2048, 2048), "mfma 128x128"), ((3072, 1024, 1024), "mfma 128x128")):
            g, b, lds, v = _lib.launch_geometry(t, o, M, N, K, (K, 1), (N, 1), (N, 1))
            assert want in _lib.variant_name(v), (M, N, K, _lib.variant_name(v))
    run_case("f16", "f16", 1024, 1024, 1024, seed=2300)
    run_case("bf16", "f32", 1536, 1152, 2048, seed=2301, b_layout="col", prologue=ora.PRO_NONE)
    run_case("i8", "i32", 1024, 960, 1024, seed=2302, a_layout="col")
    run_case("i8", "i8", 1000, 1024, 512, seed=2303)
