"""Pins the CPU oracle (oracle/) against the reference's known answers and against
what the mathematics fixes.  Everything here runs without a GPU."""
import numpy as np
import pytest
import torch

import oracle as ora


def _rand(rng, shape, t):
    if t == "f32":
        return rng.uniform(-1, 1, shape).astype(np.float32)
    if t == "f16":
        return rng.uniform(-1, 1, shape).astype(np.float16)
    if t == "bf16":
        return ora.to_bf16(rng.standard_normal(shape).astype(np.float32))
    if t == "i8":
        return rng.integers(-128, 128, shape, dtype=np.int8)
    raise ValueError(t)


# ---- reference known answers -------------------------------------------------
# docs/Tutorials/Hello_MatMul.md:165-237 (K=256 -> 1536.42) and
# docs/Tutorials/Optimized_MatMul.md:204-280 (K=128 -> 768.42): A=2, B=3, C=0.42.
@pytest.mark.parametrize("K,expected", [(256, 1536.42), (128, 768.42)])
@pytest.mark.parametrize("schedule", [ora.SCHED_NAIVE, ora.SCHED_TRANSFORMED])
def test_reference_constant_fill_known_answer(K, expected, schedule):
    M, N = 128, 256
    A = np.full((M, K), 2.0, np.float32)
    B = np.full((K, N), 3.0, np.float32)
    C = np.full((M, N), 0.42, np.float32)
    ora.gemm_relu(A, B, C, "f32", "f32", prologue=ora.PRO_NONE, epilogue=ora.EPI_NONE, schedule=schedule)
    np.testing.assert_allclose(C, expected, rtol=1e-6)
    # with ReLU the positive result is unchanged
    C2 = np.full((M, N), 0.42, np.float32)
    ora.gemm_relu(A, B, C2, "f32", "f32", prologue=ora.PRO_NONE, epilogue=ora.EPI_RELU, schedule=schedule)
    assert np.array_equal(C, C2)


# ---- brute force on small signed inputs ----------------------------------------
@pytest.mark.parametrize("in_type,out_type", [("f32", "f32"), ("f16", "f32"), ("f16", "f16"),
                                              ("bf16", "f32"), ("bf16", "bf16"), ("i8", "i32")])
@pytest.mark.parametrize("shape", [(16, 16, 16), (33, 47, 29), (128, 64, 96), (1, 5, 7)])
@pytest.mark.parametrize("schedule", [ora.SCHED_NAIVE, ora.SCHED_TRANSFORMED])
def test_small_against_numpy(in_type, out_type, shape, schedule):
    M, N, K = shape
    rng = np.random.default_rng(1000 + M * 7 + N * 3 + K + len(in_type) + len(out_type))
    A, B = _rand(rng, (M, K), in_type), _rand(rng, (K, N), in_type)
    C = np.zeros((M, N), ora.NP_STORAGE[out_type])
    ora.gemm_relu(A, B, C, in_type, out_type, schedule=schedule)
    want = ora.gemm_relu_exact(A, B, None, in_type, out_type)
    assert (ora.widen(C, out_type) < 0).sum() == 0
    assert (ora.widen(want, out_type) == 0).any() and (ora.widen(want, out_type) > 0).any()  # ReLU really clips
    if in_type == "i8":
        assert np.array_equal(C, want)
    else:
        # float32 sequential sum vs float64 sum: relative 1e-5 plus an absolute term for
        # near-cancelling sums; a narrowed output may additionally differ by one ulp of its type
        tol = {"f32": 1e-5, "f16": 2e-3, "bf16": 1e-2}[out_type]
        np.testing.assert_allclose(ora.widen(C, out_type), ora.widen(want, out_type), rtol=tol, atol=1e-5 * np.sqrt(K))


def test_python_triple_loop_bit_exact_f32():
    """The sequential-k float32 accumulation, retraced with NumPy float32 scalars."""
    rng = np.random.default_rng(7)
    M, N, K = 5, 6, 19
    A, B = _rand(rng, (M, K), "f32"), _rand(rng, (K, N), "f32")
    C0 = _rand(rng, (M, N), "f32")
    C = C0.copy()
    ora.gemm_relu(A, B, C, "f32", "f32", prologue=ora.PRO_NONE, epilogue=ora.EPI_RELU, schedule=ora.SCHED_NAIVE)
    want = np.empty_like(C0)
    for i in range(M):
        for j in range(N):
            acc = np.float32(C0[i, j])
            for k in range(K):
                acc = np.float32(acc + np.float32(A[i, k] * B[k, j]))
            want[i, j] = acc if acc > 0 else np.float32(0)
    assert np.array_equal(C, want)


@pytest.mark.parametrize("in_type,out_type", [("f32", "f32"), ("f16", "f16"), ("bf16", "f32"), ("i8", "i32")])
def test_schedules_bit_identical(in_type, out_type):
    rng = np.random.default_rng(11)
    M, N, K = 50, 70, 130
    A, B = _rand(rng, (M, K), in_type), _rand(rng, (K, N), in_type)
    C1 = np.zeros((M, N), ora.NP_STORAGE[out_type])
    C2 = C1.copy()
    ora.gemm_relu(A, B, C1, in_type, out_type, schedule=ora.SCHED_NAIVE)
    ora.gemm_relu(A, B, C2, in_type, out_type, schedule=ora.SCHED_TRANSFORMED, threads=4)
    assert np.array_equal(C1, C2)


# ---- closed forms ----------------------------------------------------------------
@pytest.mark.parametrize("in_type", ["f32", "f16", "bf16", "i8"])
def test_permutation_b_copies_a_exactly(in_type):
    rng = np.random.default_rng(3)
    M, K = 40, 64
    out_type = "i32" if in_type == "i8" else "f32"
    A = _rand(rng, (M, K), in_type)
    perm = rng.permutation(K)
    P = np.zeros((K, K), np.float32)
    P[perm, np.arange(K)] = 1  # (A@P)[:, j] = A[:, perm[j]]
    Bm = {"f32": P, "f16": P.astype(np.float16), "bf16": ora.to_bf16(P), "i8": P.astype(np.int8)}[in_type]
    C = np.zeros((M, K), ora.NP_STORAGE[out_type])
    ora.gemm_relu(A, Bm, C, in_type, out_type, epilogue=ora.EPI_NONE)
    assert np.array_equal(ora.widen(C, out_type), ora.widen(A, in_type)[:, perm])
    ora.gemm_relu(A, Bm, C, in_type, out_type, epilogue=ora.EPI_RELU)
    assert np.array_equal(ora.widen(C, out_type), np.maximum(ora.widen(A, in_type)[:, perm], 0))


def test_power_of_two_entries_are_exact():
    """Entries +-2^e with small K: every partial sum is exactly representable."""
    rng = np.random.default_rng(5)
    M, N, K = 32, 48, 16
    A = (np.ldexp(1.0, rng.integers(-3, 4, (M, K))) * rng.choice([-1, 1], (M, K))).astype(np.float16)
    B = (np.ldexp(1.0, rng.integers(-3, 4, (K, N))) * rng.choice([-1, 1], (K, N))).astype(np.float16)
    C = np.zeros((M, N), np.float32)
    ora.gemm_relu(A, B, C, "f16", "f32")
    want = np.maximum(A.astype(np.float64) @ B.astype(np.float64), 0)
    assert np.array_equal(C.astype(np.float64), want)


def test_column_major_b_and_strided_views():
    rng = np.random.default_rng(9)
    M, N, K = 24, 40, 56
    A = _rand(rng, (M, K), "bf16")
    B = _rand(rng, (K, N), "bf16")
    Bf = np.asfortranarray(B)
    assert Bf.strides == (2, 2 * K)
    C1 = np.zeros((M, N), np.uint16)
    C2 = np.zeros((M, N), np.uint16, order="F")
    ora.gemm_relu(A, B, C1, "bf16", "bf16")
    ora.gemm_relu(A, Bf, C2, "bf16", "bf16")
    assert np.array_equal(C1, C2)


def test_prologue_set_vs_accumulate():
    """GEMM alpha/beta table of docs/Tutorials/GPU/Tensor_MatMul_ElementWiseOps_GPU.md:85-99."""
    rng = np.random.default_rng(13)
    M, N, K = 32, 32, 64
    A, B = _rand(rng, (M, K), "f16"), _rand(rng, (K, N), "f16")
    C0 = rng.uniform(-4, 4, (M, N)).astype(np.float32)
    Cset, Cacc = C0.copy(), C0.copy()
    ora.gemm_relu(A, B, Cset, "f16", "f32", prologue=ora.PRO_SET0)
    ora.gemm_relu(A, B, Cacc, "f16", "f32", prologue=ora.PRO_NONE)
    P = A.astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_allclose(Cset, np.maximum(P, 0), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(Cacc, np.maximum(P + C0, 0), rtol=1e-5, atol=1e-5)
    assert not np.allclose(Cset, Cacc)


def test_int32_wraparound_and_extremes():
    K = 4
    A = np.full((1, K), -128, np.int8)
    B = np.full((K, 1), -128, np.int8)
    C = np.array([[2**31 - 1 - 3 * 16384]], np.int32)  # + 4*16384 wraps past INT32_MAX
    ora.gemm_relu(A, B, C, "i8", "i32", prologue=ora.PRO_NONE, epilogue=ora.EPI_NONE)
    assert C[0, 0] == -(2**31) + 16384 - 1
    C = np.array([[-(2**31)]], np.int32)
    ora.gemm_relu(np.zeros((1, K), np.int8), B, C, "i8", "i32", prologue=ora.PRO_NONE, epilogue=ora.EPI_RELU)
    assert C[0, 0] == 0


@pytest.mark.parametrize("epi,nan_to", [(ora.EPI_RELU, 0.0), (ora.EPI_RELU_NOCOND, np.nan)])
def test_relu_special_values(epi, nan_to):
    """relu: v>0?v:0 (NaN->0, -0->+0); relu_no_conditional: v*=(v>0) (NaN stays NaN).
    CppPrinterUtils.h:630-643."""
    vals = np.array([[-0.0, np.nan, np.inf, -np.inf, -3.5, 2.25, 0.0, 1e-38]], np.float32)
    A = np.zeros((1, 4), np.float32)  # A@B = 0, so the result is epilogue(C0)
    B = np.zeros((4, vals.shape[1]), np.float32)
    C = vals.copy()
    ora.gemm_relu(A, B, C, "f32", "f32", prologue=ora.PRO_NONE, epilogue=epi)
    got = C[0]
    assert got[2] == np.inf and got[5] == 2.25 and got[7] == np.float32(1e-38)
    assert got[4] == 0 and got[6] == 0 and got[0] == 0
    if np.isnan(nan_to):
        assert np.isnan(got[1])
        assert np.isnan(got[3])  # -inf * 0 = NaN
        assert np.signbit(got[4])  # -3.5 * 0 = -0
    else:
        assert got[1] == 0 and got[3] == 0
        assert not np.signbit(got[0]) and not np.signbit(got[4])


# ---- exhaustive conversion tables ---------------------------------------------------
def test_half_to_float_all_65536_values():
    h = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, np.float32)
    ora.lib().oracle_half_to_float_n(h.ctypes.data, out.ctypes.data, 65536)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))


def test_float_to_half_rne_against_numpy():
    rng = np.random.default_rng(17)
    # every half value, its neighbours' midpoints (ties), random bit patterns, range edges
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    mids = ((h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2).astype(np.float32)
    rnd = rng.integers(0, 2**32, 2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    edge = np.array([65504, 65519.99, 65520, 65536, 1e-8, 2**-25, np.nextafter(np.float32(2**-25), 1), 2**-24,
                     2**-14, np.nextafter(np.float32(2**-14), 0), 0.0, -0.0, np.inf, -np.inf], np.float32)
    x = np.concatenate([h, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)), rnd, edge, -edge])
    out = np.empty(x.size, np.uint16)
    ora.lib().oracle_float_to_half_n(x.ctypes.data, out.ctypes.data, x.size)
    with np.errstate(over="ignore", invalid="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(out[~nan], want[~nan])
    assert np.all(np.isnan(out[nan].view(np.float16)))


def test_bf16_conversions_against_torch():
    rng = np.random.default_rng(19)
    b = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, np.float32)
    ora.lib().oracle_bf16_to_float_n(b.ctypes.data, out.ctypes.data, 65536)
    want = torch.from_numpy(b.view(np.int16).copy()).view(torch.bfloat16).float().numpy()
    assert np.array_equal(out.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(ora.from_bf16(b).view(np.uint32), want.view(np.uint32))

    hi = (b.astype(np.uint32) << 16)
    ties = np.concatenate([hi | 0x8000, hi | 0x7FFF, hi | 0x8001])  # exact ties and their neighbours
    rnd = rng.integers(0, 2**32, 2_000_000, dtype=np.uint64).astype(np.uint32)
    x = np.concatenate([hi, ties, rnd]).astype(np.uint32).view(np.float32)
    got = np.empty(x.size, np.uint16)
    ora.lib().oracle_float_to_bf16_n(x.ctypes.data, got.ctypes.data, x.size)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(ora.from_bf16(got[nan])))
    assert np.array_equal(ora.to_bf16(x)[~nan], want[~nan])


def test_bad_type_combination_is_rejected():
    A = np.zeros((4, 4), np.int8)
    C = np.zeros((4, 4), np.float32)
    with pytest.raises(ValueError):
        ora.gemm_relu(A, A, C, "i8", "f32")


# ---- SET / SCALE fragment ops of the NumPy restatement, pinned by closed forms ------------------
def test_alpha_beta_table_constant_fill_known_answers():
    """The reference's GEMM table C = alpha*(A@B) + beta*C
    (docs/Tutorials/GPU/Tensor_MatMul_ElementWiseOps_GPU.md:85-99) on its own constant fills
    A = 2, B = 3, C = 0.42 (docs/Tutorials/Hello_MatMul.md:165-237): every entry is a closed form."""
    M, N, K = 8, 16, 256
    A = np.full((M, K), 2, np.float32)
    B = np.full((K, N), 3, np.float32)
    C = np.full((M, N), 0.42, np.float32)
    e = lambda **kw: ora.gemm_relu_exact(A, B, C, "f32", "f32", narrow_out=False, **kw)
    assert np.all(e(prologue=ora.PRO_SET, prologue_arg=0, epilogue=ora.EPI_NONE) == 6.0 * K)                       # C = A@B
    assert np.allclose(e(prologue=ora.PRO_NONE, epilogue=ora.EPI_NONE), 6.0 * K + np.float32(0.42))                # C += A@B
    assert np.allclose(e(prologue=ora.PRO_SCALE, prologue_arg=0.5, epilogue=ora.EPI_NONE), 6.0 * K + 0.5 * np.float32(0.42))
    assert np.all(e(prologue=ora.PRO_SET, prologue_arg=0, epilogue=ora.EPI_SCALE, epilogue_arg=5.0) == 30.0 * K)   # alpha = 5
    assert np.all(e(prologue=ora.PRO_SET, prologue_arg=-7.0, epilogue=ora.EPI_NONE) == 6.0 * K - 7.0)
    assert np.all(e(prologue=ora.PRO_NONE, epilogue=ora.EPI_SET, epilogue_arg=1.25) == 1.25)
    # epilogue SCALE acts on the whole fragment, prologue'd C included: (beta*C + A@B) * alpha
    got = e(prologue=ora.PRO_SCALE, prologue_arg=2.0, epilogue=ora.EPI_SCALE, epilogue_arg=-3.0)
    assert np.allclose(got, -3.0 * (6.0 * K + 2.0 * np.float32(0.42)))


def test_int_ops_cast_operands_and_wrap():
    """Operands are cast to the accumulator type (int for int8 inputs: 2.9 -> 2) and int32 sums wrap."""
    rng = np.random.default_rng(5)
    A = rng.integers(-128, 128, (16, 32), dtype=np.int8)
    B = rng.integers(-128, 128, (32, 16), dtype=np.int8)
    C = rng.integers(-1000, 1000, (16, 16)).astype(np.int32)
    P = A.astype(np.int64) @ B.astype(np.int64)
    wrap = lambda x: ((x + 2**31) % 2**32) - 2**31
    got = ora.gemm_relu_exact(A, B, C, "i8", "i32", ora.PRO_SCALE, ora.EPI_SCALE, prologue_arg=2.9, epilogue_arg=-3.7)
    assert np.array_equal(got, wrap((P + 2 * C.astype(np.int64)) * -3).astype(np.int32))
    got = ora.gemm_relu_exact(A, B, C, "i8", "i32", ora.PRO_SET, ora.EPI_SCALE, prologue_arg=11, epilogue_arg=2**20)
    assert np.array_equal(got, wrap((P + 11) * 2**20).astype(np.int32)) and (np.abs((P + 11) * 2**20) >= 2**31).any()


@pytest.mark.parametrize("out_type,np_t,bits", [("i16", np.int16, 16), ("i8", np.int8, 8)])
def test_narrow_integer_outputs_keep_low_bits_and_widen_with_sign(out_type, np_t, bits):
    """int8 -> int16 / int8 (pairs of /root/reference/accera/python/accera/Targets.py:814-821): the
    accumulator fragment is int32; C converts to it like a C integer conversion (sign kept) and
    back by dropping the high bits (CppPrinterUtils.h:277-293).  Pinned by known answers worked by
    hand and by a brute-force Python loop, on both restatements."""
    K = 512
    ones = np.ones((4, K), np.int8)
    # 512 * 127 = 65024 = 0xFE00: int16 -> -512, int8 -> 0x00 = 0
    by_hand = {"i16": -512, "i8": 0}[out_type]
    for f in (lambda A, B, C, *a: ora.gemm_relu(A, B, C.copy(), "i8", out_type, *a),
              lambda A, B, C, *a: ora.gemm_relu_exact(A, B, C, "i8", out_type, *a)):
        got = f(ones, np.full((K, 4), 127, np.int8), np.zeros((4, 4), np_t), ora.PRO_SET0, ora.EPI_NONE)
        assert got.dtype == np_t and np.all(got == by_hand)
        # C = -1 (all bits set) counts as -1: -1 + 512 = 511 = 0x1FF: int16 -> 511, int8 -> 0xFF = -1
        got = f(ones, np.ones((K, 4), np.int8), np.full((4, 4), -1, np_t), ora.PRO_NONE, ora.EPI_RELU)
        assert np.all(got == {"i16": 511, "i8": -1}[out_type])
        # ReLU acts on the int32 sum, before the narrowing: -65024 -> 0
        got = f(ones, np.full((K, 4), -127, np.int8), np.zeros((4, 4), np_t), ora.PRO_SET0, ora.EPI_RELU)
        assert np.all(got == 0)
    rng = np.random.default_rng(bits)
    A = rng.integers(-128, 128, (5, 37), dtype=np.int8)
    B = rng.integers(-128, 128, (37, 6), dtype=np.int8)
    C = rng.integers(-2 ** (bits - 1), 2 ** (bits - 1), (5, 6)).astype(np_t)
    want = np.zeros((5, 6), np_t)
    for i in range(5):
        for j in range(6):
            s = int(C[i, j]) + sum(int(A[i, k]) * int(B[k, j]) for k in range(37))
            s = max(s, 0) & (2 ** bits - 1)
            want[i, j] = s - 2 ** bits if s >= 2 ** (bits - 1) else s
    assert np.array_equal(ora.gemm_relu(A, B, C.copy(), "i8", out_type, ora.PRO_NONE, ora.EPI_RELU), want)
    assert np.array_equal(ora.gemm_relu_exact(A, B, C, "i8", out_type, ora.PRO_NONE, ora.EPI_RELU), want)
