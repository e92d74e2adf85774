"""The entry point that allocates nothing (acc950_gemm_ops_static) against acc950_gemm_ops: same kernels, the K-split
workspace in the library's own device image instead of a per-stream allocation.  Two calls in a row, the second on
a smaller problem, both bit-identical to the allocating entry point and within tolerance of the CPU oracle."""
import numpy as np
import pytest

import oracle as ora
from tests.util import assert_matches, make_input, out_zeros, to_device, to_host

pytestmark = pytest.mark.gpu


def _call(entry, dA, dB, dC, M, N, K, k_splits, stream):
    from accera_amd import _lib
    return entry(_lib.F16, _lib.F16, M, N, K, dA.data_ptr(), K, 1, dB.data_ptr(), N, 1, dC.data_ptr(), N, 1,
                 _lib.PROLOGUE_SET0, 0.0, _lib.EPILOGUE_RELU, 0.0, _lib.VARIANT_AUTO, k_splits, stream)


def test_static_workspace_entry_point_matches_the_allocating_one():
    import torch
    from accera_amd import _lib
    L = _lib.lib()
    _lib.check(L.acc950_init(0))
    stream = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(2024)
    # decode shape first (its slow-phase column blocks are shared by two workgroups each: 2.7 MiB of partial sums),
    # then a smaller problem with an explicit K split over four workgroups per column block; then a small square output
    # with a long K, which the library splits by itself on an MFMA kernel (32 slices of 64 KiB of partial sums)
    cases = [(8, 11008, 4096, 0), (4, 2048, 1024, 4), (128, 128, 8192, 0)]
    data = []
    for M, N, K, ks in cases:
        A = make_input(rng, (M, K), "f16", "normal")
        B = (make_input(rng, (K, N), "f16", "normal").astype(np.float32) * 0.05).astype(np.float16)
        dA, dB = to_device(A, "f16"), to_device(B, "f16")
        d_ref, d_new = to_device(np.full((M, N), 7, np.float16), "f16"), to_device(np.full((M, N), 9, np.float16), "f16")
        _lib.check(_call(L.acc950_gemm_ops, dA, dB, d_ref, M, N, K, ks, stream))
        data.append((A, B, dA, dB, d_ref, d_new))
    torch.cuda.synchronize()
    assert _lib.launch_geometry(_lib.F16, _lib.F16, 128, 128, 8192, (8192, 1), (128, 1), (128, 1))[0][2] > 1
    allocations_before = _lib.allocation_probe()
    assert allocations_before >= 2  # the allocating entry point made this stream's workspace
    for rep in range(2):  # the pair of calls twice: the second round finds the array as the first left it
        for (M, N, K, ks), (A, B, dA, dB, d_ref, d_new) in zip(cases, data):
            d_new.fill_(9)
            _lib.check(_call(L.acc950_gemm_ops_static, dA, dB, d_new, M, N, K, ks, stream))
    torch.cuda.synchronize()
    assert _lib.allocation_probe() == allocations_before, "the static entry point must not allocate device memory"
    for (M, N, K, ks), (A, B, dA, dB, d_ref, d_new) in zip(cases, data):
        got, ref = to_host(d_new, "f16"), to_host(d_ref, "f16")
        assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), (M, N, K)
        want = ora.gemm_relu_exact(A, B, out_zeros(M, N, "f16"), "f16", "f16", ora.PRO_SET0, ora.EPI_RELU)
        assert_matches(got, want, "f16", K)
        assert (got == 0).any() and (got > 0).any()
    # a K split whose partial sums do not fit the array is refused, nothing runs
    (M, N, K, _), (A, B, dA, dB, d_ref, d_new) = cases[0], data[0]
    d_new.fill_(9)
    rc = _call(L.acc950_gemm_ops_static, dA, dB, d_new, M, N, K, 8, stream)
    assert rc == _lib.UNSUPPORTED and b"built-in workspace" in L.acc950_last_error()
    torch.cuda.synchronize()
    assert (to_host(d_new, "f16") == 9).all()
    # an MFMA kernel's K split that does not fit runs unsplit instead (512 x 1024 x 8192: two slices of 2 MiB are the whole
    # array, part of which holds the counters)
    M, N, K = 512, 1024, 8192
    A = make_input(rng, (M, K), "f16", "normal")
    B = (make_input(rng, (K, N), "f16", "normal").astype(np.float32) * 0.03).astype(np.float16)
    dA, dB, dC = to_device(A, "f16"), to_device(B, "f16"), to_device(np.full((M, N), 9, np.float16), "f16")
    assert _lib.launch_geometry(_lib.F16, _lib.F16, M, N, K, (K, 1), (N, 1), (N, 1))[0][2] > 1
    _lib.check(_call(L.acc950_gemm_ops_static, dA, dB, dC, M, N, K, 0, stream))
    torch.cuda.synchronize()
    assert _lib.allocation_probe() == allocations_before
    rows = rng.choice(M, 16, replace=False)
    assert_matches(to_host(dC, "f16")[rows], ora.gemm_relu_exact(A[rows], B, out_zeros(16, N, "f16"), "f16", "f16", ora.PRO_SET0, ora.EPI_RELU), "f16", K)
    # few rows against a large B: the allocating entry point takes the streaming kernel's 256-column blocks in four slices
    # (8 MiB of partial sums), which the array does not hold; here the library stays with the 64-column default, unsplit
    from accera_amd import tune
    M, N, K = 8, 16384, 8192
    v, ks = tune.own_choice(_lib.F16, _lib.F16, M, N, K, False, False, 1.0, 0.0)
    assert "cols/wg=256" in _lib.variant_name(v) and ks == 4
    A = make_input(rng, (M, K), "f16", "normal")
    B = (make_input(rng, (K, N), "f16", "normal").astype(np.float32) * 0.03).astype(np.float16)
    dA, dB, dC = to_device(A, "f16"), to_device(B, "f16"), to_device(np.full((M, N), 9, np.float16), "f16")
    _lib.check(_call(L.acc950_gemm_ops_static, dA, dB, dC, M, N, K, 0, stream))
    torch.cuda.synchronize()
    assert _lib.allocation_probe() == allocations_before
    assert_matches(to_host(dC, "f16"), ora.gemm_relu_exact(A, B, out_zeros(M, N, "f16"), "f16", "f16", ora.PRO_SET0, ora.EPI_RELU), "f16", K)


def test_static_workspace_entry_point_under_graph_capture():
    """What the entry point is for: a chain of launches recorded into a HIP graph (no allocation may happen while a
    stream is capturing) and replayed.  A two-layer decode step -- skinny GEMM + ReLU, then a second skinny GEMM on its
    output -- plus a small-output GEMM that the library splits over K (two kernels); every replay is checked against the
    same calls made eagerly, with the program's own work and synchronisations between the replays."""
    import torch
    from accera_amd import _lib
    L = _lib.lib()
    _lib.check(L.acc950_init(0))
    rng = np.random.default_rng(77)
    M, H, F = 8, 4096, 11008
    X = make_input(rng, (M, H), "f16", "normal")
    W1 = (make_input(rng, (H, F), "f16", "normal").astype(np.float32) * 0.03).astype(np.float16)
    W2 = (make_input(rng, (F, H), "f16", "normal").astype(np.float32) * 0.03).astype(np.float16)
    P, Q = make_input(rng, (128, 8192), "f16", "normal"), (make_input(rng, (8192, 128), "f16", "normal").astype(np.float32) * 0.03).astype(np.float16)
    dX, dW1, dW2, dP, dQ = (to_device(a, "f16") for a in (X, W1, W2, P, Q))
    mk = lambda r, c: to_device(np.zeros((r, c), np.float16), "f16")
    hid_e, out_e, sq_e, hid_g, out_g, sq_g = mk(M, F), mk(M, H), mk(128, 128), mk(M, F), mk(M, H), mk(128, 128)

    def step(entry, hid, out, sq, stream):
        args = lambda A, B, C, m, n, k, epi: (_lib.F16, _lib.F16, m, n, k, A.data_ptr(), k, 1, B.data_ptr(), n, 1, C.data_ptr(), n, 1,
                                              _lib.PROLOGUE_SET0, 0.0, epi, 0.0, _lib.VARIANT_AUTO, 0, stream)
        _lib.check(entry(*args(dX, dW1, hid, M, F, H, _lib.EPILOGUE_RELU)))
        _lib.check(entry(*args(hid, dW2, out, M, H, F, _lib.EPILOGUE_NONE)))
        _lib.check(entry(*args(dP, dQ, sq, 128, 128, 8192, _lib.EPILOGUE_RELU)))

    # eager, on the current stream (also loads every kernel's code and sets its LDS limit before the capture)
    step(L.acc950_gemm_ops_static, hid_e, out_e, sq_e, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want = [to_host(t, "f16").copy() for t in (hid_e, out_e, sq_e)]
    assert_matches(want[0], ora.gemm_relu_exact(X, W1, out_zeros(M, F, "f16"), "f16", "f16", ora.PRO_SET0, ora.EPI_RELU), "f16", H)
    before = _lib.allocation_probe()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            step(L.acc950_gemm_ops_static, hid_g, out_g, sq_g, side.cuda_stream)
    assert _lib.allocation_probe() == before
    for replay in range(4):
        for t in (hid_g, out_g, sq_g):
            t.fill_(3)                                   # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip((hid_g, out_g, sq_g), want):
            assert np.array_equal(to_host(got, "f16").view(np.uint16), ref.view(np.uint16)), replay
        if replay == 1:                                  # the same entry point eagerly, between replays: the array is shared
            step(L.acc950_gemm_ops_static, hid_e, out_e, sq_e, torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
