"""The C-ABI library loads without a GPU and exports every symbol the header declares;
argument checking and the launch-geometry query run on the host alone."""
import ctypes
import os
import re

import pytest

from accera_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header="accera_mi355x_gemm.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(acc950_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    names = _declared()
    assert len(names) >= 9 and set(_lib.EXPORTS) == set(names)
    L = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert getattr(L, n) is not None, n
    # the measurement aids are a library of their own; the product library holds none of them
    probes = _declared("accera_mi355x_probes.h")
    assert set(_lib.PROBE_EXPORTS) == set(probes) and not set(probes) & set(names)
    P = ctypes.CDLL(_lib.PROBES_LIB_PATH)
    for n in probes:
        assert getattr(P, n) is not None, n
        assert not hasattr(L, n), f"{n} belongs in the probes library only"


def test_phase_probe_refuses_what_its_kernels_do_not_take_before_launching():
    """The timed kernels take whole 256x256 tiles of dense, aligned operands only; the probe says so itself and runs nothing
    (no GPU is needed to be refused)."""
    P = _lib.probes()
    out = (ctypes.c_double * 8)()
    ok_ptrs = (0x10000, 0x20000, 0x30000)
    for M, N, K in ((300, 512, 512), (512, 300, 512), (512, 512, 100), (128, 512, 512), (512, 512, 0)):
        rc = P.acc950_mfma_phase_probe(_lib.F16, _lib.F32, M, N, K, *ok_ptrs, out)
        assert rc == _lib.UNSUPPORTED and b"multiples of 256" in P.acc950_probes_last_error(), (M, N, K)
    assert P.acc950_mfma_phase_probe(_lib.I8, _lib.I32, 512, 512, 96, *ok_ptrs, out) == _lib.UNSUPPORTED          # K of 64 bytes
    assert P.acc950_mfma_phase_probe(_lib.F16, _lib.F32, 512, 512, 512, 0x10008, 0x20000, 0x30000, out) == _lib.UNSUPPORTED
    assert P.acc950_mfma_phase_probe(_lib.F32, _lib.F32, 512, 512, 512, *ok_ptrs, out) == _lib.UNSUPPORTED
    assert P.acc950_mfma_phase_probe(_lib.F16, _lib.I32, 512, 512, 512, *ok_ptrs, out) == _lib.INVALID_ARGUMENT
    assert P.acc950_mfma_phase_probe(_lib.F16, _lib.F32, 512, 512, 512, None, 0x20000, 0x30000, out) == _lib.INVALID_ARGUMENT
    with pytest.raises(_lib.Acc950Error) as e:
        _lib.mfma_phase_probe(_lib.F16, _lib.F32, 300, 512, 512, *ok_ptrs)
    assert e.value.code == _lib.UNSUPPORTED and "multiples of 256" in str(e.value)


def test_variant_table_is_described():
    assert _lib.num_variants() >= 8 and _lib.num_skinny_variants() >= 1
    names = [_lib.variant_name(v) for v in range(_lib.num_variants())]
    assert len(set(names)) == len(names)
    assert any("direct" in n for n in names) and any("edge" in n for n in names)
    assert "skinny" in _lib.variant_name(_lib.VARIANT_SKINNY_BASE)
    with pytest.raises(_lib.Acc950Error):
        _lib.variant_name(_lib.num_variants())


# launch geometry expectations for the BASELINE configurations: grid = tiles of the block
# tile, block = waves * 64 (Plan.py:937-956 derives the same quantities from the bound indices;
# mfma_tests.py:2562,2572 pins them as <<<dim3(...), dim3(...)>>> strings)
def test_launch_geometry_of_the_configs():
    g, b, lds, v = _lib.launch_geometry(_lib.F16, _lib.F32, 4096, 4096, 4096, (4096, 1), (4096, 1), (4096, 1))
    name = _lib.variant_name(v)
    bm, bn = map(int, re.search(r"mfma (\d+)x(\d+)", name).groups())
    assert g == [(4096 // bm) * (4096 // bn), 1, 1] and b[0] % 64 == 0 and lds == 2 * (bm + bn) * 128
    g, b, lds, v = _lib.launch_geometry(_lib.BF16, _lib.BF16, 4096, 3072, 768, (768, 1), (1, 768), (3072, 1))
    assert "B=col-major" in _lib.variant_name(v)
    g, b, lds, v = _lib.launch_geometry(_lib.I8, _lib.I32, 8192, 8192, 8192, (8192, 1), (8192, 1), (8192, 1))
    assert "mfma" in _lib.variant_name(v)
    g, b, lds, v = _lib.launch_geometry(_lib.F16, _lib.F16, 8, 11008, 4096, (4096, 1), (11008, 1), (11008, 1))
    assert "skinny" in _lib.variant_name(v) and g[0] * g[1] >= 43 and b[0] % 64 == 0
    g, b, lds, v = _lib.launch_geometry(_lib.F32, _lib.F32, 512, 512, 512, (512, 1), (512, 1), (512, 1))
    assert v == _lib.VARIANT_F32_MFMA and g[:2] == [16, 16]
    # sizes that are not multiples of the 16-byte vector take the MFMA kernel whose fill accepts unaligned chunks; an operand with
    # no unit stride falls to the thread-bound kernel; explicit variants refuse what they do not take
    g, b, lds, v = _lib.launch_geometry(_lib.F16, _lib.F32, 100, 71, 40, (40, 1), (71, 1), (71, 1))
    assert "any-alignment" in _lib.variant_name(v) and "mfma 64x64" in _lib.variant_name(v) and g == [4, 1, 1]
    g, b, lds, v = _lib.launch_geometry(_lib.F16, _lib.F32, 100, 71, 40, (80, 2), (71, 1), (71, 1))
    assert v == _lib.VARIANT_GENERIC and g[:2] == [2, 2]
    with pytest.raises(_lib.Acc950Error) as e:
        _lib.launch_geometry(_lib.F16, _lib.F32, 100, 71, 40, (40, 1), (71, 1), (71, 1), variant=0)
    assert e.value.code == _lib.UNSUPPORTED


def test_argument_checking_on_the_host():
    with pytest.raises(_lib.Acc950Error) as e:
        _lib.launch_geometry(_lib.I8, _lib.F32, 64, 64, 64, (64, 1), (64, 1), (64, 1))
    assert e.value.code == _lib.INVALID_ARGUMENT and "type pair" in str(e.value)
    with pytest.raises(_lib.Acc950Error):
        _lib.launch_geometry(_lib.F16, _lib.F32, -1, 64, 64, (64, 1), (64, 1), (64, 1))
    with pytest.raises(_lib.Acc950Error):
        _lib.launch_geometry(_lib.F16, _lib.F32, 64, 64, 64, (-64, 1), (64, 1), (64, 1))
    # null pointers are rejected before anything is launched
    rc = _lib.lib().acc950_gemm_relu(_lib.F16, _lib.F32, 64, 64, 64, None, 64, 1, None, 64, 1, None, 64, 1, 1, 1, None)
    assert rc == _lib.INVALID_ARGUMENT and b"null" in _lib.lib().acc950_last_error()
    # empty problems are a no-op
    assert _lib.lib().acc950_gemm_relu(_lib.F16, _lib.F32, 0, 64, 64, None, 64, 1, None, 64, 1, None, 64, 1, 1, 1, None) == 0


def test_sweep_tool_lists_the_variants_that_take_a_problem():
    """accera_amd.tune enumerates the points of the variant space for a shape (counterpart of
    get_variants, tools/benchmarkers/accera_gemm.py:187-348) without touching the GPU."""
    from accera_amd import tune
    c = tune.candidates(_lib.F16, _lib.F32, 4096, 4096, 4096, (4096, 1), (4096, 1), (4096, 1))
    names = [_lib.variant_name(v) for v, _ in c]
    assert any("pingpong" in n for n in names) and any("generic" in n for n in names)
    assert not any("skinny" in n or "A=col-major" in n or " B=col-major" in n for n in names)
    c = tune.candidates(_lib.F16, _lib.F16, 8, 11008, 4096, (4096, 1), (11008, 1), (11008, 1))
    assert any("skinny mfma" in _lib.variant_name(v) and sp == 4 for v, sp in c)
    c = tune.candidates(_lib.F16, _lib.F32, 1024, 1024, 1024, (1, 1024), (1024, 1), (1024, 1))
    assert all("A=col-major" in _lib.variant_name(v) or "generic" in _lib.variant_name(v) for v, _ in c)
    import csv, os
    with open(os.path.join(os.path.dirname(tune.__file__), "shapes", "transformer_gemm.csv")) as f:
        rows = list(csv.DictReader(f))
    assert len(rows) >= 10 and {"m", "n", "k", "transA", "transB", "alpha", "beta"} <= set(rows[0])


def test_sweep_tool_audits_the_library_s_own_choice(tmp_path):
    """accera_amd.tune --audit: the kernel and K slices the library takes by itself against the fastest row of a sweep csv."""
    import csv
    from accera_amd import tune
    v, ks = tune.own_choice(_lib.F16, _lib.F32, 4096, 4096, 4096, False, False, 1.0, 0.0)
    chosen = _lib.variant_name(v)
    assert "hand-laid loop" in chosen and ks == 1
    other = next(_lib.variant_name(i) for i in range(_lib.num_variants()) if "pingpong" in _lib.variant_name(i))
    rows = [dict(m=4096, n=4096, k=4096, transA=0, transB=0, alpha=1.0, beta=0.0, type="f16", out_type="f32", variant=v, k_splits=0, kernel=chosen, time_ms=0.1),
            dict(m=4096, n=4096, k=4096, transA=0, transB=0, alpha=1.0, beta=0.0, type="f16", out_type="f32", variant=0, k_splits=0, kernel=other, time_ms=0.08),
            dict(m=4096, n=4096, k=4096, transA=0, transB=0, alpha=1.0, beta=0.0, type="f16", out_type="f16", variant=-2, k_splits=0, kernel="vendor library (torch.matmul)", time_ms=0.01)]
    path = tmp_path / "sweep.csv"
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=list(rows[0]))
        w.writeheader()
        w.writerows(rows)
    lines = []
    geomean, worst = tune.audit(str(path), log=lines.append)
    assert abs(geomean - 1.25) < 1e-9 and len(worst) == 1 and worst[0][2] == chosen and worst[0][5] == other   # (the vendor row is no candidate)
    assert "1 problems" in lines[-1] and "1.2500" in lines[-1]


def test_choices_of_the_cost_model():
    """What the library takes by itself where measurements decided it (numbers in capi.hip next to each rule)."""
    from accera_amd import tune
    name = lambda *a: (lambda v, ks: (_lib.variant_name(v), ks))(*tune.own_choice(*a))
    # a last round that is half empty does not cost a whole round: one and a half rounds of 256 x 256 tiles stay on the four-wave kernel
    n, ks = name(_lib.F16, _lib.F16, 2048, 12288, 4096, False, False, 1.0, 0.0)
    assert "256x256" in n and "hand-laid loop" in n and ks == 1
    # a short K is not split, however few the tiles; a long one is
    assert name(_lib.F16, _lib.F16, 256, 256, 256, False, False, 1.0, 1.0)[1] == 1
    assert name(_lib.F16, _lib.F16, 64, 1152, 448, False, False, 1.0, 0.0)[1] == 1
    assert name(_lib.F16, _lib.F16, 2048, 256, 1536, False, False, 1.0, 0.0)[1] == 1      # (128 tiles: the partial sums cost more than the slices save)
    assert name(_lib.F16, _lib.F16, 64, 320, 1728, False, False, 1.0, 0.0)[1] > 1
    assert name(_lib.F16, _lib.F16, 768, 320, 30522, False, False, 1.0, 0.0)[1] >= 8
    # register-staged kernels (unaligned K): their steps are worth three of the direct kernels', no more
    assert name(_lib.F16, _lib.F16, 512, 128, 196, True, False, 1.0, 1.0)[1] == 1
    assert name(_lib.F16, _lib.F16, 6272, 32, 513, False, False, 1.0, 0.0)[1] == 1
    assert name(_lib.F16, _lib.F16, 196, 64, 801, False, False, 1.0, 0.0)[1] > 1
    # 128 x 128 tiles, two workgroups per CU: two stages of 128 bytes of K
    n, _ = name(_lib.F16, _lib.F16, 3072, 2304, 4096, False, True, 1.0, 1.0)
    assert ("128x128 kb128" in n and "stages=2" in n) or "256x256" in n
    # fp32: tiled kernels with direct fills where they apply, the kernel of 32 x 32 blocks for one round of blocks (512^3) and against the register-staged kernels
    assert "fp32 mfma 32x32" in name(_lib.F32, _lib.F32, 512, 512, 512, False, False, 1.0, 0.0)[0]
    assert "64x64" in name(_lib.F32, _lib.F32, 1152, 384, 64, True, False, 1.0, 1.0)[0]
    n, ks = name(_lib.F32, _lib.F32, 768, 576, 1024, False, False, 1.0, 1.0)
    assert "fill=direct" in n and ks > 1
    assert "fp32 mfma 32x32" in name(_lib.F32, _lib.F32, 800, 126, 49, True, False, 1.0, 1.0)[0]
    # few rows of A: the streaming kernel's 64-column blocks for the decode shape of the benchmark, its 256-column blocks (with
    # the K split that fills the chip in one round) once there are enough of them or the default would stream half lines
    narrow, wide = "skinny mfma cols/wg=64 waves=4 depth=4", "skinny mfma cols/wg=256 waves=4 depth=4"
    assert name(_lib.F16, _lib.F16, 8, 11008, 4096, False, False, 1.0, 0.0) == (narrow, 1)
    assert name(_lib.F16, _lib.F16, 8, 16384, 4096, False, False, 1.0, 0.0) == (narrow, 1)     # (two slices would fill half the chip)
    assert name(_lib.F16, _lib.F16, 8, 16384, 8192, False, False, 1.0, 0.0) == (wide, 4)
    assert name(_lib.BF16, _lib.BF16, 8, 22016, 8192, False, False, 1.0, 0.0) == (wide, 2)
    assert name(_lib.F16, _lib.F16, 8, 65536, 8192, False, False, 1.0, 0.0) == (wide, 1)
    assert name(_lib.F16, _lib.F16, 8, 66048, 4096, False, False, 1.0, 0.0) == (narrow, 1)     # (258 wide blocks: a second round for two of them)
    assert name(_lib.F16, _lib.F16, 32, 16384, 8192, False, False, 1.0, 0.0) == (narrow, 1)    # (more rows: the second trip costs more)
    assert name(_lib.F16, _lib.F16, 32, 16384, 16384, False, False, 1.0, 0.0) == (wide, 4)
    assert name(_lib.I8, _lib.I32, 8, 12288, 16384, False, False, 1.0, 0.0) == (wide, 4)
    assert name(_lib.I8, _lib.I32, 8, 8192, 8192, False, False, 1.0, 0.0) == (wide, 4)
    assert name(_lib.I8, _lib.I32, 8, 4096, 8192, False, False, 1.0, 0.0)[0] == narrow
    # a few dozen to a few hundred rows against a B far beyond the caches: a tile as tall as A (B is streamed once) and the K
    # slices that make about 256 workgroups (512 of the register-staged ones); the slices alone from 64 MB of B on
    n, ks = name(_lib.F16, _lib.F16, 128, 16384, 16384, False, False, 1.0, 0.0)
    assert "128x128" in n and "fill=direct" in n and ks == 2
    n, ks = name(_lib.F16, _lib.F16, 33, 8192, 28672, False, False, 1.0, 0.0)
    assert "64x64" in n and "fill=direct" in n and ks == 4                              # (fewer rows than the tile has: direct fills all the same)
    n, ks = name(_lib.F16, _lib.F16, 100, 8192, 28672, False, False, 1.0, 0.0)
    assert "128x128" in n and "fill=direct" in n and ks == 4
    n, ks = name(_lib.F16, _lib.F16, 100, 8192, 28672, True, False, 1.0, 0.0)           # (a column-major A: the register-staged edge form)
    assert "128x128" in n and "edge" in n and ks == 8
    n, ks = name(_lib.F16, _lib.F16, 8, 11008, 4096, False, True, 1.0, 0.0)            # a decode step against a K-contiguous B
    assert "64x64" in n and "fill=direct" in n and ks == 1
    n, ks = name(_lib.F16, _lib.F16, 8, 4096, 4096, False, True, 1.0, 0.0)             # (fewer than 64 rows: from 16 MB of B on)
    assert "64x64" in n and "fill=direct" in n and ks == 4
    assert "edge" in name(_lib.F16, _lib.F16, 8, 2048, 2048, False, True, 1.0, 0.0)[0]  # (8 MB of B: as before)
    assert name(_lib.F16, _lib.F16, 64, 8192, 2048, False, False, 1.0, 0.0)[1] == 1     # (64 rows and 32 MB: the general rule's slices)
    n, ks = name(_lib.BF16, _lib.BF16, 256, 28672, 8192, False, False, 1.0, 0.0)
    assert "256x256" in n and "hand-laid loop" in n and ks == 2
    n, ks = name(_lib.F16, _lib.F16, 256, 32000, 4096, False, False, 1.0, 0.0)
    assert "256x256" in n and ks == 1                                                    # (two slices' partial sums would be a quarter of B)
    n, ks = name(_lib.F16, _lib.F16, 64, 8192, 28672, False, True, 1.0, 0.0)
    assert "64x64" in n and "fill=direct" in n and ks == 4
    assert name(_lib.F16, _lib.F16, 64, 16384, 16384, False, False, 1.0, 0.0)[1] == 1   # (256 tiles stream by themselves)
    n, ks = name(_lib.F16, _lib.F16, 100, 11008, 4096, False, False, 1.0, 0.0)
    assert "64x64" in n and "fill=direct" in n and ks == 1                              # (90 MB: the general rule's tiles, 344 of them)


def test_bound_call_handles_without_launching():
    """acc950_bind validates and chooses once; handles are reused after acc950_unbind; unknown handles
    are reported.  (No launch here: there is no GPU on the CPU test tier.)"""
    import ctypes
    L = _lib.lib()
    h = ctypes.c_int(-1)
    args = (_lib.F16, _lib.F32, 1, 256, 256, 256, 0x10000, 0, 256, 1, 0x20000, 0, 256, 1, 0x30000, 0, 256, 1,
            _lib.PROLOGUE_SET0, 0.0, _lib.EPILOGUE_RELU, 0.0, _lib.VARIANT_AUTO, 0, None)
    assert L.acc950_bind(*args, ctypes.byref(h)) == _lib.OK and h.value >= 0
    first = h.value
    v, ks = ctypes.c_int(-5), ctypes.c_int(-5)
    assert L.acc950_bound_choice(first, ctypes.byref(v), ctypes.byref(ks)) == _lib.OK
    assert "mfma" in _lib.variant_name(v.value) and ks.value >= 1
    assert L.acc950_unbind(first) == _lib.OK
    assert L.acc950_unbind(first) == _lib.INVALID_ARGUMENT and L.acc950_launch(first) == _lib.INVALID_ARGUMENT
    assert L.acc950_bound_choice(first, ctypes.byref(v), ctypes.byref(ks)) == _lib.INVALID_ARGUMENT
    assert L.acc950_bind(*args, ctypes.byref(h)) == _lib.OK and h.value == first   # slot reused
    assert L.acc950_unbind(first) == _lib.OK
    bad = list(args)
    bad[6] = 0   # null A
    assert L.acc950_bind(*bad, ctypes.byref(h)) == _lib.INVALID_ARGUMENT
    bad = list(args)
    bad[22] = 57 + 1000   # unknown variant
    assert L.acc950_bind(*bad, ctypes.byref(h)) == _lib.INVALID_ARGUMENT
    # A's stride between consecutive k and B's between consecutive columns travel as 32-bit kernel arguments
    for where in (9, 13):   # a_col_stride, b_col_stride
        bad = list(args)
        bad[where] = 1 << 31
        assert L.acc950_bind(*bad, ctypes.byref(h)) == _lib.UNSUPPORTED and b"2^31" in L.acc950_last_error()


def test_tuned_table_is_consulted_by_name_and_validated(tmp_path, monkeypatch):
    """accera_amd.tuned: entries name kernels by description; unknown kernels and kernels the library
    refuses for the problem are ignored."""
    from accera_amd import tuned
    path = tmp_path / "tuned.json"
    monkeypatch.setenv("ACCERA_AMD_TUNED", str(path))
    rows = [dict(m=4096, n=4096, k=4096, transA=0, transB=0, alpha=1.0, beta=0.0, type="f16", out_type="f32", variant=1, k_splits=0,
                 kernel=_lib.variant_name(1), time_ms=0.2, TFlops=1.0, correct=True),
            dict(m=4096, n=4096, k=4096, transA=0, transB=0, alpha=1.0, beta=0.0, type="f16", out_type="f32", variant=0, k_splits=0,
                 kernel=_lib.variant_name(0), time_ms=0.3, TFlops=1.0, correct=True),
            dict(m=4096, n=4096, k=4096, transA=0, transB=0, alpha=1.0, beta=0.0, type="f16", out_type="f32", variant=5, k_splits=0,
                 kernel=_lib.variant_name(5), time_ms=0.1, TFlops=1.0, correct=False),          # failed its check: never recorded
            dict(m=1000, n=1000, k=1000, transA=0, transB=0, alpha=1.0, beta=0.0, type="f16", out_type="f32", variant=1, k_splits=0,
                 kernel=_lib.variant_name(1), time_ms=0.1, TFlops=1.0, correct=True),           # kernel cannot take this shape
            dict(m=512, n=512, k=512, transA=0, transB=0, alpha=1.0, beta=0.0, type="f16", out_type="f32", variant=1, k_splits=0,
                 kernel="a kernel this library does not have", time_ms=0.1, TFlops=1.0, correct=True),
            dict(m=4096, n=4096, k=4096, transA=0, transB=0, alpha=1.0, beta=0.0, type="f16", out_type="f32", variant=-2, k_splits=0,
                 kernel="vendor library (torch.matmul)", time_ms=0.05, TFlops=1.0, correct="")]
    assert tuned.save(rows, str(path)) == 3
    tuned.reset()
    args = (_lib.F16, _lib.F32, 4096, 4096, 4096, (4096, 1), (4096, 1), (4096, 1))
    assert tuned.lookup(*args, True) == (1, 0)                 # fastest verified row
    assert tuned.lookup(*args, False) is None                  # other op class: not recorded
    assert tuned.lookup(*args, "acc") is None and tuned.lookup(*args, "lean") == (1, 0)
    assert tuned.ops_class(_lib.PROLOGUE_SET0, 0.0, _lib.EPILOGUE_RELU) == "lean"
    assert tuned.ops_class(_lib.PROLOGUE_NONE, 0.0, _lib.EPILOGUE_NONE) == "acc"
    assert tuned.ops_class(_lib.PROLOGUE_SET, 1.0, _lib.EPILOGUE_RELU) == "full"
    assert tuned.ops_class(_lib.PROLOGUE_NONE, 0.0, _lib.EPILOGUE_SCALE) == "full"
    assert tuned.lookup(_lib.F16, _lib.F32, 1000, 1000, 1000, (1000, 1), (1000, 1), (1000, 1), True) is None
    assert tuned.lookup(_lib.F16, _lib.F32, 512, 512, 512, (512, 1), (512, 1), (512, 1), True) is None
    assert tuned.lookup(_lib.F16, _lib.F32, 4096, 4096, 4096, (4096, 1), (4096, 1), (4100, 1), True) is None  # padded C: not a table shape
    tuned.reset()
