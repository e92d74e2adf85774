"""HAT package boundary: the DSL slice records the README quick start, Package.build emits a
.hat that is valid TOML *and* a valid C header, and the hatlib-style loader validates
arguments.  The GPU-marked tests call the package functions on NumPy arrays."""
import os
import subprocess

import numpy as np
import pytest

import accera_amd as acc
import oracle as ora
from accera_amd import hat


def _quickstart_package(tmp, M=512, N=512, K=512):
    """README.md:52-92, with `import accera_amd as acc`."""
    A = acc.Array(role=acc.Role.INPUT, shape=(M, K))
    B = acc.Array(role=acc.Role.INPUT, shape=(K, N))
    C = acc.Array(role=acc.Role.INPUT_OUTPUT, shape=(M, N))
    matmul = acc.Nest(shape=(M, N, K))
    i1, j1, k1 = matmul.get_indices()

    @matmul.iteration_logic
    def _():
        C[i1, j1] += A[i1, k1] * B[k1, j1]

    relu = acc.Nest(shape=(M, N))
    i2, j2 = relu.get_indices()

    @relu.iteration_logic
    def _():
        C[i2, j2] = acc.max(C[i2, j2], 0.0)

    package = acc.Package()
    schedule = acc.fuse(matmul.create_schedule(), relu.create_schedule(), partial=2)
    package.add(schedule, args=(A, B, C), base_name="matmul_relu_fusion_naive")
    i, j, f, k = schedule.get_indices()
    ii, jj = schedule.tile({i: 16, j: 16})
    schedule.reorder(j, i, f, k, jj, ii)
    plan = schedule.create_plan()
    plan.unroll(ii)
    package.add(plan, args=(A, B, C), base_name="matmul_relu_fusion_transformed")
    files = package.build(name="hello_accera", format=acc.Package.Format.HAT_DYNAMIC, output_dir=str(tmp))
    return files


def _native_shape(in_t, wide=False):
    """An instruction shape of the target for this input type: the 16x16 family (the 32x32 one with `wide`)."""
    S = acc.MMAShape
    if in_t == acc.ScalarType.float32:
        return S.M32xN32xK2_B1
    if in_t == acc.ScalarType.int8:
        return S.M32xN32xK32_B1 if wide else S.M16xN16xK64_B1
    return S.M32xN32xK16_B1 if wide else S.M16xN16xK32_B1


def _gpu_plan_package(tmp, in_t, out_t, M, N, K, b_layout=None, epilogue=None, base_name="matmul_relu", mma_shape=None, which="gpu",
                      **build_args):
    """mfma_tests.py:359-432 (`_matmul_relu`): tensorized plan with SET prologue and ReLU epilogue.  Returns
    ((hat, so), name): the .hat with the GPU-target records (`<name>_gpu.hat` of a default build), or with which="host"
    the plain host-convention `<name>.hat`."""
    target = acc.Target(acc.Target.Model.AMD_MI355X)
    A = acc.Array(role=acc.Role.INPUT, element_type=in_t, shape=(M, K))
    B = acc.Array(role=acc.Role.INPUT, element_type=in_t, shape=(K, N), layout=b_layout or acc.Array.Layout.FIRST_MAJOR)
    C = acc.Array(role=acc.Role.INPUT_OUTPUT, element_type=out_t, shape=(M, N))
    nest = acc.Nest(shape=(M, N, K))
    i, j, k = nest.get_indices()

    @nest.iteration_logic
    def _():
        C[i, j] += A[i, k] * B[k, j]

    schedule = nest.create_schedule()
    ii, jj, kk = schedule.tile({i: 16, j: 16, k: 16})
    schedule.reorder(i, j, k, ii, jj, kk)
    plan = schedule.create_plan(target)
    plan.bind({i: target.GridUnit.BLOCK_Y, j: target.GridUnit.BLOCK_X, ii: target.GridUnit.WARP_Y, jj: target.GridUnit.WARP_X})
    plan.tensorize(indices=(ii, jj, kk), mma_shape=mma_shape or _native_shape(in_t), prologue_op=acc.MMAFragmentOp.SET,
                   prologue_arg=0, epilogue_op=epilogue or acc.MMAFragmentOp.ReLU)
    plan.cache(A, index=ii, double_buffer=True, location=target.MemorySpace.SHARED)
    plan.cache(C, index=ii, location=target.MemorySpace.MMA_FRAGMENT)
    package = acc.Package()
    name = package.add(plan, args=(A, B, C), base_name=base_name)
    files = package.build(name="gpu_pkg", output_dir=str(tmp), **build_args)
    hat_path = files[2] if which == "gpu" and len(files) > 2 else files[0]
    return (hat_path, files[1]), name


def test_quickstart_builds_a_valid_hat(tmp_path):
    hat_path, so_path = _quickstart_package(tmp_path)
    assert os.path.exists(hat_path) and os.path.exists(so_path)
    doc = hat.parse(hat_path)
    fns = doc["functions"]
    assert len(fns) == 2
    for name, rec in fns.items():
        assert rec["name"] == name and rec["calling_convention"] == "cdecl"
        assert name.rsplit("_", 1)[0] in ("matmul_relu_fusion_naive", "matmul_relu_fusion_transformed")
        assert len(name.rsplit("_", 1)[1]) == 16
        usages = [a["usage"] for a in rec["arguments"]]
        assert usages == ["input", "input", "input_output"]
        for a in rec["arguments"]:
            # docs/Tutorials/Optimized_MatMul.md:176-187: row-major 2-D float arrays
            assert a["logical_type"] == "affine_array" and a["declared_type"] == "float*" and a["element_type"] == "float"
            assert a["shape"] == [512, 512] and a["affine_map"] == [512, 1] and a["affine_offset"] == 0
        assert rec["return"]["declared_type"] == "void"
        aux = rec["auxiliary"]["accera_mi355x"]
        assert len(aux["launch_parameters"]) == 6 and aux["epilogue"] == acc.EPILOGUE_RELU and aux["prologue"] == acc.PROLOGUE_NONE
        assert "launches" not in rec and "runtime" not in rec      # HOST-target plans: a host-convention function
    assert "device_functions" not in doc
    assert doc["dependencies"]["link_target"] == "hello_accera.so"
    assert doc["target"]["required"]["GPU"]["instruction_set_version"] == "gfx950"
    assert "void (*matmul_relu_fusion_naive)(float*, float*, float*)" in doc["declaration"]["code"]


def test_hat_is_a_valid_c_header_and_links(tmp_path):
    """Second class of callers: C programs that include the .hat and call the alias
    (docs/Tutorials/Hello_MatMul.md:165-237).  Compile and link only; running needs a GPU."""
    hat_path, so_path = _quickstart_package(tmp_path)
    main_c = tmp_path / "main.c"
    main_c.write_text('#include "hello_accera.hat"\n'
                      "static float A[512*512], B[512*512], C[512*512];\n"
                      "int main(int argc, char** argv) { if (argc > 1) matmul_relu_fusion_transformed(A, B, C); return 0; }\n")
    exe = tmp_path / "main"
    subprocess.check_call(["gcc", "-o", str(exe), str(main_c), f"-I{tmp_path}", str(so_path),
                           f"-Wl,-rpath,{tmp_path}"])
    subprocess.check_call([str(exe)])  # argc == 1: loads every library, calls nothing
    subprocess.check_call(["g++", "-fsyntax-only", "-x", "c++", str(main_c), f"-I{tmp_path}"])


def test_column_major_and_types_are_recorded(tmp_path):
    (hat_path, _), name = _gpu_plan_package(tmp_path, acc.ScalarType.bfloat16, acc.ScalarType.bfloat16, 4096, 3072, 768,
                                            b_layout=acc.Array.Layout.LAST_MAJOR)
    rec = hat.parse(hat_path)["functions"][name]
    a, b, c = rec["arguments"]
    assert a["element_type"] == "bfloat16_t" and a["declared_type"] == "bfloat16_t*"
    assert b["shape"] == [768, 3072] and b["affine_map"] == [1, 768]     # column-major B
    assert c["affine_map"] == [3072, 1]
    aux = rec["auxiliary"]["accera_mi355x"]
    assert "B=col-major" in aux["kernel"] and aux["prologue"] == acc.PROLOGUE_SET0 and aux["epilogue"] == acc.EPILOGUE_RELU
    assert aux["dynamic_shared_mem_bytes"] > 0 and aux["device_entry"] == name + "__device"


def test_block_tile_of_a_gpu_plan_selects_the_kernel(tmp_path):
    """The outermost splits of i and j of a GPU plan are its block tile (mfma_tests.py:89-97 tiles, binds the
    outer indices to BLOCK_Y / BLOCK_X); a tile the library has a kernel for binds the package function to it."""
    M = N = K = 1024
    A = acc.Array(role=acc.Role.INPUT, element_type=acc.ScalarType.float16, shape=(M, K))
    B = acc.Array(role=acc.Role.INPUT, element_type=acc.ScalarType.float16, shape=(K, N))
    C = acc.Array(role=acc.Role.INPUT_OUTPUT, element_type=acc.ScalarType.float32, shape=(M, N))

    def plan_with(tile):
        nest = acc.Nest(shape=(M, N, K))
        i, j, k = nest.get_indices()

        @nest.iteration_logic
        def _():
            C[i, j] += A[i, k] * B[k, j]

        schedule = nest.create_schedule()
        target = acc.Target(acc.Target.Model.AMD_MI355X)
        ii, jj, kk = schedule.tile({i: tile[0], j: tile[1], k: 64})
        schedule.reorder(i, j, k, ii, jj, kk)
        plan = schedule.create_plan(target)
        plan.bind({i: target.GridUnit.BLOCK_Y, j: target.GridUnit.BLOCK_X})
        plan.tensorize(indices=(ii, jj, kk), mma_shape=acc.MMAShape.M16xN16xK32_B1 if tile[0] == 256 else acc.MMAShape.M32xN32xK16_B1,
                       prologue_op=acc.MMAFragmentOp.SET, prologue_arg=0, epilogue_op=acc.MMAFragmentOp.ReLU)
        return plan

    package = acc.Package()
    n256 = package.add(plan_with((256, 256)), args=(A, B, C), base_name="tile256")
    n128 = package.add(plan_with((128, 128)), args=(A, B, C), base_name="tile128")
    n64 = package.add(plan_with((64, 64)), args=(A, B, C), base_name="tile64")    # (the reference's MFMA tests tile 64 x 64: mfma_tests.py:89-97)
    n48 = package.add(plan_with((48, 80)), args=(A, B, C), base_name="tile_other")   # no such kernel: automatic choice
    files = package.build(name="tiles", format=acc.Package.Format.HAT_DYNAMIC, output_dir=str(tmp_path))
    fns = hat.parse(files[0])["functions"]
    rec = lambda n: fns[n]["auxiliary"]["accera_mi355x"]
    assert "mfma 256x256" in rec(n256)["kernel"] and rec(n256)["launch_parameters"][:3] == [16, 1, 1]
    assert "mfma 128x128" in rec(n128)["kernel"] and rec(n128)["launch_parameters"][:3] == [64, 1, 1]
    assert "mfma 64x64" in rec(n64)["kernel"] and rec(n64)["launch_parameters"][:3] == [256, 1, 1]
    assert "mfma" in rec(n48)["kernel"]


def test_gpu_target_functions_carry_the_reference_device_records(tmp_path):
    """Package.py:714-743: `runtime` / `launches` on the function, and a [device_functions.<fn>__gpu__] record with the
    launch geometry, the dynamic LDS size and the provider."""
    from accera_amd import _lib
    (hat_path, so_path), name = _gpu_plan_package(tmp_path, acc.ScalarType.float16, acc.ScalarType.float32, 4096, 4096, 4096)
    doc = hat.parse(hat_path)
    fn = doc["functions"][name]
    assert fn["runtime"] == "ROCM" and fn["launches"] == name + "__gpu__" and fn["calling_convention"] == "cdecl"
    dev = doc["device_functions"][name + "__gpu__"]
    assert dev["name"] == name + "__gpu__" and dev["calling_convention"] == "device" and dev["runtime"] == "ROCM"
    assert dev["description"] == f"Device function launched by {name}"
    assert dev["arguments"] == fn["arguments"] and dev["return"] == fn["return"]
    grid, block, lds, variant = _lib.launch_geometry(_lib.F16, _lib.F32, 4096, 4096, 4096, (4096, 1), (4096, 1), (4096, 1))
    assert dev["launch_parameters"] == grid + block == fn["auxiliary"]["accera_mi355x"]["launch_parameters"]
    assert dev["dynamic_shared_mem_bytes"] == lds > 0 and dev["provider"] == "libaccera_mi355x.so"
    assert dev["auxiliary"]["accera_mi355x"]["entry"] == name + "__device"
    assert doc["target"]["required"]["GPU"]["runtime"] == "ROCM" and doc["target"]["required"]["GPU"]["model"] == "AMD MI355X"
    # both symbols are in the package library
    import ctypes
    L = ctypes.CDLL(so_path)
    assert getattr(L, name) is not None and getattr(L, name + "__device") is not None
    # the loader pairs them
    _, functions = hat.load(hat_path)
    assert functions[name].launches == name + "__gpu__" and functions[name].device_record == dev
    # gpu_records=True: the same records in `<name>.hat` itself, and no sibling file
    target = acc.Target(acc.Target.Model.AMD_MI355X)
    (hat3, so3), name3 = _gpu_plan_package(tmp_path / "inline", acc.ScalarType.float16, acc.ScalarType.float32, 4096, 4096, 4096,
                                           gpu_records=True)
    assert os.path.basename(hat3) == "gpu_pkg.hat" and not os.path.exists(os.path.join(os.path.dirname(hat3), "gpu_pkg_gpu.hat"))
    doc3 = hat.parse(hat3)
    assert name3 == name and doc3["device_functions"][name + "__gpu__"] == dev and doc3["functions"][name]["launches"] == name + "__gpu__"


def test_default_package_is_host_convention_with_nothing_for_a_run_time_compiler(tmp_path):
    """What a stock loader does with a function that `launches` something is compile its `provider`
    (Package.py:714-743); the kernels here are prebuilt, so `<name>.hat` of a default build carries no such record:
    every function is a plain cdecl symbol on host pointers, and the GPU-target records sit in `<name>_gpu.hat`."""
    import ctypes
    (host_hat, so_path), name = _gpu_plan_package(tmp_path, acc.ScalarType.float16, acc.ScalarType.float32, 1024, 1024, 1024, which="host")
    assert os.path.basename(host_hat) == "gpu_pkg.hat"
    text = open(host_hat).read()
    assert "device_functions" not in text and "launches" not in text and "provider" not in text
    doc = hat.parse(host_hat)
    fn = doc["functions"][name]
    assert fn["calling_convention"] == "cdecl" and "runtime" not in fn
    assert doc["dependencies"]["link_target"] == "gpu_pkg.so"
    # the launch geometry is still on record, as auxiliary data a stock loader ignores
    assert fn["auxiliary"]["accera_mi355x"]["device_entry"] == name + "__device"
    # the sibling with the GPU records names the same library and the same function
    gpu_hat = os.path.join(os.path.dirname(host_hat), "gpu_pkg_gpu.hat")
    gdoc = hat.parse(gpu_hat)
    assert gdoc["dependencies"]["link_target"] == "gpu_pkg.so" and gdoc["functions"][name]["launches"] == name + "__gpu__"
    assert gdoc["functions"][name]["arguments"] == fn["arguments"]
    assert getattr(ctypes.CDLL(so_path), name) is not None
    # the loader gives a host-pointer callable for the default file and pairs the device entry for the sibling
    _, host_functions = hat.load(host_hat)
    _, gpu_functions = hat.load(gpu_hat)
    assert host_functions[name].device_record is None and gpu_functions[name].device_record is not None
    # a package of HOST-target plans only has no sibling
    files = _quickstart_package(tmp_path / "host_only")
    assert len(files) == 2


def test_tensor_core_table_and_mma_shape_validation(tmp_path):
    """Targets.py:756-793 (the table and its queries) and the checks of Plan.tensorize (lang/Plan.py:242-361)."""
    T, S = acc.ScalarType, acc.MMAShape
    target = acc.Target(acc.Target.Model.AMD_MI355X)
    info = target.tensor_core_info
    assert info.supports(T.float16, T.float32, S.M16xN16xK32_B1, 1, -1) and info.supports(T.bfloat16, T.bfloat16, S.M32xN32xK16_B1, 2, 1)
    assert info.supports(T.int8, T.int32, S.M16xN16xK64_B1) and info.supports(T.int8, T.int8, S.M32xN32xK32_B1)
    assert info.supports(T.float32, T.float32, S.M32xN32xK2_B1)
    assert not info.supports(T.float16, T.float32, S.M16xN16xK16_B1)          # an MI100 shape gfx950 kernels do not use
    assert not info.supports(T.int8, T.int32, S.M16xN16xK32_B1)               # a 16-bit shape with 8-bit inputs
    assert not info.supports(T.float16, T.float32, S.M16xN16xK32_B1, 4, 3)    # passes must divide
    assert info.mma_shape_to_tuple(S.M16xN16xK64_B1) == (16, 16, 64) and info.compute_tensor_splits(S.M32xN32xK16_B1, 4) == (32, 32, 64)

    def plan_for(in_t, out_t, tgt=target):
        A = acc.Array(role=acc.Role.INPUT, element_type=in_t, shape=(512, 512))
        B = acc.Array(role=acc.Role.INPUT, element_type=in_t, shape=(512, 512))
        C = acc.Array(role=acc.Role.INPUT_OUTPUT, element_type=out_t, shape=(512, 512))
        nest = acc.Nest(shape=(512, 512, 512))
        i, j, k = nest.get_indices()

        @nest.iteration_logic
        def _():
            C[i, j] += A[i, k] * B[k, j]

        return nest.create_schedule().create_plan(tgt), (i, j, k), (A, B, C)

    plan, idx, arrays = plan_for(T.float16, T.float32)
    with pytest.raises(ValueError, match="does not support the given tensorization dimensions"):
        plan.tensorize(indices=idx, mma_shape=S.M16xN16xK16_B1)
    with pytest.raises(ValueError, match="at least three"):
        plan.tensorize(indices=idx[:2], mma_shape=S.M16xN16xK32_B1)
    with pytest.raises(ValueError, match="fusing must be a positive"):
        plan.tensorize(indices=idx, mma_shape=S.M16xN16xK32_B1, num_fused_passes=0)
    host_plan, idx_h, _ = plan_for(T.float16, T.float32, acc.Target.HOST)
    with pytest.raises(ValueError, match="only supported on GPU"):
        host_plan.tensorize(indices=idx_h, mma_shape=S.M16xN16xK32_B1)
    # a shape of the target, but not for these types: caught when the function is added
    plan8, idx8, arrays8 = plan_for(T.int8, T.int32)
    plan8.tensorize(indices=idx8, mma_shape=S.M16xN16xK32_B1)
    with pytest.raises(ValueError, match="does not support"):
        acc.Package().add(plan8, args=arrays8, base_name="bad_shape")
    # the shape selects the kernel family
    package = acc.Package()
    names = {}
    for tag, shape in (("small", S.M16xN16xK32_B1), ("wide", S.M32xN32xK16_B1)):
        p, ix, arr = plan_for(T.float16, T.float32)
        p.tensorize(indices=ix, mma_shape=shape, prologue_op=acc.MMAFragmentOp.SET, epilogue_op=acc.MMAFragmentOp.ReLU)
        names[tag] = package.add(p, args=arr, base_name=tag)
    files = package.build(name="shapes", output_dir=str(tmp_path))
    fns = hat.parse(files[0])["functions"]
    assert " mi16" in fns[names["small"]]["auxiliary"]["accera_mi355x"]["kernel"]
    assert " mi16" not in fns[names["wide"]]["auxiliary"]["accera_mi355x"]["kernel"] and "mfma" in fns[names["wide"]]["auxiliary"]["accera_mi355x"]["kernel"]


def test_only_the_matmul_pattern_is_accepted():
    A = acc.Array(role=acc.Role.INPUT, shape=(8, 8))
    B = acc.Array(role=acc.Role.INPUT, shape=(8, 8))
    C = acc.Array(role=acc.Role.INPUT_OUTPUT, shape=(8, 8))
    nest = acc.Nest(shape=(8, 8, 8))
    i, j, k = nest.get_indices()

    @nest.iteration_logic
    def _():
        C[i, j] += A[i, k] + B[k, j]  # not a product

    with pytest.raises(NotImplementedError):
        acc.Package().add(nest, args=(A, B, C), base_name="bad")
    nest2 = acc.Nest(shape=(8, 8, 8))
    i, j, k = nest2.get_indices()

    @nest2.iteration_logic
    def _():
        C[i, j] += A[i, k] * B[j, k]  # B indexed (j, k): not B[k, j]

    with pytest.raises(NotImplementedError):
        acc.Package().add(nest2, args=(A, B, C), base_name="bad")


def test_loader_validates_arguments_before_calling(tmp_path):
    hat_path, _ = _quickstart_package(tmp_path, 64, 64, 64)
    pkg, functions = hat.load(hat_path)
    assert set(n.rsplit("_", 1)[0] for n in functions.names if n[-1].isdigit() or True) >= {"matmul_relu_fusion_naive"}
    f = functions["matmul_relu_fusion_transformed"]     # alias -> first function with that base name
    assert f is functions[f.name] and f.name.startswith("matmul_relu_fusion_transformed_")
    A = np.zeros((64, 64), np.float32)
    with pytest.raises(ValueError, match="expected 3 arguments"):
        f(A, A)
    with pytest.raises(ValueError, match="dtype"):
        f(A.astype(np.float64), A, A)
    with pytest.raises(ValueError, match="shape"):
        f(np.zeros((64, 32), np.float32), A, A)
    with pytest.raises(ValueError, match="strides"):
        f(np.asfortranarray(np.ones((64, 64), np.float32)), A, A)
    with pytest.raises(TypeError):
        f([1, 2], A, A)


# ---------------------------------------------------------------------------------------------
@pytest.mark.gpu
def test_readme_quickstart_end_to_end(tmp_path):
    """README.md:118-136, verbatim apart from the import."""
    hat_path, _ = _quickstart_package(tmp_path)
    _, functions = hat.load(hat_path)
    rng = np.random.default_rng(1001)
    A_test = rng.random((512, 512)).astype(np.float32)
    B_test = rng.random((512, 512)).astype(np.float32)
    for base in ("matmul_relu_fusion_transformed", "matmul_relu_fusion_naive"):
        C_test = np.zeros((512, 512)).astype(np.float32)
        C_numpy = np.maximum(C_test + A_test @ B_test, 0.0)
        functions[base](A_test, B_test, C_test)
        np.testing.assert_allclose(C_test, C_numpy, atol=1e-3)
    # the function accumulates into C (no SET prologue): signed data, non-zero C
    A_s, B_s = (A_test - 0.5), (B_test - 0.5)
    C0 = rng.standard_normal((512, 512)).astype(np.float32)
    C_test = C0.copy()
    functions["matmul_relu_fusion_naive"](A_s, B_s, C_test)
    want = ora.gemm_relu_exact(A_s, B_s, C0, "f32", "f32", ora.PRO_NONE, ora.EPI_RELU)
    np.testing.assert_allclose(C_test, want, atol=1e-3)
    assert (C_test == 0).any() and (C_test > 0).any()


@pytest.mark.gpu
def test_package_functions_called_from_two_host_threads_at_once(tmp_path):
    """A package function takes host arrays (README.md:124-130) and may be called from any thread.  Each call in flight has
    its own device buffers, staging buffers and stream, so calls from two threads overlap; both must be right, call after
    call, on operands large enough for several staging pieces and on an accumulating (C is read) problem."""
    import threading
    (hat_a, _), name_a = _gpu_plan_package(tmp_path / "a", acc.ScalarType.float16, acc.ScalarType.float32, 1024, 2048, 3072, which="host")
    (hat_b, _), name_b = _gpu_plan_package(tmp_path / "b", acc.ScalarType.int8, acc.ScalarType.int32, 2048, 1024, 4096, which="host",
                                           mma_shape=acc.MMAShape.M16xN16xK64_B1)
    fa, fb = hat.load(hat_a)[1][name_a], hat.load(hat_b)[1][name_b]
    rng = np.random.default_rng(5)
    from tests.util import assert_matches, make_input
    Aa, Ba = make_input(rng, (1024, 3072), "f16"), make_input(rng, (3072, 2048), "f16")
    Ab, Bb = make_input(rng, (2048, 4096), "i8"), make_input(rng, (4096, 1024), "i8")
    want_a = ora.gemm_relu_exact(Aa, Ba, None, "f16", "f32")
    want_b = ora.gemm_relu_exact(Ab, Bb, None, "i8", "i32")
    errors = []

    def worker(f, A, B, want, out_t, K, reps):
        try:
            for _ in range(reps):
                C = np.full(want.shape, 3, want.dtype)
                f(A, B, C)
                assert_matches(C, want, out_t, K)
        except BaseException as e:  # (reported by the main thread)
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(fa, Aa, Ba, want_a, "f32", 3072, 6)),
               threading.Thread(target=worker, args=(fb, Ab, Bb, want_b, "i32", 4096, 6))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[0]
    # the two contexts the calls used can be handed back; the next call on host arrays makes its own again
    from accera_amd import _lib
    before = _lib.allocation_probe()
    _lib.release_workspaces()
    worker(fa, Aa, Ba, want_a, "f32", 3072, 1)
    assert not errors, errors[0]
    assert _lib.allocation_probe() >= before + 3  # device copies of A, B and C


@pytest.mark.gpu
@pytest.mark.parametrize("in_t,out_t,shape,b_layout", [
    (acc.ScalarType.float16, acc.ScalarType.float32, (256, 384, 512), None),
    (acc.ScalarType.bfloat16, acc.ScalarType.bfloat16, (256, 256, 192), acc.Array.Layout.LAST_MAJOR),
    (acc.ScalarType.int8, acc.ScalarType.int32, (256, 256, 256), None),
    (acc.ScalarType.int8, acc.ScalarType.int16, (256, 128, 128), None),       # mfma_tests.py:2141 sizes
    (acc.ScalarType.int8, acc.ScalarType.int8, (128, 256, 512), acc.Array.Layout.LAST_MAJOR),  # mfma_tests.py:2123 sizes
    (acc.ScalarType.float16, acc.ScalarType.float16, (8, 1024, 512), None),
    (acc.ScalarType.float32, acc.ScalarType.float32, (16, 16, 16), None),     # mfma_tests.py:2579-2602 sizes
    (acc.ScalarType.float32, acc.ScalarType.float32, (128, 128, 16), None),
])
def test_tensorized_plan_package_on_numpy_arrays(tmp_path, in_t, out_t, shape, b_layout):
    M, N, K = shape
    (hat_path, _), name = _gpu_plan_package(tmp_path, in_t, out_t, M, N, K, b_layout)
    _, functions = hat.load(hat_path)
    tn = {acc.ScalarType.float16: "f16", acc.ScalarType.bfloat16: "bf16", acc.ScalarType.int8: "i8",
          acc.ScalarType.float32: "f32", acc.ScalarType.int32: "i32", acc.ScalarType.int16: "i16"}
    it, ot = tn[in_t], tn[out_t]
    from tests.util import assert_matches, make_input
    rng = np.random.default_rng(5)
    A, B = make_input(rng, (M, K), it), make_input(rng, (K, N), it)
    if b_layout is not None:
        B = np.asfortranarray(B)
    C = np.full((M, N), 3, ora.NP_STORAGE[ot])   # SET prologue: the old content must not matter
    functions[name](A, B, C)
    assert_matches(C, ora.gemm_relu_exact(A, B, None, it, ot), ot, K)


def _batched_package(tmp, batch, M, N, K, in_t=acc.ScalarType.float16, out_t=acc.ScalarType.float32, alpha=None):
    """The reference's batch matmul nest (mfma_tests.py:435-470) fused with ReLU, or with an alpha epilogue."""
    A = acc.Array(role=acc.Role.INPUT, element_type=in_t, shape=(batch, M, K))
    B = acc.Array(role=acc.Role.INPUT, element_type=in_t, shape=(batch, K, N))
    C = acc.Array(role=acc.Role.INPUT_OUTPUT, element_type=out_t, shape=(batch, M, N))
    nest = acc.Nest(shape=(batch, M, N, K))
    b, i, j, k = nest.get_indices()

    @nest.iteration_logic
    def _():
        C[b, i, j] += A[b, i, k] * B[b, k, j]

    target = acc.Target(acc.Target.Model.AMD_MI355X)
    if alpha is None:
        relu = acc.Nest(shape=(batch, M, N))
        b2, i2, j2 = relu.get_indices()

        @relu.iteration_logic
        def _():
            C[b2, i2, j2] = acc.max(C[b2, i2, j2], 0.0)

        plan = acc.fuse(nest.create_schedule(), relu.create_schedule(), partial=3).create_plan(target)
        plan.tensorize(indices=plan.schedule.get_indices()[1:4], mma_shape=acc.MMAShape.M32xN32xK16_B1,
                       prologue_op=acc.MMAFragmentOp.SET, prologue_arg=0)
    else:
        plan = nest.create_schedule().create_plan(target)
        plan.tensorize(indices=(i, j, k), mma_shape=acc.MMAShape.M32xN32xK16_B1, prologue_op=acc.MMAFragmentOp.SCALE, prologue_arg=0.5,
                       epilogue_op=acc.MMAFragmentOp.SCALE, epilogue_arg=alpha)
    package = acc.Package()
    name = package.add(plan, args=(A, B, C), base_name="batch_matmul")
    return package.build(name="batch_pkg", format=acc.Package.Format.HAT_DYNAMIC, output_dir=str(tmp)), name


def test_batched_nest_is_recorded_with_three_dimensional_arguments(tmp_path):
    files, name = _batched_package(tmp_path, 3, 128, 256, 64)
    pkg = hat.parse(files[0])
    fn = pkg["functions"][name]
    assert [a["shape"] for a in fn["arguments"]] == [[3, 128, 64], [3, 64, 256], [3, 128, 256]]
    assert [a["affine_map"] for a in fn["arguments"]] == [[8192, 64, 1], [16384, 256, 1], [32768, 256, 1]]
    assert fn["auxiliary"]["accera_mi355x"]["launch_parameters"][2] == 3  # batch index on grid.z


@pytest.mark.gpu
@pytest.mark.parametrize("alpha", [None, 2.0])
def test_batched_package_on_numpy_arrays(tmp_path, alpha):
    batch, M, N, K = 3, 256, 384, 128
    files, name = _batched_package(tmp_path, batch, M, N, K, alpha=alpha)
    _, functions = hat.load(files[0])
    from tests.util import assert_matches, make_input
    rng = np.random.default_rng(9)
    A = np.stack([make_input(rng, (M, K), "f16") for _ in range(batch)])
    B = np.stack([make_input(rng, (K, N), "f16") for _ in range(batch)])
    C0 = rng.standard_normal((batch, M, N)).astype(np.float32)
    C = C0.copy()
    functions[name](A, B, C)
    for b in range(batch):
        want = (ora.gemm_relu_exact(A[b], B[b], None, "f16", "f32") if alpha is None else
                ora.gemm_relu_exact(A[b], B[b], C0[b], "f16", "f32", ora.PRO_SCALE, ora.EPI_SCALE, prologue_arg=0.5, epilogue_arg=alpha))
        assert_matches(C[b], want, "f32", K)


@pytest.mark.gpu
def test_run_benchmark_reports_hatlib_style_rows(tmp_path):
    hat_path, _ = _quickstart_package(tmp_path, 256, 256, 256)
    results = hat.run_benchmark(hat_path, batch_size=5, min_time_in_sec=0.2, input_sets_minimum_size_MB=2)
    assert len(results) == 2
    for r in results:
        assert r.function_name.startswith("matmul_relu_fusion_")
        assert 0 < r.min_of_means <= r.median_of_means and r.min_of_means <= r.mean
        assert r.mean_of_small_means <= r.mean and r.robust_mean > 0


@pytest.mark.gpu
@pytest.mark.parametrize("in_t,out_t,shape,wide", [
    (acc.ScalarType.float16, acc.ScalarType.float32, (512, 512, 256), False),
    (acc.ScalarType.int8, acc.ScalarType.int32, (256, 512, 512), True),
    (acc.ScalarType.float16, acc.ScalarType.float16, (8, 2048, 1024), False),
])
def test_device_function_of_a_package_on_device_pointers(tmp_path, in_t, out_t, shape, wide):
    """What the [device_functions.<fn>__gpu__] record stands for: `<fn>__device(A, B, C, stream)` of the package library
    on DEVICE pointers, asynchronous on a stream, checked against the oracle; and the loader's `device_id=` form of the
    call (copies on this side of the boundary), hatlib's calling form for GPU packages (accera_gemm.py:612-615)."""
    import ctypes
    import torch
    from tests.util import assert_matches, make_input, to_device, to_host
    M, N, K = shape
    (hat_path, so_path), name = _gpu_plan_package(tmp_path, in_t, out_t, M, N, K, mma_shape=_native_shape(in_t, wide))
    tn = {acc.ScalarType.float16: "f16", acc.ScalarType.int8: "i8", acc.ScalarType.float32: "f32", acc.ScalarType.int32: "i32"}
    it, ot = tn[in_t], tn[out_t]
    rng = np.random.default_rng(11)
    A, B = make_input(rng, (M, K), it), make_input(rng, (K, N), it)
    want = ora.gemm_relu_exact(A, B, None, it, ot)
    dA, dB = to_device(A, it), to_device(B, it)
    dC = to_device(np.full((M, N), 5, ora.NP_STORAGE[ot]), ot)
    L = ctypes.CDLL(so_path)
    entry = getattr(L, name + "__device")
    entry.restype, entry.argtypes = ctypes.c_int, [ctypes.c_void_p] * 4
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        assert entry(dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), stream.cuda_stream) == 0
    stream.synchronize()
    assert_matches(to_host(dC, ot), want, ot, K)
    # through the loader
    _, functions = hat.load(hat_path)
    f = functions[name]
    assert f.device_record["launch_parameters"][3] % 64 == 0
    C = np.full((M, N), 3, ora.NP_STORAGE[ot])
    f(A, B, C, device_id=0)
    assert_matches(C, want, ot, K)
    dC.fill_(1)
    f.launch_on_device([dA.data_ptr(), dB.data_ptr(), dC.data_ptr()])
    torch.cuda.synchronize()
    assert_matches(to_host(dC, ot), want, ot, K)


@pytest.mark.gpu
def test_run_benchmark_times_gpu_functions_device_resident(tmp_path):
    """accera_gemm.py:621-626, 648: `run_benchmark(..., device_id=)` of a GPU package gives kernel time (inputs resident
    in device memory, HIP events around each batch), far below the time of the host-pointer entry with its copies."""
    (hat_path, _), name = _gpu_plan_package(tmp_path, acc.ScalarType.float16, acc.ScalarType.float32, 2048, 2048, 2048)
    dev = hat.run_benchmark(hat_path, batch_size=10, min_time_in_sec=0.3, input_sets_minimum_size_MB=40, device_id=0)
    host = hat.run_benchmark(hat_path, batch_size=3, min_time_in_sec=0.3, input_sets_minimum_size_MB=40, device_id=0, host_pointers=True)
    assert len(dev) == len(host) == 1 and dev[0].function_name == name
    r = dev[0]
    assert 0 < r.min_of_means <= r.median_of_means and r.min_of_means <= r.mean
    tflops = 2 * 2048 ** 3 / r.min_of_means / 1e12
    assert 100 < tflops < 2500, tflops          # a kernel time, not a copy time (PCIe alone takes milliseconds here)
    assert host[0].min_of_means > 5 * r.min_of_means


def test_cache_and_bind_check_their_arguments_and_the_cached_k_depth_selects_the_kernel(tmp_path):
    """Plan.cache / Plan.bind of the reference (lang/Plan.py:381-703, 793-878): the same argument checks; and the split of
    k inside a SHARED cache of A or B -- the K depth of the staged block, the `k_split` axis of the reference's sweep
    (tools/benchmarkers/accera_gemm.py:281-293, 554-555) -- picks a kernel with K tiles of that many bytes."""
    T = acc.ScalarType
    target = acc.Target(acc.Target.Model.AMD_MI355X)
    SHARED, GLOBAL, FRAG = target.MemorySpace.SHARED, target.MemorySpace.GLOBAL, target.MemorySpace.MMA_FRAGMENT

    def plan_for(k_split, tgt=target, in_t=T.float16):
        A = acc.Array(role=acc.Role.INPUT, element_type=in_t, shape=(1024, 1024))
        B = acc.Array(role=acc.Role.INPUT, element_type=in_t, shape=(1024, 1024))
        C = acc.Array(role=acc.Role.INPUT_OUTPUT, element_type=T.float32 if in_t != T.int8 else T.int32, shape=(1024, 1024))
        nest = acc.Nest(shape=(1024, 1024, 1024))
        i, j, k = nest.get_indices()

        @nest.iteration_logic
        def _():
            C[i, j] += A[i, k] * B[k, j]

        schedule = nest.create_schedule()
        ii, jj, kk = schedule.tile({i: 256, j: 256, k: k_split})
        schedule.reorder(i, j, k, ii, jj, kk)
        return schedule.create_plan(tgt), (i, j, k, ii, jj, kk), (A, B, C)

    plan, (i, j, k, ii, jj, kk), (A, B, C) = plan_for(32)
    with pytest.raises(ValueError, match="one and only one of index, level, or max_elements"):
        plan.cache(A, location=SHARED)
    with pytest.raises(ValueError, match="one and only one of index, level, or max_elements"):
        plan.cache(A, index=ii, level=2, location=SHARED)
    with pytest.raises(ValueError, match="greater than 0"):
        plan.cache(A, max_elements=0)
    with pytest.raises(ValueError, match="only supported for CONST and INPUT"):
        plan.cache(C, index=ii, double_buffer=True, location=SHARED)
    with pytest.raises(ValueError, match="double_buffer_location is only valid"):
        plan.cache(A, index=ii, double_buffer_location=target.MemorySpace.PRIVATE)
    with pytest.raises(ValueError, match="Global memory caches are not yet supported on GPU"):
        plan.cache(A, index=ii, location=GLOBAL)
    with pytest.raises(ValueError, match="not supported with Tensor caching"):
        plan.cache(A, index=ii, double_buffer=True, location=FRAG)
    with pytest.raises(ValueError, match="cache index and a cache level or trigger level"):
        plan.cache(A, index=ii, trigger_level=4, location=SHARED)
    with pytest.raises(ValueError, match="at or outside"):
        plan.cache(A, index=ii, trigger_index=kk, location=SHARED)
    with pytest.raises(ValueError, match="Multicaching is only supported"):
        plan.cache(C, index=ii, trigger_index=i, location=SHARED)
    with pytest.raises(ValueError, match="not an index of this plan"):
        plan.cache(A, index=acc.Nest(shape=(4, 4, 4)).get_indices()[0], location=SHARED)
    host_plan, hidx, harr = plan_for(32, acc.Target.HOST)
    with pytest.raises(ValueError, match="Only AUTO strategy"):
        host_plan.cache(harr[0], index=hidx[3], strategy=acc.CacheStrategy.BLOCKED)
    with pytest.raises(ValueError, match="GPU targets"):
        host_plan.bind({hidx[0]: target.GridUnit.BLOCK_Y})
    with pytest.raises(ValueError, match="not an index"):
        plan.bind({acc.Nest(shape=(4, 4, 4)).get_indices()[0]: target.GridUnit.BLOCK_X})
    with pytest.raises(ValueError, match="not a grid unit"):
        plan.bind({i: "BLOCK_X"})
    # what the checks let through returns a handle with the reference's defaults resolved
    c = plan.cache(A, index=ii, double_buffer=True, location=SHARED)
    assert c.double_buffer and c.double_buffer_location == target.MemorySpace.PRIVATE and c.strategy == acc.CacheStrategy.STRIPED
    assert plan.cache(B, level=3, location=SHARED).index is ii                    # level 3 of (i, j, k, ii, jj, kk) is ii
    assert plan.cache(C, index=ii, location=FRAG).double_buffer_location == target.MemorySpace.NONE
    plan.bind({i: target.GridUnit.BLOCK_Y, j: target.GridUnit.BLOCK_X, (ii, jj): target.GridUnit.WARP_X})

    # ---- K depth of the cached block -> K tile of the kernel
    package = acc.Package()
    names = {}
    for tag, in_t, k_split, cached in (("f16_k32", T.float16, 32, True), ("f16_k64", T.float16, 64, True), ("i8_k128", T.int8, 128, True),
                                       ("f16_k64_uncached", T.float16, 64, False), ("f16_k16", T.float16, 16, True)):
        p, (i, j, k, ii, jj, kk), arr = plan_for(k_split, in_t=in_t)
        p.bind({i: target.GridUnit.BLOCK_Y, j: target.GridUnit.BLOCK_X})
        p.tensorize(indices=(ii, jj, kk), mma_shape=acc.MMAShape.M16xN16xK64_B1 if in_t == T.int8 else acc.MMAShape.M16xN16xK32_B1,
                    prologue_op=acc.MMAFragmentOp.SET, prologue_arg=0, epilogue_op=acc.MMAFragmentOp.ReLU)
        if cached:
            p.cache(arr[0], index=ii, double_buffer=True, location=SHARED)
            p.cache(arr[1], index=ii, double_buffer=True, location=SHARED)
        names[tag] = package.add(p, args=arr, base_name=tag)
    files = package.build(name="kdepth", format=acc.Package.Format.HAT_DYNAMIC, output_dir=str(tmp_path))
    fns = hat.parse(files[0])["functions"]
    kernel = lambda tag: fns[names[tag]]["auxiliary"]["accera_mi355x"]["kernel"]
    assert " kb64 " in kernel("f16_k32") and "mfma 256x256" in kernel("f16_k32")      # 32 fp16 = 64 bytes of K
    assert " kb128 " in kernel("f16_k64") and "mfma 256x256" in kernel("f16_k64") and "mi16" in kernel("f16_k64")
    assert " kb128 " in kernel("i8_k128")
    assert " kb64 " in kernel("f16_k64_uncached")      # no cache call: the library's choice for the tile
    assert " kb64 " in kernel("f16_k16")               # a depth no kernel has: the library's choice
