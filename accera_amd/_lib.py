"""ctypes binding of libaccera_mi355x.so (the C ABI declared in include/accera_mi355x_gemm.h) and of
libaccera_mi355x_probes.so (the measurement aids of include/accera_mi355x_probes.h, a library of its own that only the
benchmark and the tests of its aids load).

There is no CPU fallback: if the shared library is missing, loading raises with the
build command; if a call fails, the library's own error text is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libaccera_mi355x.so")
PROBES_LIB_PATH = os.path.join(LIB_DIR, "libaccera_mi355x_probes.so")
INCLUDE_DIR = os.path.join(os.path.dirname(_HERE), "include")

# element types / ops / status codes / variant ids (accera_mi355x_gemm.h)
F32, F16, BF16, I8, I32, I16 = 0, 1, 2, 3, 4, 5
PROLOGUE_NONE, PROLOGUE_SET0, PROLOGUE_SET, PROLOGUE_SCALE = 0, 1, 1, 2
EPILOGUE_NONE, EPILOGUE_RELU, EPILOGUE_RELU_NOCOND, EPILOGUE_SCALE, EPILOGUE_SET = 0, 1, 2, 3, 4
OK, INVALID_ARGUMENT, UNSUPPORTED, HIP_ERROR = 0, 1, 2, 3
VARIANT_AUTO, VARIANT_SKINNY_BASE, VARIANT_GENERIC, VARIANT_F32_MFMA = -1, 100, 200, 201

EXPORTS = [
    "acc950_init", "acc950_gemm_relu", "acc950_gemm_relu_ex", "acc950_gemm_relu_host", "acc950_gemm_ops", "acc950_gemm_ops_host", "acc950_gemm_ops_static",
    "acc950_gemm_batched", "acc950_gemm_batched_host", "acc950_bind", "acc950_launch", "acc950_unbind",
    "acc950_launch_geometry", "acc950_num_variants", "acc950_num_skinny_variants",
    "acc950_variant_name", "acc950_last_error",
    "acc950_bound_choice", "acc950_workspace_probe", "acc950_allocation_probe", "acc950_release_workspaces",
]
# measurement aids (include/accera_mi355x_probes.h, libaccera_mi355x_probes.so): not part of the product
PROBE_EXPORTS = ["acc950_mfma_ceiling", "acc950_mfma_traffic_probe", "acc950_mfma_phase_probe", "acc950_copy_probe", "acc950_stream_read_probe",
                 "acc950_probes_last_error"]


class Acc950Error(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"acc950 status {code}: {message}")
        self.code = code


_lib = None


def lib():
    """The loaded library (loads it on first use)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            f"(or `make -C accera_amd/csrc`). There is no CPU fallback.")
    L = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    ci, i64, vp, cu = ctypes.c_int, ctypes.c_int64, ctypes.c_void_p, ctypes.c_uint
    mat = [vp, i64, i64]
    L.acc950_init.argtypes = [ci]
    L.acc950_gemm_relu.argtypes = [ci, ci, ci, ci, ci] + mat * 3 + [ci, ci, vp]
    L.acc950_gemm_relu_ex.argtypes = [ci, ci, ci, ci, ci] + mat * 3 + [ci, ci, ci, ci, vp]
    L.acc950_gemm_relu_host.argtypes = [ci, ci, ci, ci, ci] + mat * 3 + [ci, ci]
    cd = ctypes.c_double
    L.acc950_gemm_ops.argtypes = [ci, ci, ci, ci, ci] + mat * 3 + [ci, cd, ci, cd, ci, ci, vp]
    L.acc950_gemm_ops_static.argtypes = L.acc950_gemm_ops.argtypes
    L.acc950_gemm_ops_host.argtypes = [ci, ci, ci, ci, ci] + mat * 3 + [ci, cd, ci, cd]
    bmat = [vp, i64, i64, i64]
    L.acc950_gemm_batched.argtypes = [ci, ci, ci, ci, ci, ci] + bmat * 3 + [ci, cd, ci, cd, ci, ci, vp]
    L.acc950_gemm_batched_host.argtypes = [ci, ci, ci, ci, ci, ci] + bmat * 3 + [ci, cd, ci, cd, ci, ci]
    L.acc950_bind.argtypes = [ci, ci, ci, ci, ci, ci] + bmat * 3 + [ci, cd, ci, cd, ci, ci, vp, ctypes.POINTER(ci)]
    L.acc950_launch.argtypes = [ci]
    L.acc950_unbind.argtypes = [ci]
    L.acc950_launch_geometry.argtypes = [ci, ci, ci, ci, ci] + [i64] * 6 + [ci, ci, ctypes.POINTER(cu), ctypes.POINTER(cu),
                                                                           ctypes.POINTER(cu), ctypes.POINTER(ci)]
    L.acc950_variant_name.argtypes = [ci, ctypes.c_char_p, ctypes.c_size_t]
    L.acc950_allocation_probe.argtypes = [ctypes.POINTER(ctypes.c_ulonglong)]
    L.acc950_workspace_probe.argtypes = [vp, ctypes.POINTER(vp), ctypes.POINTER(vp)]
    L.acc950_bound_choice.argtypes = [ci, ctypes.POINTER(ci), ctypes.POINTER(ci)]
    L.acc950_release_workspaces.argtypes = []
    L.acc950_last_error.restype = ctypes.c_char_p
    for name in EXPORTS:
        if name != "acc950_last_error":
            getattr(L, name).restype = ci
    _lib = L
    return L


_probes = None


def probes():
    """The measurement-aid library (loads it on first use): machine ceilings, copy / read probes, the in-kernel phase probe."""
    global _probes
    if _probes is not None:
        return _probes
    if not os.path.exists(PROBES_LIB_PATH):
        raise RuntimeError(f"{PROBES_LIB_PATH} is missing: build it with `make -C accera_amd/csrc`")
    L = ctypes.CDLL(PROBES_LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    ci, vp = ctypes.c_int, ctypes.c_void_p
    L.acc950_mfma_ceiling.argtypes = [ci, ci, ci, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    L.acc950_mfma_traffic_probe.argtypes = [ci, ci, ci, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    L.acc950_mfma_phase_probe.argtypes = [ci, ci, ci, ci, ci, vp, vp, vp, ctypes.POINTER(ctypes.c_double)]
    L.acc950_copy_probe.argtypes = [vp, vp, ctypes.c_size_t, vp]
    L.acc950_stream_read_probe.argtypes = [vp, ctypes.c_size_t, vp, vp]
    L.acc950_probes_last_error.restype = ctypes.c_char_p
    for name in PROBE_EXPORTS:
        if name != "acc950_probes_last_error":
            getattr(L, name).restype = ci
    _probes = L
    return L


def check(rc):
    if rc != OK:
        raise Acc950Error(rc, lib().acc950_last_error().decode())


def check_probe(rc):
    if rc != OK:
        raise Acc950Error(rc, probes().acc950_probes_last_error().decode() or "probe failed")


def mfma_phase_probe(in_type, out_type, M, N, K, a_ptr, b_ptr, c_ptr):
    """In-kernel phase times of the 256x256 kernel the automatic choice takes, on device operands; returns a dict."""
    out = (ctypes.c_double * 8)()
    check_probe(probes().acc950_mfma_phase_probe(in_type, out_type, M, N, K, a_ptr, b_ptr, c_ptr, out))
    return {"prologue_us": out[0] / 1e3, "main_loop_us": out[1] / 1e3, "write_back_us": out[2] / 1e3,
            "clock_ghz_prologue": out[3], "clock_ghz_main_loop": out[4], "clock_ghz_write_back": out[5],
            "kernel_span_us": out[6] / 1e3, "mfma_pipe_busy_main_loop": out[7]}


def mfma_ceiling(in_type, data_mode=2, iters=20000):
    """(tera-ops/s, sustained shader clock in GHz) of a pure MFMA loop on this GPU;
    data_mode 0 zeros, 1 constant, 2 random operands."""
    t, g = ctypes.c_double(), ctypes.c_double()
    check_probe(probes().acc950_mfma_ceiling(in_type, data_mode, iters, ctypes.byref(t), ctypes.byref(g)))
    return t.value, g.value


def mfma_traffic_probe(in_type, traffic, iters=2000):
    """(tera-ops/s, sustained shader clock in GHz) of the four-wave loop's MFMAs with its traffic added piece by piece:
    traffic 0 none, 1 its LDS reads, 2 also its direct-to-LDS fills from the caches, 3 the fills from a 1 GiB buffer."""
    t, g = ctypes.c_double(), ctypes.c_double()
    check_probe(probes().acc950_mfma_traffic_probe(in_type, traffic, iters, ctypes.byref(t), ctypes.byref(g)))
    return t.value, g.value


def allocation_probe():
    """Device allocations made by the GEMM entry points of this process so far."""
    n = ctypes.c_ulonglong()
    check(lib().acc950_allocation_probe(ctypes.byref(n)))
    return n.value


def workspace_probe(stream):
    """(partial sums, counters) device addresses of the K-split workspace of `stream` (a raw hipStream_t or None)."""
    a, b = ctypes.c_void_p(), ctypes.c_void_p()
    check(lib().acc950_workspace_probe(stream, ctypes.byref(a), ctypes.byref(b)))
    return a.value, b.value


def release_workspaces():
    """Frees the K-split workspaces of the current device (all streams) after waiting for the device to go idle."""
    check(lib().acc950_release_workspaces())


def variant_name(variant):
    buf = ctypes.create_string_buffer(128)
    check(lib().acc950_variant_name(int(variant), buf, 128))
    return buf.value.decode()


def num_variants():
    return lib().acc950_num_variants()


def num_skinny_variants():
    return lib().acc950_num_skinny_variants()


def launch_geometry(in_type, out_type, M, N, K, a_strides, b_strides, c_strides, variant=VARIANT_AUTO, k_splits=0):
    """(grid, block, dynamic_lds_bytes, chosen_variant) of the kernel a call would launch."""
    grid = (ctypes.c_uint * 3)()
    block = (ctypes.c_uint * 3)()
    lds = ctypes.c_uint()
    chosen = ctypes.c_int()
    check(lib().acc950_launch_geometry(in_type, out_type, M, N, K, *a_strides, *b_strides, *c_strides, variant, k_splits,
                                       grid, block, ctypes.byref(lds), ctypes.byref(chosen)))
    return list(grid), list(block), lds.value, chosen.value
