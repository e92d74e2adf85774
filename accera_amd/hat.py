"""HAT package boundary: a `.hat` writer that follows Accera's emitter, and a loader /
benchmark runner with hatlib's call surface.

Why both live here: the reference delivers compiled functions as a HAT package
(`<name>.hat` = TOML-annotated C header, plus the library it names) and consumers open it
with the third-party `hatlib` (`hat.load`, per-function calls on NumPy arrays,
`hat.run_benchmark`).  hatlib is not part of the reference tree and is not installed in
this image, so the tests of this repository use `load` / `run_benchmark` below, which
implement the same contract on top of `tomli` + `ctypes`; the `.hat` files themselves
stick to the emitter's schema so that the real hatlib reads them unchanged.

Format sources (emitter side, all in the reference tree):
  /root/reference/accera/hat/include/HATEmitter.h:22-97,1197-1265   TOML/C interleaving, table order
  /root/reference/accera/ir/src/TranslateToHeader.cpp:165-201        C prologue / epilogue of the header
  /root/reference/accera/ir/src/TranslateToHeader.cpp:403-506        prototypes + base-name alias
  /root/reference/accera/ir/src/TranslateToHeader.cpp:713-762        argument records (shape, affine_map)
  /root/reference/accera/python/accera/Package.py:672-784            fields completed after emission
  /root/reference/docs/Tutorials/Optimized_MatMul.md:176-193         sample function record
Consumer contract: /root/reference/README.md:118-136, /root/reference/accera/python/accera/test/verifiers.py:18-38,
/root/reference/tools/benchmarkers/accera_gemm.py:612-654.
"""
import ctypes
import os
import time
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

# element_type names of the header (TranslateToHeader.cpp:165-192, 329-400) <-> NumPy
ELEMENT_TYPES = {
    "float": np.float32, "double": np.float64, "float16_t": np.float16, "bfloat16_t": np.uint16,
    "int8_t": np.int8, "int16_t": np.int16, "int32_t": np.int32, "int64_t": np.int64,
    "uint8_t": np.uint8, "uint16_t": np.uint16, "uint32_t": np.uint32, "uint64_t": np.uint64, "bool": np.bool_,
}


@dataclass
class Argument:
    name: str = ""
    description: str = ""
    logical_type: str = "affine_array"
    declared_type: str = "float*"
    element_type: str = "float"
    usage: str = "input"  # input | input_output | output
    shape: List[int] = field(default_factory=list)
    affine_map: List[int] = field(default_factory=list)  # strides in elements
    affine_offset: int = 0

    def to_toml(self):
        return ("{" f"name = '{self.name}', description = '{self.description}', logical_type = \"{self.logical_type}\", "
                f"declared_type = '{self.declared_type}', element_type = '{self.element_type}', usage = \"{self.usage}\", "
                f"shape = {list(self.shape)}, affine_map = {list(self.affine_map)}, affine_offset = {self.affine_offset}" "}")


@dataclass
class Function:
    """A `[functions.<name>]` record, or with calling_convention "device" a `[device_functions.<name>]` one
    (the fields the reference fills in for GPU targets: /root/reference/accera/python/accera/Package.py:714-743)."""
    name: str
    base_name: str
    arguments: List[Argument]
    description: str = ""
    calling_convention: str = "cdecl"
    auxiliary: Dict[str, object] = field(default_factory=dict)
    runtime: str = ""                  # host function of a GPU target: "ROCM"
    launches: str = ""                 # host function of a GPU target: name of its device function
    launch_parameters: List[int] = field(default_factory=list)   # device function: grid x, y, z, block x, y, z
    dynamic_shared_mem_bytes: int = 0  # device function
    provider: str = ""                 # device function: the file that holds the kernel

    @property
    def c_signature(self):
        return ", ".join(a.declared_type for a in self.arguments)


def _toml_value(v):
    if isinstance(v, bool):
        return "true" if v else "false"
    if isinstance(v, (int, float)):
        return repr(v)
    if isinstance(v, (list, tuple)):
        return "[" + ", ".join(_toml_value(x) for x in v) + "]"
    if isinstance(v, dict):
        return "{" + ", ".join(f"{k} = {_toml_value(x)}" for k, x in v.items()) + "}"
    return "'" + str(v).replace("'", "") + "'"


def _function_record(table, fn):
    out = [f"[{table}.{fn.name}]", f"name = '{fn.name}'", f"description = '{fn.description}'",
           f"calling_convention = \"{fn.calling_convention}\"", "arguments = ["]
    out += ["    " + a.to_toml() + ("," if i + 1 < len(fn.arguments) else "") for i, a in enumerate(fn.arguments)]
    out += ["]", "return = {name = '', description = '', logical_type = \"void\", declared_type = 'void', "
            "element_type = 'void', usage = \"output\"}"]
    if fn.calling_convention == "device":
        out += [f"launch_parameters = {list(fn.launch_parameters)}", f"dynamic_shared_mem_bytes = {int(fn.dynamic_shared_mem_bytes)}",
                f"provider = '{fn.provider}'"]
    elif fn.launches:
        out.append(f"launches = '{fn.launches}'")
    if fn.runtime:
        out.append(f"runtime = '{fn.runtime}'")
    out.append("")
    for sub, values in fn.auxiliary.items():
        out.append(f"[{table}.{fn.name}.auxiliary.{sub}]")
        out += [f"{k} = {_toml_value(v)}" for k, v in values.items()]
        out.append("")
    return out


def write_hat(path, package_name, functions, link_target, author="", version="", license_url="", comment=None,
              required_gpu=None, compiled_with=None, device_functions=None):
    """Write `<package>.hat` in the emitter's layout (table order: HATEmitter.h:1197-1265); `device_functions`
    become the `[device_functions.*]` tables of a GPU package (Package.py:733-743)."""
    guard = f"__{package_name}__"
    out = [f"#ifndef {guard}", f"#define {guard}", "", "#ifdef TOML", "", "[description]",
           f"author = '{author}'", f"comment = '{comment if comment is not None else package_name}'",
           f"license_url = '{license_url}'", f"version = '{version}'", ""]
    out.append("[functions]")
    for fn in functions:
        out += _function_record("functions", fn)
    if device_functions:
        out.append("[device_functions]")
        for fn in device_functions:
            out += _function_record("device_functions", fn)
    out += ["[target]", "[target.required]", "os = \"linux\"", "[target.required.CPU]", "architecture = 'x86_64'",
            "extensions = []", ""]
    if required_gpu:
        out += ["[target.required.GPU]"] + [f"{k} = {_toml_value(v)}" for k, v in required_gpu.items()] + [""]
    out += ["[target.optimized_for]", "", "[dependencies]", f"link_target = '{link_target}'", "deploy_files = []",
            "dynamic = []", "[dependencies.auxiliary]", f"dynamic = '{link_target}'", "", "[compiled_with]"]
    cw = {"compiler": "", "flags": "", "crt": "", "libraries": []}
    cw.update(compiled_with or {})
    out += [f"{k} = {_toml_value(v)}" for k, v in cw.items()]
    out += ["", "[declaration]", "code = '''", "#endif // TOML", "//", f"// Header for Accera library {package_name}", "//",
            "#if defined(__cplusplus)", "#include <cstdint>", "#else", "#include <stdint.h>", "#include <stdbool.h>",
            "#endif // defined(__cplusplus)", "#if !defined(ACCERA_FLOAT)", "#define ACCERA_FLOAT 1",
            "typedef uint16_t float16_t;", "typedef uint16_t bfloat16_t;", "#endif // !defined(ACCERA_FLOAT)",
            "#if defined(__cplusplus)", "extern \"C\"", "{", "#endif // defined(__cplusplus)", "//", "// Functions", "//"]
    aliased = set()
    for fn in functions:
        out.append(f"void {fn.name}({fn.c_signature});")
        out.append("")
        if fn.base_name not in aliased:  # the first function of a base name gets the alias (Manual/10 Packages.md:32-40)
            aliased.add(fn.base_name)
            out += [f"#ifndef __{fn.base_name}_DEFINED__", f"#define __{fn.base_name}_DEFINED__",
                    f"void (*{fn.base_name})({fn.c_signature}) = {fn.name};", "#endif", ""]
    out += ["#if defined(__cplusplus)", "} // extern \"C\"", "#endif // defined(__cplusplus)", "#ifdef TOML", "'''", "",
            "#endif // TOML", "", f"#endif // {guard}", ""]
    with open(path, "w") as f:
        f.write("\n".join(out))
    return path


# ---------------------------------------------------------------------------------------------
# consumer side: hatlib-style loader
# ---------------------------------------------------------------------------------------------

def parse(hat_path):
    """The TOML content of a .hat file.  The preprocessor lines start with '#', a TOML
    comment, and the C code sits inside the `declaration.code` literal string, so the
    whole file is one TOML document."""
    import tomli
    with open(hat_path, "rb") as f:
        return tomli.load(f)


class _Hip:
    """The few HIP runtime calls the device-resident paths need (device buffers, copies, events), bound with ctypes:
    what hatlib's own ROCm path does through its pyhip module.  The runtime is already in the process once a package
    library is loaded."""
    _lib = None

    @classmethod
    def lib(cls):
        if cls._lib is None:
            L = ctypes.CDLL("libamdhip64.so")
            vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
            L.hipSetDevice.argtypes = [ci]
            L.hipMalloc.argtypes = [ctypes.POINTER(vp), sz]
            L.hipFree.argtypes = [vp]
            L.hipMemcpy.argtypes = [vp, vp, sz, ci]
            L.hipEventCreate.argtypes = [ctypes.POINTER(vp)]
            L.hipEventRecord.argtypes = [vp, vp]
            L.hipEventSynchronize.argtypes = [vp]
            L.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), vp, vp]
            L.hipEventDestroy.argtypes = [vp]
            L.hipGetErrorString.argtypes = [ci]
            L.hipGetErrorString.restype = ctypes.c_char_p
            cls._lib = L
        return cls._lib

    @classmethod
    def check(cls, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what}: {cls.lib().hipGetErrorString(rc).decode()}")

    @classmethod
    def set_device(cls, device_id):
        cls.check(cls.lib().hipSetDevice(int(device_id)), "hipSetDevice")

    @classmethod
    def to_device(cls, arr):
        """Device copy of a NumPy array's memory extent, as it lies (any strides)."""
        p = ctypes.c_void_p()
        lo, hi = np.lib.array_utils.byte_bounds(arr) if hasattr(np.lib, "array_utils") else np.byte_bounds(arr)
        nbytes = max(16, hi - lo)
        cls.check(cls.lib().hipMalloc(ctypes.byref(p), nbytes), "hipMalloc")
        if hi > lo:
            cls.check(cls.lib().hipMemcpy(p, ctypes.c_void_p(lo), hi - lo, 1), "hipMemcpy to device")
        return p, lo, hi

    @classmethod
    def to_host(cls, p, lo, hi):
        if hi > lo:
            cls.check(cls.lib().hipMemcpy(ctypes.c_void_p(lo), p, hi - lo, 2), "hipMemcpy to host")

    @classmethod
    def free(cls, p):
        cls.lib().hipFree(p)


class HATFunctionCall:
    """One package function, callable on NumPy arrays; checks the arguments against the
    .hat record (count, dtype, shape, strides) before handing raw pointers to the library.

    A function of a GPU package (`launches` names a `[device_functions]` record) can also be called with
    `device_id=`: the arrays are copied to that GPU, the function's device-pointer entry runs there and the
    written arrays are copied back -- hatlib's calling form for GPU packages
    (/root/reference/tools/benchmarkers/accera_gemm.py:612-615).  Without `device_id` the host-pointer symbol is
    called, which does the same copies inside the library."""

    def __init__(self, name, record, cfunc, device_record=None, device_cfunc=None):
        self.name = name
        self.record = record
        self.arguments = record["arguments"]
        self.device_record = device_record
        self._cfunc = cfunc
        self._cfunc.restype = None
        self._cfunc.argtypes = [ctypes.c_void_p] * len(self.arguments)
        self._device_cfunc = device_cfunc
        if device_cfunc is not None:
            device_cfunc.restype = ctypes.c_int
            device_cfunc.argtypes = [ctypes.c_void_p] * (len(self.arguments) + 1)

    @property
    def launches(self):
        return self.record.get("launches")

    def launch_on_device(self, device_pointers, stream=None):
        """Asynchronous launch on DEVICE pointers (ints or c_void_p), one per argument, on `stream` (hipStream_t or None)."""
        if self._device_cfunc is None:
            raise RuntimeError(f"{self.name}: the package records no device function for it")
        rc = self._device_cfunc(*device_pointers, stream)
        if rc != 0:
            raise RuntimeError(f"{self.name}: device entry point returned status {rc}")

    def _check(self, i, arr, arg):
        if not isinstance(arr, np.ndarray):
            raise TypeError(f"{self.name}: argument {i} must be a NumPy array")
        want = np.dtype(ELEMENT_TYPES[arg["element_type"]])
        if arr.dtype != want and not (arg["element_type"] == "bfloat16_t" and arr.dtype.itemsize == 2):
            raise ValueError(f"{self.name}: argument {i} has dtype {arr.dtype}, the package expects {want} ({arg['element_type']})")
        if list(arr.shape) != list(arg["shape"]):
            raise ValueError(f"{self.name}: argument {i} has shape {arr.shape}, the package expects {tuple(arg['shape'])}")
        strides = [s * arr.itemsize for s in arg["affine_map"]]
        got = [st for st, n in zip(arr.strides, arr.shape)]
        if any(n > 1 and g != s for g, s, n in zip(got, strides, arr.shape)):
            raise ValueError(f"{self.name}: argument {i} has byte strides {tuple(got)}, the package expects {tuple(strides)} "
                             f"(affine_map {arg['affine_map']})")
        if arg["usage"] != "input" and not arr.flags.writeable:
            raise ValueError(f"{self.name}: argument {i} is written by the function but is read-only")

    def __call__(self, *arrays, device_id=None):
        if len(arrays) != len(self.arguments):
            raise ValueError(f"{self.name}: expected {len(self.arguments)} arguments, got {len(arrays)}")
        for i, (arr, arg) in enumerate(zip(arrays, self.arguments)):
            self._check(i, arr, arg)
        if device_id is None or self._device_cfunc is None:
            self._cfunc(*[a.ctypes.data for a in arrays])
            return
        _Hip.set_device(device_id)
        bufs = [_Hip.to_device(a) for a in arrays]
        try:
            # (a pointer to the array's first element: the extent may start below it for negative strides, which _check refuses)
            self.launch_on_device([ctypes.c_void_p(p.value + (a.ctypes.data - lo)) for (p, lo, hi), a in zip(bufs, arrays)])
            for (p, lo, hi), arg in zip(bufs, self.arguments):
                if arg["usage"] != "input":
                    _Hip.to_host(p, lo, hi)  # (a synchronous copy on the null stream: it follows the kernel)
        finally:
            for p, _, _ in bufs:
                _Hip.free(p)


class FunctionDict(dict):
    """name -> callable; also attribute access and `.names`, as verifiers.py:20-30 uses."""

    @property
    def names(self):
        return list(self.keys())

    def __getattr__(self, name):
        try:
            return self[name]
        except KeyError:
            raise AttributeError(name)


@dataclass
class HATPackage:
    name: str
    path: str
    link_target_path: str
    hat: dict
    library: Optional[ctypes.CDLL] = None


def load(hat_path):
    """(package, functions): parse the .hat, dlopen `dependencies.link_target` (relative to
    the .hat), and wrap every entry of `[functions]`.  Base-name aliases resolve to the
    first function carrying that base name, like the header's function-pointer alias."""
    hat_path = os.path.abspath(hat_path)
    doc = parse(hat_path)
    link = doc["dependencies"]["link_target"]
    lib_path = os.path.join(os.path.dirname(hat_path), link)
    if not os.path.exists(lib_path):
        raise FileNotFoundError(f"link_target {lib_path} named by {hat_path} does not exist")
    lib = ctypes.CDLL(lib_path)
    funcs = FunctionDict()
    aliases = {}
    device_functions = doc.get("device_functions", {})
    for name, rec in doc.get("functions", {}).items():
        dev_rec = device_functions.get(rec.get("launches", ""))
        # the device-pointer entry of the host function lives in the same library (`<fn>__device`; the auxiliary
        # table names it) -- the kernels are prebuilt, there is no source for a run-time compiler
        dev_name = rec.get("auxiliary", {}).get("accera_mi355x", {}).get("device_entry", name + "__device")
        dev_fn = getattr(lib, dev_name, None) if dev_rec is not None else None
        call = HATFunctionCall(name, rec, getattr(lib, name), dev_rec, dev_fn)
        funcs[name] = call
        base = rec.get("auxiliary", {}).get("accera", {}).get("base_name")
        if base and base not in aliases:
            aliases[base] = call
    for base, call in aliases.items():
        funcs.setdefault(base, call)
    pkg = HATPackage(name=os.path.splitext(os.path.basename(hat_path))[0], path=hat_path, link_target_path=lib_path,
                     hat=doc, library=lib)
    return pkg, funcs


# ---------------------------------------------------------------------------------------------
# run_benchmark
# ---------------------------------------------------------------------------------------------

@dataclass
class BenchmarkResult:
    """Per-function timing statistics, in seconds (field names as in hatlib's result rows:
    /root/reference/docs/Tutorials/GPU/Hello_MatMul_GPU.md:207-209; `min_of_means` is what the
    reference's sweep consumes, accera_gemm.py:648).  The estimator itself is this
    library's: hatlib's exact statistics are not pinned by anything in the reference."""
    function_name: str
    mean: float
    median_of_means: float
    mean_of_small_means: float
    robust_mean: float
    min_of_means: float


def _random_args(rec, rng):
    args = []
    for a in rec["arguments"]:
        dt = np.dtype(ELEMENT_TYPES[a["element_type"]])
        shape = tuple(a["shape"])
        order = "F" if (len(shape) == 2 and a["affine_map"][0] == 1 and shape[1] > 1) else "C"
        if a["element_type"] == "bfloat16_t":
            x = (rng.standard_normal(shape).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        elif dt.kind == "f":
            x = rng.random(shape).astype(dt)
        else:
            x = rng.integers(-2, 3, shape).astype(dt)
        args.append(np.asarray(x, order=order))
    return args


def _stats(name, means, verbose):
    m = np.sort(np.array(means))
    small = m[: max(1, len(m) // 2)]
    trimmed = m[len(m) // 5: max(len(m) // 5 + 1, len(m) - len(m) // 5)]
    r = BenchmarkResult(name, float(m.mean()), float(np.median(m)), float(small.mean()), float(trimmed.mean()), float(m[0]))
    if verbose:
        print(r)
    return r


def run_benchmark(hat_path, store_in_hat=False, batch_size=10, min_time_in_sec=10, input_sets_minimum_size_MB=50,
                  device_id=0, verbose=False, functions=None, host_pointers=False):
    """Time every function of a package, hatlib-style: enough distinct input sets to exceed
    `input_sets_minimum_size_MB`, a warm-up call, then batches of `batch_size` calls until `min_time_in_sec` has
    passed.  Returns a list of BenchmarkResult (seconds per call).

    A function of a GPU package (one that `launches` a device function) is timed the way hatlib times GPU
    functions, which is what the reference's sweep consumes (/root/reference/tools/benchmarkers/accera_gemm.py:621-626, 648):
    inputs resident on GPU `device_id`, every batch bracketed by HIP events on the launch stream, no copies in the
    timed region.  `host_pointers=True` (or a function without a device record) times the HAT entry point on host
    arrays instead, copies to and from the GPU included."""
    del store_in_hat
    _, funcs = load(hat_path)
    rng = np.random.default_rng(0)
    results = []
    seen = set()
    for name, call in funcs.items():
        if id(call) in seen or (functions and name not in functions):
            continue
        seen.add(id(call))
        one = _random_args(call.record, rng)
        set_bytes = max(1, sum(a.nbytes for a in one))
        n_sets = max(1, min(64, int(np.ceil(input_sets_minimum_size_MB * 1e6 / set_bytes))))
        sets = [one] + [_random_args(call.record, rng) for _ in range(n_sets - 1)]
        means = []
        if call.device_record is not None and not host_pointers:
            H = _Hip.lib()
            _Hip.set_device(device_id)
            dev_sets = [[_Hip.to_device(a) for a in s] for s in sets]
            ptrs = [[ctypes.c_void_p(p.value + (a.ctypes.data - lo)) for (p, lo, hi), a in zip(ds, s)] for ds, s in zip(dev_sets, sets)]
            e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
            _Hip.check(H.hipEventCreate(ctypes.byref(e0)), "hipEventCreate")
            _Hip.check(H.hipEventCreate(ctypes.byref(e1)), "hipEventCreate")
            try:
                call.launch_on_device(ptrs[0])  # warm-up
                t_start, i = time.perf_counter(), 0
                while True:
                    _Hip.check(H.hipEventRecord(e0, None), "hipEventRecord")
                    for _ in range(batch_size):
                        call.launch_on_device(ptrs[i % n_sets])
                        i += 1
                    _Hip.check(H.hipEventRecord(e1, None), "hipEventRecord")
                    _Hip.check(H.hipEventSynchronize(e1), "hipEventSynchronize")
                    ms = ctypes.c_float()
                    _Hip.check(H.hipEventElapsedTime(ctypes.byref(ms), e0, e1), "hipEventElapsedTime")
                    means.append(ms.value * 1e-3 / batch_size)
                    if time.perf_counter() - t_start >= min_time_in_sec:
                        break
            finally:
                H.hipEventDestroy(e0)
                H.hipEventDestroy(e1)
                for ds in dev_sets:
                    for p, _, _ in ds:
                        _Hip.free(p)
        else:
            call(*sets[0])  # warm-up
            t_start, i = time.perf_counter(), 0
            while True:
                t0 = time.perf_counter()
                for _ in range(batch_size):
                    call(*sets[i % n_sets])
                    i += 1
                means.append((time.perf_counter() - t0) / batch_size)
                if time.perf_counter() - t_start >= min_time_in_sec:
                    break
        results.append(_stats(call.name, means, verbose))
    return results
