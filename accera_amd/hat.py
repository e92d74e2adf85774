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
    name: str
    base_name: str
    arguments: List[Argument]
    description: str = ""
    calling_convention: str = "cdecl"
    auxiliary: Dict[str, object] = field(default_factory=dict)

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


def write_hat(path, package_name, functions, link_target, author="", version="", license_url="", comment=None,
              required_gpu=None, compiled_with=None):
    """Write `<package>.hat` in the emitter's layout (table order: HATEmitter.h:1197-1265)."""
    guard = f"__{package_name}__"
    out = [f"#ifndef {guard}", f"#define {guard}", "", "#ifdef TOML", "", "[description]",
           f"author = '{author}'", f"comment = '{comment if comment is not None else package_name}'",
           f"license_url = '{license_url}'", f"version = '{version}'", ""]
    out.append("[functions]")
    for fn in functions:
        out += [f"[functions.{fn.name}]", f"name = '{fn.name}'", f"description = '{fn.description}'",
                f"calling_convention = \"{fn.calling_convention}\"", "arguments = ["]
        out += ["    " + a.to_toml() + ("," if i + 1 < len(fn.arguments) else "") for i, a in enumerate(fn.arguments)]
        out += ["]", "return = {name = '', description = '', logical_type = \"void\", declared_type = 'void', "
                "element_type = 'void', usage = \"output\"}", ""]
        for table, values in fn.auxiliary.items():
            out.append(f"[functions.{fn.name}.auxiliary.{table}]")
            out += [f"{k} = {_toml_value(v)}" for k, v in values.items()]
            out.append("")
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


class HATFunctionCall:
    """One package function, callable on NumPy arrays; checks the arguments against the
    .hat record (count, dtype, shape, strides) before handing raw pointers to the library."""

    def __init__(self, name, record, cfunc):
        self.name = name
        self.record = record
        self.arguments = record["arguments"]
        self._cfunc = cfunc
        self._cfunc.restype = None
        self._cfunc.argtypes = [ctypes.c_void_p] * len(self.arguments)

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

    def __call__(self, *arrays):
        if len(arrays) != len(self.arguments):
            raise ValueError(f"{self.name}: expected {len(self.arguments)} arguments, got {len(arrays)}")
        for i, (arr, arg) in enumerate(zip(arrays, self.arguments)):
            self._check(i, arr, arg)
        self._cfunc(*[a.ctypes.data for a in arrays])


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
    for name, rec in doc.get("functions", {}).items():
        call = HATFunctionCall(name, rec, getattr(lib, name))
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


def run_benchmark(hat_path, store_in_hat=False, batch_size=10, min_time_in_sec=10, input_sets_minimum_size_MB=50,
                  device_id=0, verbose=False, functions=None):
    """Time every function of a package through its HAT entry point (host pointers, i.e.
    including the copies to and from the GPU), hatlib-style: enough distinct input sets
    to exceed `input_sets_minimum_size_MB`, a warm-up call, then batches of `batch_size`
    calls until `min_time_in_sec` has passed.  Returns a list of BenchmarkResult."""
    del store_in_hat, device_id
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
        call(*sets[0])  # warm-up
        means, t_start, i = [], time.perf_counter(), 0
        while True:
            t0 = time.perf_counter()
            for _ in range(batch_size):
                call(*sets[i % n_sets])
                i += 1
            means.append((time.perf_counter() - t0) / batch_size)
            if time.perf_counter() - t_start >= min_time_in_sec:
                break
        m = np.sort(np.array(means))
        small = m[: max(1, len(m) // 2)]
        trimmed = m[len(m) // 5: max(len(m) // 5 + 1, len(m) - len(m) // 5)]
        r = BenchmarkResult(call.name, float(m.mean()), float(np.median(m)), float(small.mean()), float(trimmed.mean()),
                            float(m[0]))
        if verbose:
            print(r)
        results.append(r)
    return results
