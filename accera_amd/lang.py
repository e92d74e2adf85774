"""The slice of Accera's Python DSL that describes the matmul (+ fused ReLU) hot path.

Scripts written against the reference -- the README quick start
(/root/reference/README.md:52-92) and the GPU matmul / matmul+ReLU plans of
/root/reference/accera/python/accera/test/mfma_tests.py:58-101,359-432 -- run against
this module with `import accera_amd as acc`:

    A = acc.Array(role=acc.Role.INPUT, element_type=acc.ScalarType.float16, shape=(M, K))
    ...
    nest = acc.Nest(shape=(M, N, K)); i, j, k = nest.get_indices()
    @nest.iteration_logic
    def _(): C[i, j] += A[i, k] * B[k, j]
    plan = nest.create_schedule().create_plan(acc.Target(acc.Target.Model.AMD_MI355X))
    plan.tensorize(..., prologue_op=acc.MMAFragmentOp.SET, prologue_arg=0, epilogue_op=acc.MMAFragmentOp.ReLU)
    package.add(plan, args=(A, B, C), base_name="matmul_relu")
    package.build("pkg", format=acc.Package.Format.HAT_DYNAMIC, output_dir=...)

There is no compiler behind it.  `Package.add` pattern-matches the recorded logic to
`C[i,j] += A[i,k] * B[k,j]` optionally fused with `C[i,j] = max(C[i,j], 0)` -- exactly the
pattern the reference's tensorization matcher accepts
(/root/reference/accera/transforms/src/exec/ExecutionPlanToAffineLoweringPass.cpp:5986-6167) --
and binds the function to the prebuilt gfx950 kernels of libaccera_mi355x.so; schedule and
plan transformations (tile, reorder, cache, bind, unroll, ...) are accepted and recorded,
because the kernels embody their own tiling, caching and binding.  Anything that is not this
pattern raises NotImplementedError.  `Package.build` emits `<name>.hat` + `<name>.so`.
"""
import enum
import hashlib
import re
import os
import subprocess

from . import _lib
from . import hat as _hat


class Role(enum.Enum):
    INPUT = "input"
    INPUT_OUTPUT = "input_output"
    OUTPUT = "output"
    CONST = "const"
    TEMP = "temp"


class ScalarType(enum.Enum):
    float32 = ("float", _lib.F32)
    float16 = ("float16_t", _lib.F16)
    bfloat16 = ("bfloat16_t", _lib.BF16)
    int8 = ("int8_t", _lib.I8)
    int32 = ("int32_t", _lib.I32)
    int16 = ("int16_t", _lib.I16)

    @property
    def c_name(self):
        return self.value[0]

    @property
    def lib_id(self):
        return self.value[1]


class MMAFragmentOp(enum.Enum):  # /root/reference/docs/Reference/enumerations/MMAFragmentOp.md
    NONE = 0
    ReLU = 1
    ReLU_NoConditional = 2
    SET = 3
    SCALE = 4


class MMAShape(enum.Enum):
    """The reference's shape names (/root/reference/accera/ir/include/value/ValueMMAOp.h:27-49) plus the gfx950 ones.
    M x N x K is the product one matrix instruction forms, in elements.  Only the shapes in
    Target.MI355X_TENSORCORE_INFO exist on this target; `plan.tensorize` refuses the others, and the shape it is given
    selects the kernel family (16x16 or 32x32 instruction shapes)."""
    M64xN64xK1_B4 = 0
    M64xN64xK1_B2 = 1
    M32xN32xK2_B1 = 2     # gfx950: v_mfma_f32_32x32x2_f32
    M16xN16xK4_B1 = 3
    M64xN64xK4_B4 = 4
    M64xN64xK4_B2 = 5
    M32xN32xK8_B1 = 6
    M16xN16xK16_B1 = 7
    M64xN64xK2_B4 = 8
    M64xN64xK2_B2 = 9
    M32xN32xK4_B1 = 10
    M16xN16xK8_B1 = 11
    M32xN32xK16_B1 = 12   # gfx950: v_mfma_f32_32x32x16_{f16,bf16}
    M32xN32xK32_B1 = 13   # gfx950: v_mfma_i32_32x32x32_i8
    M16xN16xK32_B1 = 14   # gfx950: v_mfma_f32_16x16x32_{f16,bf16}
    M16xN16xK64_B1 = 15   # gfx950: v_mfma_i32_16x16x64_i8
    M32xN8xK16_B1 = 16
    M8xN32xK16_B1 = 17

    @property
    def dims(self):
        """(M, N, K) of the shape."""
        m, n, k = self.name.split("_")[0].split("x")
        return int(m[1:]), int(n[1:]), int(k[1:])


class MMASchedulingPolicy(enum.Enum):
    PASS_ORDER = 0
    BLOCK_ORDER = 1


class _Auto:
    def __repr__(self):
        return "AUTO"


AUTO = _Auto()  # "let the compiler decide" default of cache arguments (the reference's accera.AUTO)


class CacheStrategy(enum.Enum):
    BLOCKED = 0
    STRIPED = 1


class _MemorySpace(enum.Enum):
    NONE = 0
    GLOBAL = 1
    SHARED = 2
    PRIVATE = 3
    MMA_FRAGMENT = 4


class TensorCoreInformationEntry:
    """One matrix-instruction shape for one (input, output) type pair
    (/root/reference/accera/python/accera/Targets.py:748-753)."""

    def __init__(self, shape, inType, outType):
        self.shape, self.inType, self.outType = shape, inType, outType

    def __repr__(self):
        return f"TensorCoreInformationEntry({self.shape.name}, {self.inType.name} -> {self.outType.name})"


class TensorCoreInformation:
    """The matrix-core table of a target with the reference's queries (Targets.py:756-793)."""

    def __init__(self, entries=()):
        self.entries = list(entries)

    def supports(self, input_type, output_type, shape, num_total_passes=1, num_fused_passes=-1):
        if not (num_total_passes >= 1 and (num_fused_passes == -1 or num_total_passes % num_fused_passes == 0)):
            return False
        return any(e.inType == input_type and e.outType == output_type and e.shape == shape for e in self.entries)

    def supports_shape(self, shape, num_total_passes=1, num_fused_passes=-1):
        """Some type pair runs this shape (what plan.tensorize can check before it knows the arrays)."""
        return any(self.supports(e.inType, e.outType, shape, num_total_passes, num_fused_passes) for e in self.entries)

    def mma_shape_to_tuple(self, mma_shape):
        return mma_shape.dims

    def compute_tensor_splits(self, mma_shape, num_total_passes=1):
        m, n, k = mma_shape.dims
        return (m, n, k * num_total_passes)


class Target:
    """Device description.  Only the HOST default and the MI355X GPU exist here; the
    tensor-core table row is the gfx950 analogue of MI100_TENSORCORE_INFO
    (/root/reference/accera/python/accera/Targets.py:748-830)."""

    class Model(enum.Enum):
        HOST = "HOST"
        AMD_MI355X = "AMD MI355X"

    class Category(enum.Enum):
        CPU = 0
        GPU = 1

    class Runtime(enum.Enum):
        NONE = 0
        ROCM = 1

    class _GridUnit(enum.Enum):
        BLOCK_X = 0
        BLOCK_Y = 1
        BLOCK_Z = 2
        THREAD_X = 3
        THREAD_Y = 4
        THREAD_Z = 5
        WARP_X = 6
        WARP_Y = 7

    class _GridUnits:
        def __getattr__(self, name):
            return Target._GridUnit[name]

    # the matrix instructions of gfx950 this library's kernels are built on, per (input, output) type pair: the 16x16
    # shapes sum 64 bytes of K per instruction (the large-tile kernels), the 32x32 shapes 32 bytes
    MI355X_TENSORCORE_INFO = TensorCoreInformation(
        [TensorCoreInformationEntry(shape, tin, tout)
         for tin, outs, shapes in (
             (ScalarType.float16, (ScalarType.float32, ScalarType.float16), (MMAShape.M16xN16xK32_B1, MMAShape.M32xN32xK16_B1)),
             (ScalarType.bfloat16, (ScalarType.float32, ScalarType.bfloat16), (MMAShape.M16xN16xK32_B1, MMAShape.M32xN32xK16_B1)),
             (ScalarType.int8, (ScalarType.int32, ScalarType.int16, ScalarType.int8), (MMAShape.M16xN16xK64_B1, MMAShape.M32xN32xK32_B1)),
             (ScalarType.float32, (ScalarType.float32,), (MMAShape.M32xN32xK2_B1,)))
         for tout in outs for shape in shapes])

    def __init__(self, model=None, category=None, runtime=None):
        if isinstance(model, str):
            model = Target.Model(model)
        self.model = model or Target.Model.HOST
        gpu = self.model == Target.Model.AMD_MI355X or category == Target.Category.GPU
        self.category = Target.Category.GPU if gpu else Target.Category.CPU
        self.runtime = Target.Runtime.ROCM if gpu else Target.Runtime.NONE
        self.name = self.model.value
        self.GridUnit = Target._GridUnits()
        self.MemorySpace = _MemorySpace
        self.warp_size = 64
        self.compute_units = 256
        self.max_shared_memory_per_block = 160 * 1024
        self.tensor_core_info = Target.MI355X_TENSORCORE_INFO


Target.HOST = Target()


# ---- expression recording ---------------------------------------------------------------------

class Index:
    _count = 0

    def __init__(self, name=None):
        Index._count += 1
        self.name = name or f"i{Index._count}"

    def __repr__(self):
        return self.name


class _Expr:
    def __mul__(self, other):
        return _Bin("mul", self, _wrap(other))

    __rmul__ = __mul__

    def __add__(self, other):
        return _Bin("add", self, _wrap(other))

    __radd__ = __add__


class _Const(_Expr):
    def __init__(self, v):
        self.v = v


class _Bin(_Expr):
    def __init__(self, op, a, b):
        self.op, self.a, self.b = op, a, b


class _Cast(_Expr):
    def __init__(self, x, t):
        self.x, self.t = x, t


class _Ref(_Expr):
    def __init__(self, array, idx):
        self.array, self.idx = array, tuple(idx)

    def __iadd__(self, other):
        return _Bin("add", self, _wrap(other))


def _wrap(x):
    return x if isinstance(x, _Expr) else _Const(x)


def _strip_cast(e):
    while isinstance(e, _Cast):
        e = e.x
    return e


def max(a, b):  # noqa: A001 - mirrors acc.max
    return _Bin("max", _wrap(a), _wrap(b))


def min(a, b):  # noqa: A001
    return _Bin("min", _wrap(a), _wrap(b))


def cast(x, t):
    return _Cast(_wrap(x), t)


_recording = []  # stack of statement lists


class Array:
    class Layout(enum.Enum):
        FIRST_MAJOR = 0   # row-major   (/root/reference/accera/python/accera/lang/Layout.py:11-33)
        LAST_MAJOR = 1    # column-major
        DEFERRED = 2

    def __init__(self, role, element_type=ScalarType.float32, layout=None, shape=None, name="", **_):
        if shape is None or len(shape) not in (2, 3):
            raise NotImplementedError("this build handles matrices and batches of matrices (2-D / 3-D arrays) only")
        self.role = role
        self.element_type = element_type
        self.layout = layout or Array.Layout.FIRST_MAJOR
        self.shape = tuple(int(s) for s in shape)
        self.name = name

    @property
    def strides(self):
        """Element strides: FIRST_MAJOR has the last dimension contiguous, LAST_MAJOR the first
        (/root/reference/accera/python/accera/lang/Layout.py:36-58)."""
        dims = self.shape if self.layout == Array.Layout.FIRST_MAJOR else self.shape[::-1]
        out, step = [], 1
        for d in reversed(dims):
            out.append(step)
            step *= d
        out = out[::-1]
        return tuple(out if self.layout == Array.Layout.FIRST_MAJOR else out[::-1])

    def __getitem__(self, idx):
        return _Ref(self, idx)

    def __setitem__(self, idx, value):
        if not _recording:
            raise RuntimeError("array assignment outside of an iteration_logic function")
        _recording[-1].append((_Ref(self, idx), _wrap(value)))


class Nest:
    def __init__(self, shape):
        self.shape = tuple(int(s) for s in shape)
        self.indices = tuple(Index() for _ in self.shape)
        self.statements = []

    def get_indices(self):
        return self.indices if len(self.indices) > 1 else self.indices[0]

    def iteration_logic(self, fn):
        _recording.append([])
        try:
            fn()
        finally:
            self.statements += _recording.pop()
        return fn

    def create_schedule(self):
        return Schedule([self])

    def create_plan(self, target=None):
        return self.create_schedule().create_plan(target)


class Schedule:
    """Loop transformations are recorded, not applied: the gfx950 kernels carry their own
    tiling (reference semantics: /root/reference/accera/python/accera/lang/Schedule.py)."""

    def __init__(self, nests, fused=False, partial=None):
        self.nests = nests
        self.fused = fused
        self.partial = partial
        self.commands = []
        if fused:
            # fused indices, then the fusing index f, then the unfused ones (Schedule.py:522-628)
            first = nests[0]
            self.indices = list(first.indices[:partial]) + [Index("f")] + [ix for n in nests for ix in n.indices[partial:]]
        else:
            self.indices = list(nests[0].indices)

    def get_indices(self):
        return tuple(self.indices)

    def split(self, index, size):
        inner = Index(f"{index.name}i")
        self.indices.insert(self.indices.index(index) + 1, inner)
        self.commands.append(("split", index, size, inner))
        return inner

    def tile(self, shape):
        return tuple(self.split(ix, sz) for ix, sz in shape.items())

    def reorder(self, *order):
        order = order[0] if len(order) == 1 and isinstance(order[0], (tuple, list)) else order
        self.commands.append(("reorder", tuple(order)))
        self.indices = list(order)

    def skew(self, *a, **k):
        self.commands.append(("skew", a, k))

    def pad(self, *a, **k):
        self.commands.append(("pad", a, k))

    def create_plan(self, target=None):
        return Plan(self, target or Target.HOST)


def fuse(*schedules, partial=None):
    scheds = schedules[0] if len(schedules) == 1 and isinstance(schedules[0], (tuple, list)) else schedules
    nests = [n for s in scheds for n in s.nests]
    if partial is None:
        partial = len(nests[0].shape)
    return Schedule(nests, fused=True, partial=partial)


class Plan:
    """Execution-plan calls of the reference (Plan.py:134-703, 793-956).  `tensorize` carries semantics (prologue /
    epilogue op) and its `mma_shape` selects the kernel family; the block tile comes from the schedule's splits, its K
    depth from the split of k inside a SHARED cache of A or B; `cache` and `bind` check their arguments as the
    reference does; the rest (unroll, vectorize, ...) selects nothing here and is recorded."""

    def __init__(self, schedule, target):
        self.schedule = schedule
        self.target = target
        self.commands = []
        self.prologue_op, self.prologue_arg = MMAFragmentOp.NONE, 0
        self.epilogue_op, self.epilogue_arg = MMAFragmentOp.NONE, 0
        self.mma_shape, self.num_total_passes = None, 1
        self.caches = []

    def tensorize(self, indices, mma_shape=None, use_static_offsets=False, num_total_passes=1, num_fused_passes=None,
                  scheduling_policy=MMASchedulingPolicy.PASS_ORDER, prologue_op=MMAFragmentOp.NONE, prologue_arg=0,
                  epilogue_op=MMAFragmentOp.NONE, epilogue_arg=0, **_):
        # (the checks of the reference's Plan.tensorize / _tensorize, lang/Plan.py:242-361)
        if self.target.category != Target.Category.GPU:
            raise ValueError("tensorization currently only supported on GPU targets")
        indices = [indices] if isinstance(indices, Index) else list(indices)
        if len(indices) < 3:
            raise ValueError("tensorization requires at least three input indices")
        if num_fused_passes is not None and num_fused_passes <= 0:
            raise ValueError("Number of passes used for fusing must be a positive number greater than 0.")
        if mma_shape is None:
            raise ValueError("tensorize needs an mma_shape; this target's shapes are listed in target.tensor_core_info")
        if not self.target.tensor_core_info.supports_shape(mma_shape, num_total_passes, -1 if num_fused_passes is None else num_fused_passes):
            raise ValueError("The target does not support the given tensorization dimensions with shape=", mma_shape)
        self.mma_shape, self.num_total_passes = mma_shape, num_total_passes
        if prologue_op not in (MMAFragmentOp.NONE, MMAFragmentOp.SET, MMAFragmentOp.SCALE):
            raise NotImplementedError("prologue must be NONE, SET or SCALE")
        if epilogue_op not in (MMAFragmentOp.NONE, MMAFragmentOp.ReLU, MMAFragmentOp.ReLU_NoConditional, MMAFragmentOp.SET,
                               MMAFragmentOp.SCALE):
            raise NotImplementedError("unknown epilogue op")
        self.prologue_op, self.prologue_arg = prologue_op, prologue_arg
        self.epilogue_op, self.epilogue_arg = epilogue_op, epilogue_arg
        self.commands.append(("tensorize", mma_shape, num_total_passes))

    def cache(self, source, index=None, trigger_index=None, layout=None, max_elements=None, element_type=None, thrifty=None,
              location=_MemorySpace.NONE, level=None, trigger_level=None, double_buffer=False, double_buffer_location=AUTO,
              vectorize=AUTO, strategy=AUTO, **_):
        """The reference's `Plan.cache` (lang/Plan.py:381-703): same arguments, same argument checks.  What a cache means
        here: the kernels always stage blocks of A and B in LDS (the reference's SHARED caches) several K tiles deep
        (its double buffering, one tile deeper) and keep C in accumulator registers (its MMA_FRAGMENT cache), so a
        cache call does not switch staging on or off.  A SHARED cache of A or B does name the K depth of the staged block:
        the extent of the split of k inside the cache index -- the `k_split` axis of the reference's sweep
        (tools/benchmarkers/accera_gemm.py:281-293, 554-555) -- and a depth the library has kernels for (64 or 128 bytes
        of K) binds the package function to one of them."""
        if sum(x is not None for x in (index, level, max_elements)) != 1:
            raise ValueError("Specify one and only one of index, level, or max_elements")
        if max_elements is not None and max_elements <= 0:
            raise ValueError("Max element count specified as a cache budget must be greater than 0")
        target_array = source.array if isinstance(source, Cache) else source
        if not isinstance(target_array, Array):
            raise ValueError("the source of a cache is an Array or a Cache")
        if double_buffer and target_array.role not in (Role.CONST, Role.INPUT):
            raise ValueError("Double-buffering is only supported for CONST and INPUT arrays")
        if not double_buffer and double_buffer_location is not AUTO:
            raise ValueError("double_buffer_location is only valid to specify when double_buffer is set to True")
        gpu = self.target.category == Target.Category.GPU
        if gpu and location == _MemorySpace.GLOBAL:
            raise ValueError("Global memory caches are not yet supported on GPU targets.")
        if not gpu and strategy is not AUTO:
            raise ValueError("Only AUTO strategy is supported on the CPU")
        if double_buffer and location == _MemorySpace.MMA_FRAGMENT:
            raise ValueError("Double buffering is not supported with Tensor caching")
        if index is not None and (level is not None or trigger_level is not None):
            raise ValueError("Can't specify both a cache index and a cache level or trigger level")
        if level is not None and trigger_index is not None:
            raise ValueError("Can't specify both a cache level and a cache index or trigger index")
        order = self.schedule.indices
        if max_elements is None:
            if level is not None:
                if not 0 < level <= len(order):
                    raise ValueError("cache level out of range of the schedule's indices")
                index = order[-level]
            elif index not in order:
                raise ValueError("the cache index is not an index of this plan's schedule")
            if (trigger_level or trigger_index is not None) and target_array.role not in (Role.CONST, Role.INPUT):
                raise ValueError("Multicaching is only supported for CONST and INPUT arrays")
            if trigger_index is not None:
                if trigger_index not in order:
                    raise ValueError("the trigger index is not an index of this plan's schedule")
                if order.index(trigger_index) > order.index(index):
                    raise ValueError("Trigger index must be at or outside of the cache index")
            if trigger_level is not None and trigger_level < len(order) - order.index(index):
                raise ValueError("Trigger level must be greater than or equal to the cache level")
        if double_buffer_location is AUTO:
            double_buffer_location = ((_MemorySpace.PRIVATE if gpu and location == _MemorySpace.SHARED else location)
                                      if double_buffer else _MemorySpace.NONE)
        c = Cache(target_array, index, location, bool(double_buffer), double_buffer_location, layout,
                  CacheStrategy.STRIPED if strategy is AUTO else strategy)
        self.caches.append(c)
        self.commands.append(("cache", target_array.name, location.name, bool(double_buffer)))
        return c

    def bind(self, mapping):
        """The reference's `Plan.bind` (lang/Plan.py:793-878): indices (or tuples of indices) to the target's grid units.
        GPU targets only, indices of this plan only.  The launch geometry itself belongs to the kernel the block tile
        selects (one workgroup per tile, or per compute unit for the multi-tile form); the binding is recorded."""
        if self.target.category != Target.Category.GPU:
            raise ValueError("Only supported on plans with GPU targets")
        for ix, unit in dict(mapping).items():
            for one in (ix if isinstance(ix, (tuple, list)) else (ix,)):
                if one not in self.schedule.indices:
                    raise ValueError("bind: not an index of this plan's schedule")
            if not isinstance(unit[0] if isinstance(unit, (tuple, list)) else unit, Target._GridUnit):
                raise ValueError("bind: not a grid unit of the target")
        self.commands.append(("bind", len(dict(mapping))))

    def _record(name):
        def f(self, *a, **k):
            self.commands.append((name, a, k))
            return None
        return f

    unroll = _record("unroll")
    vectorize = _record("vectorize")
    parallelize = _record("parallelize")
    kernelize = _record("kernelize")
    del _record


class Cache:
    """Handle a `Plan.cache` call returns (usable as the source of a further cache: lang/Cache.py in the reference)."""

    def __init__(self, array, index, location, double_buffer, double_buffer_location, layout, strategy):
        self.array, self.index, self.location = array, index, location
        self.double_buffer, self.double_buffer_location, self.layout, self.strategy = double_buffer, double_buffer_location, layout, strategy


# ---- pattern match to the GEMM (+ReLU) hot path -------------------------------------------------

class _GemmSpec:
    def __init__(self, A, B, C, M, N, K, prologue, epilogue, prologue_arg=0.0, epilogue_arg=0.0, batch=None):
        self.A, self.B, self.C, self.M, self.N, self.K = A, B, C, M, N, K
        self.batch = batch  # None: plain GEMM; n: C[b,i,j] += A[b,i,k] * B[b,k,j] for b < n
        self.prologue, self.epilogue = prologue, epilogue
        self.prologue_arg, self.epilogue_arg = float(prologue_arg), float(epilogue_arg)
        self.block_tile = None               # (bm, bn) when a GPU plan's outermost splits of i and j name one
        self.mma_shape = None                # the tensorized plan's instruction shape
        self.gpu_target = False              # the function was added from a plan for a GPU target
        self.k_tile_bytes = None             # K depth of the block a SHARED cache of A or B stages, when the library has kernels of that depth
        self.variant = _lib.VARIANT_AUTO     # kernel instantiation picked from the block tile, else automatic


def _match(source):
    plan = source if isinstance(source, Plan) else None
    sched = plan.schedule if plan else (source if isinstance(source, Schedule) else source.create_schedule())
    nests = sched.nests
    unsupported = NotImplementedError(
        "this build compiles exactly one pattern: C[i,j] += A[i,k] * B[k,j] (or its batched form C[b,i,j] += A[b,i,k] * B[b,k,j]), "
        "optionally fused with C[i,j] = max(C[i,j], 0)")
    if len(nests) not in (1, 2) or len(nests[0].shape) not in (3, 4) or len(nests[0].statements) != 1:
        raise unsupported
    mm = nests[0]
    batched = len(mm.shape) == 4
    bidx = mm.indices[:1] if batched else ()
    i, j, k = mm.indices[-3:]
    dst, val = mm.statements[0]
    val = _strip_cast(val)
    if not (isinstance(val, _Bin) and val.op == "add"):
        raise unsupported
    acc_ref, prod = _strip_cast(val.a), _strip_cast(val.b)
    if not (isinstance(acc_ref, _Ref) and acc_ref.array is dst.array and acc_ref.idx == (*bidx, i, j) and dst.idx == (*bidx, i, j)):
        raise unsupported
    if not (isinstance(prod, _Bin) and prod.op == "mul"):
        raise unsupported
    a, b = _strip_cast(prod.a), _strip_cast(prod.b)
    if not (isinstance(a, _Ref) and isinstance(b, _Ref)):
        raise unsupported
    if a.idx == (*bidx, k, j) and b.idx == (*bidx, i, k):
        a, b = b, a
    if a.idx != (*bidx, i, k) or b.idx != (*bidx, k, j):
        raise unsupported
    M, N, K = mm.shape[-3:]
    nb = (mm.shape[0],) if batched else ()
    A, B, C = a.array, b.array, dst.array
    if A.shape != (*nb, M, K) or B.shape != (*nb, K, N) or C.shape != (*nb, M, N):
        raise ValueError(f"array shapes {A.shape}, {B.shape}, {C.shape} do not match the nest {mm.shape}")
    epilogue = _lib.EPILOGUE_NONE
    if len(nests) == 2:
        relu = nests[1]
        if not (sched.fused and sched.partial == len(nb) + 2 and relu.shape == (*nb, M, N) and len(relu.statements) == 1):
            raise unsupported
        ridx = tuple(relu.indices)
        rdst, rval = relu.statements[0]
        rval = _strip_cast(rval)
        ok = (rdst.array is C and rdst.idx == ridx and isinstance(rval, _Bin) and rval.op == "max")
        if ok:
            x, z = _strip_cast(rval.a), _strip_cast(rval.b)
            if isinstance(x, _Const):
                x, z = z, x
            ok = isinstance(x, _Ref) and x.array is C and x.idx == ridx and isinstance(z, _Const) and z.v == 0
        if not ok:
            raise unsupported
        epilogue = _lib.EPILOGUE_RELU
    prologue, prologue_arg, epilogue_arg = _lib.PROLOGUE_NONE, 0.0, 0.0
    if plan:
        if plan.prologue_op == MMAFragmentOp.SET:
            prologue, prologue_arg = _lib.PROLOGUE_SET, plan.prologue_arg
        elif plan.prologue_op == MMAFragmentOp.SCALE:
            prologue, prologue_arg = _lib.PROLOGUE_SCALE, plan.prologue_arg
        if plan.epilogue_op != MMAFragmentOp.NONE and epilogue != _lib.EPILOGUE_NONE:
            raise NotImplementedError("a fused ReLU nest and a tensorize epilogue op at the same time")
        if plan.epilogue_op == MMAFragmentOp.ReLU:
            epilogue = _lib.EPILOGUE_RELU
        elif plan.epilogue_op == MMAFragmentOp.ReLU_NoConditional:
            epilogue = _lib.EPILOGUE_RELU_NOCOND
        elif plan.epilogue_op == MMAFragmentOp.SCALE:
            epilogue, epilogue_arg = _lib.EPILOGUE_SCALE, plan.epilogue_arg
        elif plan.epilogue_op == MMAFragmentOp.SET:
            epilogue, epilogue_arg = _lib.EPILOGUE_SET, plan.epilogue_arg
    spec = _GemmSpec(A, B, C, M, N, K, prologue, epilogue, prologue_arg, epilogue_arg, batch=mm.shape[0] if batched else None)
    if plan and plan.target.category == Target.Category.GPU:
        spec.gpu_target = True
        # The outermost split of i and of j is the block tile of a GPU plan (the reference binds the
        # resulting outer indices to BLOCK_Y / BLOCK_X: lang/Plan.py:793-825, mfma_tests.py:89-97).  If
        # the library has an MFMA instantiation with that tile which takes this problem, the package
        # function is bound to it; otherwise the library chooses.
        first = {}
        for cmd in sched.commands:
            if cmd[0] == "split" and cmd[1] in (i, j) and cmd[1] not in first:
                first[cmd[1]] = int(cmd[2])
        family = None
        if plan.mma_shape is not None:
            # the shape must exist for the nest's own types (tensorize could only check that some type pair has it)
            if not plan.target.tensor_core_info.supports(A.element_type, C.element_type, plan.mma_shape, plan.num_total_passes):
                raise ValueError("The target does not support the given tensorization dimensions with shape=", plan.mma_shape,
                                 f"for {A.element_type.name} inputs and a {C.element_type.name} result")
            spec.mma_shape = plan.mma_shape
            if A.element_type != ScalarType.float32:
                family = "mi16" if plan.mma_shape.dims[0] == 16 else "mi32"
        if i in first and j in first:
            spec.block_tile = (first[i], first[j])
        # K depth of the staged block: the split of k inside the index of a SHARED cache of A or B (the cached block
        # then spans that many k); 64 or 128 bytes of K are depths the library has kernels for
        k_bytes = None
        shared = [c for c in plan.caches if c.location == _MemorySpace.SHARED and c.array in (A, B) and c.index is not None]
        if shared:
            order = sched.indices
            for cmd in sched.commands:
                if cmd[0] == "split" and cmd[1] is k:
                    # (the block cached at an index spans the loops at and inside it: the outer k loop runs over blocks,
                    # the inner one inside them)
                    inside = all(order.index(k) < order.index(c.index) <= order.index(cmd[3]) for c in shared
                                 if k in order and cmd[3] in order and c.index in order)
                    if inside:
                        k_bytes = int(cmd[2]) * {ScalarType.int8: 1, ScalarType.float32: 4}.get(A.element_type, 2)
                    break
        spec.k_tile_bytes = k_bytes if k_bytes in (64, 128) else None
        if family or spec.block_tile or spec.k_tile_bytes:
            spec.variant = _variant_for(spec, spec.block_tile, family, spec.k_tile_bytes)
    if spec.variant == _lib.VARIANT_AUTO and spec.batch is None:
        # no tile named by the plan: a choice recorded for this very shape by `accera_amd.tune --save`, if any
        from . import tuned
        hit = tuned.lookup(spec.A.element_type.lib_id, spec.C.element_type.lib_id, spec.M, spec.N, spec.K,
                           spec.A.strides[-2:], spec.B.strides[-2:], spec.C.strides[-2:],
                           tuned.ops_class(spec.prologue, spec.prologue_arg, spec.epilogue))
        if hit and hit[1] == 0:  # (package functions carry a variant, not a K split)
            spec.variant = hit[0]
    return spec


def _variant_for(spec, tile=None, family=None, k_bytes=None):
    """MFMA variant for a plan that names a block tile (bm, bn), an instruction-shape family ("mi16": the
    16x16 shapes, "mi32": the 32x32 ones) and / or the K depth of the staged block in bytes.  Among the variants that
    accept the problem: those of the named tile if there are any (else any tile), of the named family if there are
    any, of the named depth if there are any; the library's own choice when it is one of them, else the best-ranked.
    VARIANT_AUTO when nothing matches."""
    lean = spec.prologue == _lib.PROLOGUE_SET and spec.prologue_arg == 0 and spec.epilogue in (_lib.EPILOGUE_RELU, _lib.EPILOGUE_NONE)
    geometry = (spec.A.element_type.lib_id, spec.C.element_type.lib_id, spec.M, spec.N, spec.K,
                spec.A.strides[-2:], spec.B.strides[-2:], spec.C.strides[-2:])
    cands = []
    for v in range(_lib.num_variants()):
        name = _lib.variant_name(v)
        try:
            _lib.launch_geometry(*geometry, v, 0)
        except _lib.Acc950Error:
            continue
        if "hand-laid loop" in name and spec.prologue != _lib.PROLOGUE_SET and spec.C.element_type.lib_id == _lib.I8:
            continue  # (the four-wave kernels do not read an int8 C)
        cands.append((v, name))
    named = []
    if tile:
        named = [(v, n) for v, n in cands if f"mfma {tile[0]}x{tile[1]} " in n]
        if not named and not family and not k_bytes:
            return _lib.VARIANT_AUTO
        cands = named or cands
    if family:
        cands = [(v, n) for v, n in cands if ("mi16" in n) == (family == "mi16")] or cands
    if k_bytes:
        cands = [(v, n) for v, n in cands if f" kb{k_bytes} " in n] or cands
    if not cands:
        return _lib.VARIANT_AUTO
    try:
        auto = _lib.launch_geometry(*geometry, _lib.VARIANT_AUTO, 0)[3]
    except _lib.Acc950Error:
        auto = None
    if auto in [v for v, _ in cands]:
        return auto
    if auto is not None and auto >= _lib.num_variants() and not (tile and named):
        return _lib.VARIANT_AUTO  # the library runs this problem on a streaming / fp32 / thread-bound kernel: no MFMA tile to name

    def rank(name):
        bm, bn = map(int, re.search(r"mfma (\d+)x(\d+)", name).groups())
        tiles = -(-spec.M // bm) * -(-spec.N // bn)
        # ping-pong over software-pipelined; the 16x16 shapes where the library runs their lean build; four waves with
        # the hand-laid loop ahead of both (the multi-tile form when there is more than one round of tiles); then larger tiles
        r = 2 * ("pingpong" in name) + (1 if "mi16" in name and lean else -1 if "mi16" in name else 0)
        if "hand-laid loop" in name:
            # (multi-tile form when there is more than one round of tiles -- for a row-major A; the forms for a column-major A measured level)
            r = 4 + (("multi-tile" in name) == (tiles > 256 and "A=col-major" not in name))
        return (r, bm * bn if tiles >= 256 else -bm * bn, "edge" not in name)
    return sorted(cands, key=lambda c: rank(c[1]))[-1][0]  # (`max` is the DSL's elementwise maximum in this module)


# ---- package -------------------------------------------------------------------------------------

class Package:
    class Format(enum.Flag):
        HAT_DYNAMIC = enum.auto()
        HAT_STATIC = enum.auto()
        MLIR = enum.auto()
        DEFAULT = HAT_DYNAMIC

    class Mode(enum.Enum):
        RELEASE = "Release"
        DEBUG = "Debug"

    class Platform(enum.Enum):
        HOST = "host"
        LINUX = "linux"

    def __init__(self):
        self._functions = []
        self._description = {}

    def add(self, source, args, base_name="", parameters=None, function_opts=None, auxiliary=None):
        """Bind one function to the package; returns its full name `<base_name>_<16 hex>`
        (/root/reference/accera/python/accera/Package.py:203-259, 310-335)."""
        spec = _match(source)
        args = tuple(args)
        if set(map(id, args)) != {id(spec.A), id(spec.B), id(spec.C)} or len(args) != 3:
            raise ValueError("args must be exactly the three arrays used by the nest")
        if spec.A.element_type != spec.B.element_type:
            raise ValueError("A and B must have the same element type")
        sig = repr((base_name, [(a.role.value, a.element_type.c_name, a.shape, a.layout.name) for a in args],
                    spec.prologue, spec.prologue_arg, spec.epilogue, spec.epilogue_arg, sorted((parameters or {}).items())))
        name = f"{base_name}_{hashlib.md5(sig.encode()).hexdigest()[:16]}"
        self._functions.append(dict(name=name, base_name=base_name, spec=spec, args=args, auxiliary=auxiliary or {},
                                    parameters=parameters or {}))
        return name

    def add_description(self, author=None, license=None, other=None, version=None):
        self._description.update({k: v for k, v in dict(author=author, license=license, version=version).items() if v})
        self._description.setdefault("other", {}).update(other or {})

    def _stub_source(self):
        lines = ["/* generated by accera_amd.Package.build: HAT entry points forwarding to libaccera_mi355x.so */",
                 "#include <stdint.h>", "#include <stdio.h>", '#include "accera_mi355x_gemm.h"', ""]
        for f in self._functions:
            s = f["spec"]
            order = {id(a): n for a, n in zip(f["args"], ("a0", "a1", "a2"))}
            pa, pb, pc = order[id(s.A)], order[id(s.B)], order[id(s.C)]
            nb = s.batch if s.batch is not None else 1
            st = lambda arr: ((0,) + tuple(arr.strides))[-3:] if len(arr.strides) == 2 else tuple(arr.strides)
            (abs_, ars, acs), (bbs, brs, bcs), (cbs, crs, ccs) = st(s.A), st(s.B), st(s.C)
            call_args = (f"{s.A.element_type.lib_id}, {s.C.element_type.lib_id}, {nb}, {s.M}, {s.N}, {s.K}, "
                         f"{pa}, {abs_}, {ars}, {acs}, {pb}, {bbs}, {brs}, {bcs}, {pc}, {cbs}, {crs}, {ccs}, "
                         f"{s.prologue}, {s.prologue_arg!r}, {s.epilogue}, {s.epilogue_arg!r}")
            # (a variant recorded at build time that the library refuses at call time -- pointer alignment, a table that
            # changed under a rebuilt library -- gives way to the library's own choice)
            retry = f" if (rc == ACC950_UNSUPPORTED) rc = acc950_gemm_batched_host({call_args}, ACC950_VARIANT_AUTO, 0);" \
                if s.variant != _lib.VARIANT_AUTO else ""
            retry_dev = f" if (rc == ACC950_UNSUPPORTED) rc = acc950_gemm_batched({call_args}, ACC950_VARIANT_AUTO, 0, stream);" \
                if s.variant != _lib.VARIANT_AUTO else ""
            lines += [
                f"void {f['name']}(void* a0, void* a1, void* a2)", "{",
                f"    int rc = acc950_gemm_batched_host({call_args}, {s.variant}, 0);{retry}",
                f"    if (rc != ACC950_OK) fprintf(stderr, \"{f['name']}: %s\\n\", acc950_last_error());", "}",
                "/* same function on device pointers, asynchronous on `stream` (hipStream_t or NULL): what the record",
                f"   [device_functions.{f['name']}__gpu__] of the .hat stands for */",
                f"int {f['name']}__device(void* a0, void* a1, void* a2, void* stream)", "{",
                f"    int rc = acc950_gemm_batched({call_args}, {s.variant}, 0, stream);{retry_dev}",
                "    return rc;", "}", ""]
        return "\n".join(lines)

    def build(self, name, format=None, mode=None, platform=None, tolerance=1e-5, output_dir=None, gpu_records=False, **_):
        """Emit `<output_dir>/<name>.hat` and `<name>.so` (HAT_DYNAMIC).  Returns the list of
        files written (Package.py:551-788 returns the same kind of list): the .hat, the .so, and -- when the package
        holds functions of GPU-target plans and gpu_records is False -- `<name>_gpu.hat` as a third entry.

        `<name>.hat` is by default a plain host-convention package: every function is a cdecl symbol of `<name>.so` that
        takes host pointers, with nothing a stock loader would hand to a run-time compiler (hatlib compiles the `provider`
        of a function that `launches` a device function, /root/reference/accera/python/accera/Package.py:714-743).  The
        records the reference writes for GPU targets -- `runtime = "ROCM"` and `launches = "<fn>__gpu__"` on the function,
        a `[device_functions.<fn>__gpu__]` table with `launch_parameters`, `dynamic_shared_mem_bytes` and `provider` --
        go into the sibling `<name>_gpu.hat` over the same library, for loaders that know the provider is prebuilt
        (accera_amd.hat does).  gpu_records=True puts them into `<name>.hat` itself instead and writes no sibling.
        Functions of HOST-target plans (the quick-start form) never carry them."""
        fmt = format or Package.Format.DEFAULT
        if not (fmt & Package.Format.HAT_DYNAMIC):
            raise NotImplementedError("only Package.Format.HAT_DYNAMIC is produced by this build")
        output_dir = os.path.abspath(output_dir or os.getcwd())
        os.makedirs(output_dir, exist_ok=True)
        if not os.path.exists(_lib.LIB_PATH):
            raise RuntimeError(f"{_lib.LIB_PATH} is missing; build the kernel library first")
        c_path = os.path.join(output_dir, f"{name}.c")
        so_path = os.path.join(output_dir, f"{name}.so")
        hat_path = os.path.join(output_dir, f"{name}.hat")
        with open(c_path, "w") as f:
            f.write(self._stub_source())
        rel = os.path.relpath(_lib.LIB_DIR, output_dir)
        cmd = ["gcc", "-shared", "-fPIC", "-O2", "-o", so_path, c_path, f"-I{_lib.INCLUDE_DIR}", f"-L{_lib.LIB_DIR}",
               "-laccera_mi355x", f"-Wl,-rpath,$ORIGIN/{rel}", f"-Wl,-rpath,{_lib.LIB_DIR}"]
        subprocess.check_call(cmd)

        required_gpu = {"runtime": "ROCM", "model": "AMD MI355X", "instruction_set_version": "gfx950"}
        compiled_with = {"compiler": "hipcc (kernels), gcc (entry points)", "flags": "--offload-arch=gfx950 -O3",
                         "libraries": ["libaccera_mi355x.so"]}

        def write(path, with_gpu_records):
            functions, device_functions = self._records(with_gpu_records)
            _hat.write_hat(path, name, functions, link_target=f"{name}.so", device_functions=device_functions,
                           author=self._description.get("author", ""), version=self._description.get("version", ""),
                           license_url=self._description.get("license", ""), required_gpu=required_gpu, compiled_with=compiled_with)

        write(hat_path, gpu_records)
        files = [hat_path, so_path]
        if not gpu_records and any(f["spec"].gpu_target for f in self._functions):
            gpu_hat_path = os.path.join(output_dir, f"{name}_gpu.hat")
            write(gpu_hat_path, True)
            files.append(gpu_hat_path)
        return files

    def _records(self, gpu_records):
        """(functions, device_functions) of the .hat; gpu_records: with the GPU-target records of Package.py:714-743."""
        functions, device_functions = [], []
        for f in self._functions:
            s = f["spec"]
            arguments = []
            for a in f["args"]:
                ct = a.element_type.c_name
                arguments.append(_hat.Argument(name=a.name, declared_type=f"{ct}*", element_type=ct, usage=a.role.value,
                                               shape=list(a.shape), affine_map=list(a.strides)))
            grid, block, lds, variant = _lib.launch_geometry(s.A.element_type.lib_id, s.C.element_type.lib_id, s.M, s.N, s.K,
                                                             s.A.strides[-2:], s.B.strides[-2:], s.C.strides[-2:], s.variant)
            if s.batch is not None:
                grid = grid[:2] + [s.batch]  # the batch index is bound to grid.z
            aux = {"accera": {"base_name": f["base_name"], "parameters": {k: str(v) for k, v in f["parameters"].items()}},
                   # structural counterpart of the device-function record of the reference's GPU packages
                   # (Package.py:714-743): launch geometry of the kernel behind this entry point
                   "accera_mi355x": {"device_entry": f"{f['name']}__device", "kernel": _lib.variant_name(variant),
                                     "launch_parameters": grid + block, "dynamic_shared_mem_bytes": lds,
                                     "prologue": s.prologue, "prologue_arg": s.prologue_arg, "epilogue": s.epilogue,
                                     "epilogue_arg": s.epilogue_arg}}
            aux.update(f["auxiliary"])
            fn = _hat.Function(name=f["name"], base_name=f["base_name"], arguments=arguments, auxiliary=aux)
            if gpu_records and s.gpu_target:
                # the kernel is prebuilt: the "provider" is the kernel library, and the device function is reached through
                # the package's `<fn>__device` entry (there is no source for hatlib's run-time compiler)
                fn.runtime, fn.launches = "ROCM", f"{f['name']}__gpu__"
                device_functions.append(_hat.Function(
                    name=fn.launches, base_name=f["base_name"], arguments=arguments, calling_convention="device",
                    description=f"Device function launched by {f['name']}", launch_parameters=grid + block,
                    dynamic_shared_mem_bytes=lds, provider=os.path.basename(_lib.LIB_PATH), runtime="ROCM",
                    auxiliary={"accera_mi355x": {"kernel": _lib.variant_name(variant), "entry": f"{f['name']}__device"}}))
            functions.append(fn)
        return functions, device_functions
