"""accera_amd: MI355X-native (gfx950) kernels for Accera's matmul + fused-ReLU GPU path,
delivered behind the HAT package boundary.

Sub-modules
  _lib      ctypes binding of the C ABI (libaccera_mi355x.so)
  gemm      device-tensor entry point (torch for memory and streams only)
  hat       .hat writer, hatlib-style loader and run_benchmark
  lang      the slice of Accera's Python DSL that describes this path
            (Array, Nest, fuse, Plan.tensorize/cache/bind, Package.add/build)
"""
from . import _lib  # noqa: F401
from ._lib import (Acc950Error, EPILOGUE_NONE, EPILOGUE_RELU, EPILOGUE_RELU_NOCOND, EPILOGUE_SCALE, EPILOGUE_SET,  # noqa: F401
                   PROLOGUE_NONE, PROLOGUE_SCALE, PROLOGUE_SET, PROLOGUE_SET0, VARIANT_AUTO, VARIANT_F32_MFMA, VARIANT_GENERIC, VARIANT_SKINNY_BASE)

__all__ = ["gemm_relu", "GemmCall", "hat"]


def __getattr__(name):
    # torch and the DSL are imported on first use so that `import accera_amd` stays light
    if name in ("gemm_relu", "GemmCall"):
        from . import gemm
        return getattr(gemm, name)
    if name == "hat":
        import importlib
        return importlib.import_module(".hat", __name__)
    if name in _LANG_NAMES:
        import importlib
        return getattr(importlib.import_module(".lang", __name__), name)
    raise AttributeError(name)


_LANG_NAMES = {"Array", "Role", "ScalarType", "Nest", "fuse", "Package", "Target", "MMAShape", "MMAFragmentOp",
               "MMASchedulingPolicy", "CacheStrategy", "max", "min", "cast", "Schedule", "Plan", "Cache", "AUTO"}
