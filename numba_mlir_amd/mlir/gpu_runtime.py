"""Selects and loads the GPU runtime library and registers its entry points.

Counterpart of the reference's loader (reference:
numba_mlir/numba_mlir/mlir/gpu_runtime.py:14-82).  ``NUMBA_MLIR_GPU_RUNTIME``
picks the library ``numba-mlir-gpu-runtime-<kind>``; the kind this package
ships is ``"hip"``.  The thirteen ``gpux*`` names are resolved and handed to
the lowered host code's symbol table, which is what ``register_cfunc`` does
for JIT'd code in the reference.  Unlike the reference (which binds missing
names to a dummy address and logs a load failure), a missing library or a
missing ``gpux*`` symbol is an error here: there is no other backend to fall
back to.
"""

import ctypes

from .utils import load_lib, readenv

GPU_RUNTIME = readenv("NUMBA_MLIR_GPU_RUNTIME", str, "hip")

# gpu_runtime.py:35-56 of the reference (gpuxDuplicateQueue included).
GPUX_FUNCS = [
    "gpuxAlloc",
    "gpuxDeAlloc",
    "gpuxKernelDestroy",
    "gpuxKernelGet",
    "gpuxLaunchKernel",
    "gpuxModuleDestroy",
    "gpuxModuleLoad",
    "gpuxQueueCreate",
    "gpuxQueueDestroy",
    "gpuxSuggestBlockSize",
    "gpuxWait",
    "gpuxDestroyEvent",
    "gpuxDuplicateQueue",
]


def _get_gpu_runtime_name():
    if GPU_RUNTIME == "hip":
        return "numba-mlir-gpu-runtime-hip"

    raise ValueError(f'Invalid GPU runtime type: "{GPU_RUNTIME}", expected "hip"')


class GPUParamDesc(ctypes.Structure):
    """GPUParamDesc of the C-ABI: {const void* data; int32 size; int32 type}."""

    _fields_ = [
        ("data", ctypes.c_void_p),
        ("size", ctypes.c_int32),
        ("type", ctypes.c_int32),
    ]


class GPUAllocResult(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("event", ctypes.c_void_p)]


def _declare(lib):
    vp, sz = ctypes.c_void_p, ctypes.c_size_t
    lib.gpuxQueueCreate.restype = vp
    lib.gpuxQueueCreate.argtypes = [ctypes.c_char_p]
    lib.gpuxQueueDestroy.restype = None
    lib.gpuxQueueDestroy.argtypes = [vp]
    lib.gpuxModuleLoad.restype = vp
    lib.gpuxModuleLoad.argtypes = [vp, vp, sz]
    lib.gpuxModuleDestroy.restype = None
    lib.gpuxModuleDestroy.argtypes = [vp]
    lib.gpuxKernelGet.restype = vp
    lib.gpuxKernelGet.argtypes = [vp, ctypes.c_char_p]
    lib.gpuxKernelDestroy.restype = None
    lib.gpuxKernelDestroy.argtypes = [vp]
    lib.gpuxLaunchKernel.restype = vp
    lib.gpuxLaunchKernel.argtypes = [vp, vp, sz, sz, sz, sz, sz, sz, vp, vp]
    lib.gpuxWait.restype = None
    lib.gpuxWait.argtypes = [vp, vp]
    lib.gpuxDestroyEvent.restype = None
    lib.gpuxDestroyEvent.argtypes = [vp, vp]
    lib.gpuxAlloc.restype = None
    lib.gpuxAlloc.argtypes = [vp, sz, sz, ctypes.c_int, vp,
                              ctypes.POINTER(GPUAllocResult)]
    lib.gpuxDeAlloc.restype = None
    lib.gpuxDeAlloc.argtypes = [vp, vp]
    lib.gpuxSuggestBlockSize.restype = None
    lib.gpuxSuggestBlockSize.argtypes = [vp, vp, ctypes.POINTER(ctypes.c_uint32),
                                         ctypes.POINTER(ctypes.c_uint32), sz]
    lib.gpuxDuplicateQueue.restype = vp
    lib.gpuxDuplicateQueue.argtypes = [vp]


runtime_lib = load_lib(_get_gpu_runtime_name())
IS_GPU_RUNTIME_AVAILABLE = True

for _name in GPUX_FUNCS:
    if not hasattr(runtime_lib, _name):
        raise ImportError(
            f"GPU runtime {_get_gpu_runtime_name()} does not export {_name}")
_declare(runtime_lib)


def register_funcs(register_cfunc):
    """Hands every gpux* address to ``register_cfunc(name, address)``."""
    for name in GPUX_FUNCS:
        func = getattr(runtime_lib, name)
        register_cfunc(name, ctypes.cast(func, ctypes.c_void_p).value)
