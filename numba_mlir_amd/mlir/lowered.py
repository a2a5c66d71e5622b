"""ctypes binding of the lowered host code (libnumba-mlir-hip-offload.so).

Importing this module does what importing ``numba_mlir`` does in the reference
(reference: numba_mlir/numba_mlir/mlir/lowering.py:23-26): it loads the runtime
libraries and registers their entry points for the compiled host code.  Here
the compiled host code is the offload library, and registration goes through
its ``nmhipRegisterSymbol`` (reference: ``register_cfunc``,
numba_mlir/numba_mlir/mlir/utils.py:63-68).
"""

import ctypes

from . import gpu_runtime, math_runtime
from .gpu_runtime import GPUParamDesc
from .utils import load_lib

lib = load_lib("numba-mlir-hip-offload")

_vp, _sz, _i64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int64
_i64x2 = ctypes.c_int64 * 2

_SIGNATURES = {
    "nmhipRegisterSymbol": (ctypes.c_int, [ctypes.c_char_p, _vp]),
    "nmhipContextCreate": (_vp, [ctypes.c_char_p]),
    "nmhipContextDestroy": (None, [_vp]),
    "nmhipContextSetAsync": (None, [_vp, ctypes.c_int]),
    "nmhipContextSynchronize": (None, [_vp]),
    "nmhipContextQueue": (_vp, [_vp]),
    "nmhipLastKernelName": (ctypes.c_char_p, [_vp]),
    "nmhipAlloc": (_vp, [_vp, _sz, ctypes.c_int]),
    "nmhipFree": (None, [_vp, _vp]),
    "nmhipMemcpyHtoD": (None, [_vp, _vp, _vp, _sz]),
    "nmhipMemcpyDtoH": (None, [_vp, _vp, _vp, _sz]),
    "nmhipCopy": (None, [_vp, _vp, _vp, _sz]),
    "nmhipMapBinary": (None, [_vp, ctypes.c_int, ctypes.c_int, _vp, _i64x2, _vp,
                              _i64x2, _vp, _i64x2, _i64, _i64]),
    "nmhipBlackScholesF32": (None, [_vp, _vp, _vp, _vp, ctypes.c_float,
                                    ctypes.c_float, _vp, _vp, _i64,
                                    ctypes.c_int]),
    "nmhipReduce": (None, [_vp, ctypes.c_int, ctypes.c_int, _vp, _i64, _i64, _i64,
                           _i64, ctypes.c_int, _vp]),
    "nmhipNorm2F32": (None, [_vp, _vp, _i64, _vp]),
    "nmhipNorm2RowsF32": (None, [_vp, _vp, _i64, _i64, _i64, _vp]),
    "nmhipGemm": (None, [_vp, ctypes.c_int, _vp, _i64x2, _vp, _i64x2, _vp, _i64x2,
                         _i64, _i64, _i64, ctypes.c_double, ctypes.c_double]),
    "nmhipSuggestBlockSize": (None, [_vp, ctypes.c_char_p,
                                     ctypes.POINTER(ctypes.c_uint32),
                                     ctypes.POINTER(ctypes.c_uint32), _sz]),
    "nmhipLaunch": (None, [_vp, ctypes.c_char_p, ctypes.POINTER(_sz),
                           ctypes.POINTER(_sz), ctypes.POINTER(GPUParamDesc)]),
    "nmhipPairwiseF64": (None, [_vp, _vp, _vp, _vp, _i64, _i64]),
    "nmhipKernelBlob": (_vp, [ctypes.c_char_p, ctypes.POINTER(_sz)]),
    "nmhipSetTuning": (None, [ctypes.c_char_p, _i64]),
}

for _name, (_res, _args) in _SIGNATURES.items():
    _f = getattr(lib, _name)
    _f.restype = _res
    _f.argtypes = _args

_registered_cfuncs = []


def register_cfunc(name, address):
    _registered_cfuncs.append((name, address))
    if lib.nmhipRegisterSymbol(name.encode(), address) != 0:
        raise ImportError(f"lowered host code does not use symbol {name}")


gpu_runtime.register_funcs(register_cfunc)
math_runtime.register_funcs(register_cfunc)

# dtype / op codes of include/numba_mlir_hip/Offload.h
I32, I64, F32, F64 = 0, 1, 2, 3
ADD, SUB, MUL, DIV = 0, 1, 2, 3
SUM, PROD, MIN, MAX = 0, 1, 2, 3
ALLOC_DEVICE, ALLOC_SHARED, ALLOC_LOCAL, ALLOC_HOST = 0, 1, 2, 3

# GpuParamType codes of include/numba_mlir_hip/GpuRuntime.h
PARAM_NULL, PARAM_BOOL, PARAM_INT8, PARAM_INT16, PARAM_INT32 = 0, 1, 2, 3, 4
PARAM_INT64, PARAM_FLOAT32, PARAM_FLOAT64, PARAM_PTR = 5, 6, 7, 8


def kernel_blob(family):
    size = _sz(0)
    ptr = lib.nmhipKernelBlob(family.encode(), ctypes.byref(size))
    return ctypes.string_at(ptr, size.value)


def set_tuning(knob, value):
    lib.nmhipSetTuning(knob.encode(), int(value))
