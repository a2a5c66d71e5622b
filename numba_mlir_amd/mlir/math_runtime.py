"""Loads the HIP math runtime and registers the device gemm entry points.

Counterpart of the reference's math-runtime loader (reference:
numba_mlir/numba_mlir/mlir/math_runtime.py:10-49): the library is initialised
with ``nmrtMathRuntimeInit`` at import, finalised at exit, and
``mkl_gemm_<dtype>_device`` are registered under their ``_mlir_ciface_`` names.
"""

import atexit
import ctypes

from .utils import load_lib, mlir_func_name

runtime_hip_lib = load_lib("numba-mlir-math-hip-runtime")

_init_hip_func = runtime_hip_lib.nmrtMathRuntimeInit
_init_hip_func.restype = None
_init_hip_func()

DEVICE_GEMM_SUFFIXES = ["float32", "float64"]

runtime_hip_lib.nmhipMathLastKernel.restype = ctypes.c_char_p


def load_function_variants(runtime_lib, func_name, suffixes, register_cfunc):
    for s in suffixes:
        name = func_name % s
        func = getattr(runtime_lib, name)
        register_cfunc(mlir_func_name(name),
                       ctypes.cast(func, ctypes.c_void_p).value)


def register_funcs(register_cfunc):
    load_function_variants(runtime_hip_lib, "mkl_gemm_%s_device",
                           DEVICE_GEMM_SUFFIXES, register_cfunc)


def last_kernel():
    return runtime_hip_lib.nmhipMathLastKernel().decode()


_finalize_hip_func = runtime_hip_lib.nmrtMathRuntimeFinalize
_finalize_hip_func.restype = None


@atexit.register
def _cleanup():
    _finalize_hip_func()
