"""Loads the Python-runtime library of the HIP backend and names its entry
points for compiled code.

Counterpart of the reference's loader (reference:
numba_mlir/numba_mlir/mlir/python_rt.py:9-27): the library is
``libnumba-mlir-python-runtime-hip.so`` beside the package; ``nmrtAllocMemInfo``
and the unboxer are the functions compiled code calls by name
(mlir_compiler/lib/pipelines/LowerToLlvm.cpp:869, mlir/dpctl_interop.py:236-241);
the MemInfo allocator is handed over once, at import.  Numba's NRT allocator
is used when Numba is importable; otherwise the C library's ``malloc`` (the
records are then plain heap blocks, which is all the host-side tests need).
"""

import ctypes

from .utils import load_lib

runtime_lib = ctypes.PyDLL(load_lib("numba-mlir-python-runtime-hip")._name)

# name -> address, as the JIT's symbol map wants them
SYMBOLS = {}


def _allocator_address():
    try:
        from numba.core.runtime import _nrt_python as _nrt
        return ctypes.cast(_nrt.c_helpers["Allocate"], ctypes.c_void_p).value
    except Exception:     # noqa: BLE001 -- Numba absent or of another layout
        libc = ctypes.CDLL(None)
        return ctypes.cast(libc.malloc, ctypes.c_void_p).value


def _register_funcs():
    runtime_lib.nmrtUnboxHipInterface.restype = ctypes.c_int
    runtime_lib.nmrtUnboxHipInterface.argtypes = [ctypes.py_object, ctypes.c_void_p]
    runtime_lib.nmrtAllocMemInfo.restype = ctypes.c_void_p
    runtime_lib.nmrtAllocMemInfo.argtypes = [ctypes.c_void_p, ctypes.c_size_t,
                                             ctypes.c_void_p, ctypes.c_void_p]
    runtime_lib.nmrtSetMemInfoAllocFunc.restype = None
    runtime_lib.nmrtSetMemInfoAllocFunc.argtypes = [ctypes.c_void_p]
    for name in ("nmrtAllocMemInfo", "nmrtUnboxHipInterface"):
        SYMBOLS[name] = ctypes.cast(getattr(runtime_lib, name), ctypes.c_void_p).value
    runtime_lib.nmrtSetMemInfoAllocFunc(_allocator_address())


_register_funcs()
del _register_funcs


def array_record(ndim):
    """ctypes layout of the native array record for ``ndim`` dimensions
    (Numba's arystruct_t)."""
    class ArrayRecord(ctypes.Structure):
        _fields_ = [("meminfo", ctypes.c_void_p), ("parent", ctypes.c_void_p),
                    ("nitems", ctypes.c_ssize_t), ("itemsize", ctypes.c_ssize_t),
                    ("data", ctypes.c_void_p), ("shape", ctypes.c_ssize_t * ndim),
                    ("strides", ctypes.c_ssize_t * ndim)]
    return ArrayRecord


class MemInfo(ctypes.Structure):
    """Numba's NRT MemInfo."""
    _fields_ = [("refct", ctypes.c_size_t), ("dtor", ctypes.c_void_p),
                ("dtor_info", ctypes.c_void_p), ("data", ctypes.c_void_p),
                ("size", ctypes.c_size_t), ("external_allocator", ctypes.c_void_p)]


def unbox(obj, ndim=None):
    """The native record of ``obj`` (anything with ``__hip_array_interface__``):
    what compiled code receives for the argument.  Raises what the unboxer
    set, or TypeError in the words of the reference's unboxing hook
    (dpctl_interop.py:252-259)."""
    iface = obj.__hip_array_interface__
    try:
        rank = len(iface["shape"])
    except (TypeError, KeyError):
        rank = None                # malformed: the unboxer says what is wrong
    if ndim is None:
        ndim = rank or 0
    elif rank is not None and isinstance(iface["shape"], tuple) and ndim != rank:
        # The unboxer writes 2 * rank trailing integers: a record typed for
        # another rank would be overrun or left half filled.
        raise TypeError(f"can't unbox a {rank}-dimensional array into a native "
                        f"value of {ndim} dimensions")
    record = array_record(ndim)()
    code = runtime_lib.nmrtUnboxHipInterface(obj, ctypes.byref(record))
    if code != 0:
        raise TypeError("can't unbox array from PyObject into native value.  "
                        "The object maybe of a different type")
    return record
