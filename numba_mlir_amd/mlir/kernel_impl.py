"""``@kernel`` launches on the HIP runtime.

In the reference ``Kernel.__call__`` hands the Python body to the compiler,
which wraps it in one ``_gpu_range`` loop per dimension and emits a GPU kernel
(reference: numba_mlir/numba_mlir/mlir/kernel_impl.py:97-206).  Without the
compiler the body cannot be translated, so a kernel is bound to a hand-written
gfx950 twin of the same body (``twin=`` names its symbol in the built-in
"twins" code object; ``{dtype}`` and ``{rank}`` are filled from the first
array argument).  Everything around the body is the reference's behaviour:

* launch geometry: ``grid_k = ceil(global_k / local_k)``, tail guarded
  in-kernel, dimension 0 <-> x (reference: LowerToGpu.cpp:1113-1137);
* an empty local size asks ``gpuxSuggestBlockSize`` (LowerToGpu.cpp:373-471);
* all array arguments must live on one device (dpctl_interop.py:270-275).

The index builtins exist as Python stubs only; calling them outside a kernel
is an error, as in the reference.
"""

import ctypes

import numpy as np

from . import lowered
from .device_array import HipNdArray
from .kernel_base import KernelBase
from .lowered import GPUParamDesc, lib

DEFAULT_LOCAL_SIZE = ()
LOCAL_MEM_FENCE = 1
GLOBAL_MEM_FENCE = 2

_DTYPE_TAGS = {
    np.dtype(np.int32): "i32",
    np.dtype(np.int64): "i64",
    np.dtype(np.float32): "f32",
    np.dtype(np.float64): "f64",
}


def _stub_error():
    raise NotImplementedError("This is a stub")


def get_global_id(axis):
    _stub_error()


def get_local_id(axis):
    _stub_error()


def get_group_id(axis):
    _stub_error()


def get_global_size(axis):
    _stub_error()


def get_local_size(axis):
    _stub_error()


class Stub(object):
    """Namespace of kernel-only functions; not instantiable (reference:
    numba_mlir/numba_mlir/mlir/kernel_impl.py:252-260)."""

    __slots__ = ()

    def __new__(cls):
        raise NotImplementedError("%s is not instantiable" % cls)


def _stub(name, params):
    exec(f"def {name}({params}): _stub_error()", globals())
    return globals()[name]


class atomic(Stub):
    """``atomic.add(arr, idx, val)`` / ``atomic.sub`` (kernel_impl.py:263-322)."""

    add = staticmethod(_stub("atomic_add", "arr, idx, val"))
    sub = staticmethod(_stub("atomic_sub", "arr, idx, val"))


def barrier(flags=None):
    """Work-group barrier with LOCAL_MEM_FENCE / GLOBAL_MEM_FENCE
    (kernel_impl.py:330-345)."""
    _stub_error()


def mem_fence(flags=None):
    _stub_error()


class local(Stub):
    """``local.array(shape, dtype)``: work-group memory (kernel_impl.py:366-400)."""

    array = staticmethod(_stub("local_array", "shape, dtype"))


class private(Stub):
    """``private.array(shape, dtype)``: per-work-item memory."""

    array = staticmethod(_stub("private_array", "shape, dtype"))


class group(Stub):
    """Work-group reductions (kernel_impl.py:440-482)."""

    reduce_add = staticmethod(_stub("group_reduce_add", "value"))
    reduce_mul = staticmethod(_stub("group_reduce_mul", "value"))
    reduce_min = staticmethod(_stub("group_reduce_min", "value"))
    reduce_max = staticmethod(_stub("group_reduce_max", "value"))


def kernel_func(func):
    """Device function callable from kernels (``mlir_njit(mlir_force_inline=
    True)`` in the reference, kernel_impl.py:209); a plain function here, the
    twin inlines it by construction."""
    return func


def check_device_args(args):
    """All device arrays of a launch must share a queue."""
    ctx = None
    for a in args:
        if isinstance(a, HipNdArray):
            if ctx is None:
                ctx = a.ctx
            elif a.ctx is not ctx:
                raise ValueError(
                    f"Device arrays must share a device: {ctx.device} and "
                    f"{a.ctx.device}")
    if ctx is None:
        raise ValueError("A kernel launch needs at least one device array")
    return ctx


class _ParamList:
    """Builds the GPUParamDesc array the compiled host code would build
    (reference: mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:444-628)."""

    def __init__(self):
        self._slots = []

    def _add(self, cvalue, ptype):
        self._slots.append((cvalue, ptype))

    def add_array(self, arr):
        self._add(ctypes.c_void_p(arr.ptr), lowered.PARAM_PTR)
        for n in arr.shape:
            self._add(ctypes.c_int64(n), lowered.PARAM_INT64)
        for s in arr.elem_strides:
            self._add(ctypes.c_int64(s), lowered.PARAM_INT64)

    def add_local(self, nbytes):
        self._slots.append((None, nbytes))

    def add_scalar(self, value):
        if isinstance(value, (bool, np.bool_)):
            self._add(ctypes.c_bool(bool(value)), lowered.PARAM_BOOL)
        elif isinstance(value, (int, np.integer)) and not isinstance(
                value, np.int32):
            self._add(ctypes.c_int64(int(value)), lowered.PARAM_INT64)
        elif isinstance(value, np.int32):
            self._add(ctypes.c_int32(int(value)), lowered.PARAM_INT32)
        elif isinstance(value, np.float32):
            self._add(ctypes.c_float(float(value)), lowered.PARAM_FLOAT32)
        elif isinstance(value, (float, np.floating)):
            self._add(ctypes.c_double(float(value)), lowered.PARAM_FLOAT64)
        else:
            raise TypeError(f"Unsupported kernel argument type: {type(value)}")

    def build(self):
        descs = (GPUParamDesc * (len(self._slots) + 1))()
        for i, (cvalue, ptype) in enumerate(self._slots):
            if cvalue is None:     # workgroup memory: data == NULL, size = bytes
                descs[i].data = None
                descs[i].size = ptype
                descs[i].type = lowered.PARAM_PTR
                continue
            descs[i].data = ctypes.cast(ctypes.pointer(cvalue), ctypes.c_void_p)
            descs[i].size = ctypes.sizeof(cvalue)
            descs[i].type = ptype
        descs[len(self._slots)].data = None
        descs[len(self._slots)].size = 0
        descs[len(self._slots)].type = lowered.PARAM_NULL
        return descs


class Kernel(KernelBase):
    def __init__(self, func, kwargs):
        super().__init__(func)
        self.twin = kwargs.get("twin")
        # local.array sizes of the body in bytes: a list, or a callable
        # (global_size, local_size) -> list.  Each becomes a workgroup-memory
        # parameter after the user arguments (GpuRuntimeToLlvm.cpp:507-536).
        self.local_bytes = kwargs.get("local_bytes", ())
        self.last_launch = None

    def _twin_name(self, args):
        if self.twin is None:
            raise NotImplementedError(
                f"@kernel '{self.py_func.__name__}' has no hand-written gfx950 "
                "twin; compiling arbitrary kernel bodies needs the ROCDL "
                "lowering of the compiler")
        first = next((a for a in args if isinstance(a, HipNdArray)), None)
        tag = _DTYPE_TAGS.get(first.dtype) if first is not None else None
        return self.twin.format(dtype=tag, rank=len(self.global_size))

    def __call__(self, *args, **kwargs):
        self.check_call_args(args, kwargs)
        ctx = check_device_args(args)

        ndim = len(self.global_size)
        assert 1 <= ndim <= 3, f"Invalid dim count: {ndim}"
        name = self._twin_name(args)

        if len(self.local_size) != 0:
            block = list(self.local_size)
        else:
            gsize = (ctypes.c_uint32 * ndim)(*[min(int(g), 0xFFFFFFFF)
                                               for g in self.global_size])
            bsize = (ctypes.c_uint32 * ndim)()
            lib.nmhipSuggestBlockSize(ctx.handle, name.encode(), gsize, bsize,
                                      ndim)
            block = list(bsize)
        block += [1] * (3 - ndim)
        gsize3 = [int(g) for g in self.global_size] + [1] * (3 - ndim)
        grid = [(g + b - 1) // b for g, b in zip(gsize3, block)]

        params = _ParamList()
        for a in args:
            if isinstance(a, HipNdArray):
                params.add_array(a)
            else:
                params.add_scalar(a)
        local_bytes = self.local_bytes
        if callable(local_bytes):
            local_bytes = local_bytes(tuple(gsize3[:ndim]), tuple(block[:ndim]))
        for nbytes in local_bytes:
            params.add_local(int(nbytes))
        for g in gsize3:
            params.add_scalar(int(g))
        descs = params.build()

        self.last_launch = {"kernel": name, "grid": tuple(grid),
                            "block": tuple(block)}
        lib.nmhipLaunch(ctx.handle, name.encode(),
                        (ctypes.c_size_t * 3)(*grid),
                        (ctypes.c_size_t * 3)(*block), descs)


def kernel(func=None, **kwargs):
    if func is None:

        def wrapper(f):
            return Kernel(f, kwargs)

        return wrapper
    return Kernel(func, kwargs)
