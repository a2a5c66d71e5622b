"""Device arrays for the HIP backend.

The reference takes its device arrays from dpctl (``usm_ndarray``; typing and
unboxing in reference: numba_mlir/numba_mlir/mlir/dpctl_interop.py:77-262,
numba_mlir/numba_mlir/python_runtime/lib/Boxing.cpp:45-136).  ``HipNdArray`` is
the analogue for HIP: a strided view over memory obtained from ``gpuxAlloc``,
carrying the queue it belongs to, exposing ``__hip_array_interface__`` with the
fields of ``__sycl_usm_array_interface__`` (data, shape, strides, typestr,
version, syclobj -> queue), and released through ``gpuxDeAlloc`` when the last
view dies, as the reference's NRT MemInfo destructor does
(reference: mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:717-720).
"""

import ctypes
import math
import weakref

import numpy as np

from . import gpu_runtime, lowered
from .lowered import lib
from .utils import readenv

DEFAULT_DEVICE = readenv("NUMBA_MLIR_DEFAULT_DEVICE", str, "hip:gpu:0")

_USM_TYPES = {
    "device": lowered.ALLOC_DEVICE,
    "shared": lowered.ALLOC_SHARED,
    "host": lowered.ALLOC_HOST,
}


class Context:
    """Queue plus cached module/kernel handles of one device string.

    Counterpart of the per-function context the reference's compiled code
    obtains from ``nmrtTakeContext`` (reference:
    numba_mlir_runtime/lib/Context.cpp:25-60): created on first use, reused by
    every later call, purged at interpreter exit.
    """

    def __init__(self, device):
        self.device = device
        self.handle = lib.nmhipContextCreate(device.encode() if device else None)
        self._finalizer = weakref.finalize(self, lib.nmhipContextDestroy,
                                           self.handle)
        # events of launches enqueued from Python and not yet retired, oldest
        # first (kernel_impl.LaunchPlan.enqueue / retire)
        self.pending = []

    @property
    def queue(self):
        return lib.nmhipContextQueue(self.handle)

    def set_async(self, flag):
        lib.nmhipContextSetAsync(self.handle, 1 if flag else 0)

    def synchronize(self):
        """Returns when everything submitted through this context is done:
        the library's own launches and the launches enqueued from Python (the
        queue is in order, so waiting for the youngest of those covers all;
        their events stay the caller's to retire)."""
        lib.nmhipContextSynchronize(self.handle)
        pending = self.pending
        if pending:
            gpu_runtime.runtime_lib.gpuxWait(self.queue, pending[-1])

    def last_kernel(self):
        return lib.nmhipLastKernelName(self.handle).decode()


_contexts = {}


def get_context(device=None):
    device = DEFAULT_DEVICE if device is None else device
    ctx = _contexts.get(device)
    if ctx is None:
        ctx = _contexts[device] = Context(device)
    return ctx


class DeviceCaps:
    """Capabilities the compiler asks of a device (reference:
    dpctl_interop.py:148-209, 293-306): MI355X has native fp64 and fp16."""

    def __init__(self, filter_string):
        self.filter_string = filter_string
        self.arch = "gfx950"
        self.has_fp64 = True
        self.has_fp16 = True
        self.subgroup_size = 64


def get_default_device():
    return DeviceCaps(DEFAULT_DEVICE)


def _dense_strides(shape, itemsize, order="C"):
    """Byte strides of a dense array (NumPy reports zeros for empty arrays)."""
    strides = [0] * len(shape)
    step = itemsize
    dims = range(len(shape) - 1, -1, -1) if order == "C" else range(len(shape))
    for i in dims:
        strides[i] = step
        step *= max(int(shape[i]), 1)
    return tuple(strides)


class _Buffer:
    """Owner of one gpuxAlloc allocation."""

    def __init__(self, ctx, nbytes, usm_type):
        self.ctx = ctx
        self.nbytes = nbytes
        self.usm_type = usm_type
        self.ptr = lib.nmhipAlloc(ctx.handle, max(nbytes, 1), _USM_TYPES[usm_type])
        self._finalizer = weakref.finalize(self, lib.nmhipFree, ctx.handle,
                                           self.ptr)


class HipNdArray:
    def __init__(self, buffer, shape, dtype, strides, offset):
        self._buffer = buffer
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.strides = tuple(int(s) for s in strides)  # bytes, as NumPy
        self._offset = int(offset)                      # bytes

    # -- construction --------------------------------------------------------
    @classmethod
    def empty(cls, shape, dtype, usm_type="device", device=None, order="C"):
        if isinstance(shape, int):
            shape = (shape,)
        dtype = np.dtype(dtype)
        ctx = get_context(device)
        count = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
        buf = _Buffer(ctx, count * dtype.itemsize, usm_type)
        return cls(buf, shape, dtype, _dense_strides(shape, dtype.itemsize, order),
                   0)

    @classmethod
    def from_numpy(cls, arr, usm_type="device", device=None):
        arr = np.asarray(arr)
        order = "F" if (arr.flags["F_CONTIGUOUS"] and not
                        arr.flags["C_CONTIGUOUS"]) else "C"
        host = np.asarray(arr, order=order)
        if not (host.flags["C_CONTIGUOUS"] or host.flags["F_CONTIGUOUS"]):
            host = np.ascontiguousarray(host)
            order = "C"
        res = cls.empty(host.shape, host.dtype, usm_type, device, order)
        if host.nbytes:
            lib.nmhipMemcpyHtoD(res.ctx.handle, res.ptr,
                                host.ctypes.data_as(ctypes.c_void_p), host.nbytes)
        return res

    # -- properties ----------------------------------------------------------
    @property
    def ctx(self):
        return self._buffer.ctx

    @property
    def usm_type(self):
        return self._buffer.usm_type

    @property
    def ptr(self):
        return self._buffer.ptr + self._offset

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        return math.prod(self.shape)

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    @property
    def elem_strides(self):
        return tuple(s // self.dtype.itemsize for s in self.strides)

    @property
    def T(self):
        return HipNdArray(self._buffer, self.shape[::-1], self.dtype,
                          self.strides[::-1], self._offset)

    def transpose(self, *axes):
        """numpy.transpose: a view with the dimensions permuted (reversed
        when no permutation is given)."""
        if len(axes) == 1 and (axes[0] is None or isinstance(axes[0], (tuple, list))):
            axes = axes[0]
        if not axes:
            return self.T
        axes = [int(a) + self.ndim if int(a) < 0 else int(a) for a in axes]
        if sorted(axes) != list(range(self.ndim)):
            raise ValueError("axes don't match array")
        return HipNdArray(self._buffer, [self.shape[a] for a in axes], self.dtype,
                          [self.strides[a] for a in axes], self._offset)

    def __len__(self):
        if not self.shape:
            raise TypeError("len() of a 0-d device array")
        return self.shape[0]

    def broadcast_to(self, shape):
        """Read-only style view with stride 0 along broadcast dimensions
        (NumPy's rules: trailing dimensions align, extents are equal or 1)."""
        shape = tuple(int(n) for n in shape)
        if len(shape) < self.ndim:
            raise ValueError(f"cannot broadcast {self.shape} to {shape}")
        pad = len(shape) - self.ndim
        strides = [0] * pad
        for n, st, want in zip(self.shape, self.strides, shape[pad:]):
            if n == want:
                strides.append(st)
            elif n == 1:
                strides.append(0)
            else:
                raise ValueError(f"cannot broadcast {self.shape} to {shape}")
        return HipNdArray(self._buffer, shape, self.dtype, strides, self._offset)

    def __getitem__(self, key):
        """Basic indexing (integers and slices): a view of the same
        allocation, as ``usm_ndarray`` gives."""
        if not isinstance(key, tuple):
            key = (key,)
        if len(key) > self.ndim:
            raise IndexError("too many indices for device array")
        shape, strides, offset = [], [], self._offset
        for dim, k in enumerate(key):
            n, st = self.shape[dim], self.strides[dim]
            if isinstance(k, slice):
                start, stop, step = k.indices(n)
                shape.append(len(range(start, stop, step)))
                strides.append(st * step)
                offset += start * st
            elif isinstance(k, (int, np.integer)):
                k = int(k)
                if not -n <= k < n:
                    raise IndexError(f"index {k} is out of bounds for axis {dim} "
                                     f"with size {n}")
                offset += (k % n) * st
            else:
                raise IndexError("only integers and slices index a device array")
        shape += self.shape[len(key):]
        strides += self.strides[len(key):]
        return HipNdArray(self._buffer, shape, self.dtype, strides, offset)

    @property
    def __hip_array_interface__(self):
        return {
            "data": (self.ptr, False),
            "shape": self.shape,
            # in elements, None for a dense row-major array: the convention
            # of __sycl_usm_array_interface__, which the unboxer follows
            "strides": None if self.is_c_contiguous() else self.elem_strides,
            "typestr": self.dtype.str,
            "version": 1,
            "queue": self.ctx.queue,
            "usm_type": self.usm_type,
        }

    def is_c_contiguous(self):
        if self.size == 0:
            return True
        expect = self.dtype.itemsize
        for n, s in zip(reversed(self.shape), reversed(self.strides)):
            if n != 1 and s != expect:
                return False
            expect *= n
        return True

    def is_f_contiguous(self):
        return self.T.is_c_contiguous()

    def reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        if not self.is_c_contiguous():
            raise ValueError("reshape needs a C-contiguous device array")
        shape = tuple(int(n) for n in shape)
        if shape.count(-1) == 1:              # one extent left to be worked out
            known = math.prod(n for n in shape if n != -1)
            if known == 0 or self.size % known:
                raise ValueError(f"cannot reshape array of size {self.size} into shape {shape}")
            shape = tuple(self.size // known if n == -1 else n for n in shape)
        if any(n < 0 for n in shape):
            raise ValueError("negative dimensions are not allowed")
        strides = _dense_strides(shape, self.dtype.itemsize)
        if math.prod(int(n) for n in shape) != self.size:
            raise ValueError("cannot reshape: size mismatch")
        return HipNdArray(self._buffer, shape, self.dtype, strides, self._offset)

    # -- host transfer -------------------------------------------------------
    def asnumpy(self):
        """Copies the viewed elements back into a new NumPy array."""
        self.ctx.synchronize()
        if self.size == 0:
            return np.empty(self.shape, self.dtype)
        if self.is_c_contiguous() or self.is_f_contiguous():
            order = "C" if self.is_c_contiguous() else "F"
            out = np.empty(self.shape, self.dtype, order=order)
            lib.nmhipMemcpyDtoH(self.ctx.handle,
                                out.ctypes.data_as(ctypes.c_void_p), self.ptr,
                                out.nbytes)
            return out
        # Strided view: fetch the whole allocation and view it on the host.
        raw = np.empty(self._buffer.nbytes, np.uint8)
        lib.nmhipMemcpyDtoH(self.ctx.handle, raw.ctypes.data_as(ctypes.c_void_p),
                            self._buffer.ptr, raw.nbytes)
        view = np.ndarray(self.shape, self.dtype, raw.data, self._offset,
                          self.strides)
        return view.copy()

    def copy_from_host(self, arr):
        arr = np.ascontiguousarray(arr, dtype=self.dtype)
        if arr.shape != self.shape or not self.is_c_contiguous():
            raise ValueError("copy_from_host needs a C-contiguous array of the "
                             "same shape")
        if arr.nbytes:
            lib.nmhipMemcpyHtoD(self.ctx.handle, self.ptr,
                                arr.ctypes.data_as(ctypes.c_void_p), arr.nbytes)

    def as_host_view(self):
        """NumPy view of a shared/host allocation (host-dereferenceable, as the
        reference's results over shared USM are, dpctl_interop.py:113-115)."""
        if self.usm_type == "device":
            raise ValueError("device allocations are not host-dereferenceable")
        self.ctx.synchronize()
        buf = (ctypes.c_uint8 * max(self._buffer.nbytes, 1)).from_address(
            self._buffer.ptr)
        view = np.ndarray(self.shape, self.dtype, buf, self._offset, self.strides)
        view.flags.writeable = True
        self._host_keepalive = buf
        return view

    def __repr__(self):
        return (f"HipNdArray(shape={self.shape}, dtype={self.dtype}, "
                f"usm_type={self.usm_type!r})")


def asarray(arr, usm_type="device", device=None):
    if isinstance(arr, HipNdArray):
        return arr
    return HipNdArray.from_numpy(arr, usm_type, device)


def asnumpy(arr):
    return arr.asnumpy() if isinstance(arr, HipNdArray) else np.asarray(arr)


def empty(shape, dtype, usm_type="device", device=None):
    return HipNdArray.empty(shape, dtype, usm_type, device)


def disjoint(arrays):
    """True when no two of the device arrays share a byte (then the kernel may
    reorder their loads and stores freely)."""
    spans = []
    for a in arrays:
        lo = hi = a.ptr
        for n, st in zip(a.shape, a.strides):
            if n == 0:
                lo = hi = a.ptr
                break
            if st >= 0:
                hi += (n - 1) * st
            else:
                lo += (n - 1) * st
        spans.append((lo, hi + a.dtype.itemsize))
    spans.sort()
    return all(spans[k][1] <= spans[k + 1][0] for k in range(len(spans) - 1))


STREAM_BYTES = 128 << 20


def streams(arrays):
    """True when the device arrays of a launch are too large to stay in the
    256 MiB memory-side cache from one launch to the next: generated kernels
    then read and write them with streaming accesses."""
    total = 0
    for a in arrays:
        total += a.size * a.dtype.itemsize
    return total >= STREAM_BYTES
