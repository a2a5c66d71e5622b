"""NumPy-level entry points of the offloaded hot path.

Each function stands for what the reference compiles an ``@njit`` function
calling the same NumPy primitive on device arrays into: dtype and shape rules
follow the reference's op catalogue
(reference: numba_mlir/numba_mlir/mlir/numpy/funcs.py), the work is done by
the lowered host code behind the gpux* C-ABI.
"""

import numpy as np

from . import lowered
from .device_array import HipNdArray, asarray, empty
from .lowered import lib

_DTYPES = {
    np.dtype(np.int32): lowered.I32,
    np.dtype(np.int64): lowered.I64,
    np.dtype(np.float32): lowered.F32,
    np.dtype(np.float64): lowered.F64,
}


def _code(dtype):
    try:
        return _DTYPES[np.dtype(dtype)]
    except KeyError:
        raise TypeError(f"dtype {dtype} is not supported by the HIP kernels")


def _i64x2(a, b):
    return (lowered.ctypes.c_int64 * 2)(int(a), int(b))


def _as_2d(arr, shape2):
    """Element strides of ``arr`` broadcast to the 2-D iteration space
    ``shape2``; a broadcast dimension gets stride 0 (reference:
    mlir/lib/Conversion/NtensorToLinalg.cpp:487-557)."""
    shape = (1,) * (2 - arr.ndim) + arr.shape
    strides = (0,) * (2 - arr.ndim) + arr.elem_strides
    out = []
    for n, s, full in zip(shape, strides, shape2):
        if n == full:
            out.append(s if n != 1 else 0)
        elif n == 1:
            out.append(0)
        else:
            raise ValueError(f"operands could not be broadcast: {arr.shape} "
                             f"into {shape2}")
    return out


def _binary(op, a, b, out=None):
    a, b = asarray(a), asarray(b)
    if a.ndim > 2 or b.ndim > 2:
        raise NotImplementedError("maps are implemented for rank <= 2")
    # numpy.add etc.: operands are converted to the promoted dtype before the
    # generic (linalg_builder.py:297-305, broadcast_type 261-275).
    dtype = np.promote_types(a.dtype, b.dtype)
    if a.dtype != dtype or b.dtype != dtype:
        raise NotImplementedError("mixed-dtype maps need a convert kernel")
    res_shape = np.broadcast_shapes(a.shape, b.shape)
    if out is None:
        out = empty(res_shape, dtype, usm_type=a.usm_type, device=a.ctx.device)
    elif out.shape != tuple(res_shape) or out.dtype != dtype:
        raise ValueError("out has the wrong shape or dtype")
    shape2 = (1,) * (2 - len(res_shape)) + tuple(res_shape)
    sa, sb, so = _as_2d(a, shape2), _as_2d(b, shape2), _as_2d(out, shape2)
    # A size-1 output dimension still needs its real stride: recompute.
    so = list((0,) * (2 - out.ndim) + out.elem_strides)
    lib.nmhipMapBinary(a.ctx.handle, op, _code(dtype), a.ptr, _i64x2(*sa), b.ptr,
                       _i64x2(*sb), out.ptr, _i64x2(*so), shape2[0], shape2[1])
    return out


def add(a, b, out=None):
    """numpy.add (reference: numpy/funcs.py:457-462)."""
    return _binary(lowered.ADD, a, b, out)


def subtract(a, b, out=None):
    return _binary(lowered.SUB, a, b, out)


def multiply(a, b, out=None):
    return _binary(lowered.MUL, a, b, out)


def divide(a, b, out=None):
    """numpy.divide of two float32 or two float64 arrays (integer operands
    give float64: not a same-type map)."""
    if np.dtype(asarray(a).dtype).kind != "f":
        raise NotImplementedError("true division of integers yields float64")
    return _binary(lowered.DIV, a, b, out)


def black_scholes(price, strike, t, rate, volatility, call, put,
                  float64_literals=True):
    """The fused Black-Scholes body of the reference's test
    (reference: numba_mlir/numba_mlir/mlir/tests/test_numpy.py:2827-2852);
    writes ``call`` and ``put`` in place.

    ``float64_literals=True`` types the Python literals as float64, as the
    reference does; ``False`` evaluates everything in float32.
    """
    arrs = [price, strike, t, call, put]
    n = price.size
    for x in arrs:
        if x.dtype != np.float32 or x.ndim != 1 or x.size != n or \
                not x.is_c_contiguous():
            raise ValueError("black_scholes needs 1-D contiguous float32 arrays "
                             "of one length")
    lib.nmhipBlackScholesF32(price.ctx.handle, price.ptr, strike.ptr, t.ptr,
                             float(np.float32(rate)),
                             float(np.float32(volatility)), call.ptr, put.ptr, n,
                             1 if float64_literals else 0)


def _reduce(op, x, axis, result_dtype=None):
    x = asarray(x)
    if x.ndim == 1:
        x2 = HipNdArray(x._buffer, (1,) + x.shape, x.dtype, (0,) + x.strides,
                        x._offset)
        if axis in (0, -1):
            axis = None
    elif x.ndim == 2:
        x2 = x
    else:
        raise NotImplementedError("reductions are implemented for rank <= 2")
    if axis is not None:
        if axis < 0:
            axis += 2
        if axis not in (0, 1):
            raise ValueError("axis out of range")
    # Integer reductions accumulate and return int64 (promote_int,
    # numpy/funcs.py:120-123, 176, 210); a full reduction is cast back to the
    # input dtype (185).
    is_int = np.issubdtype(x.dtype, np.integer)
    acc_dtype = np.dtype(np.int64) if is_int else x.dtype
    n0, n1 = x2.shape
    s0, s1 = x2.elem_strides
    if axis is None:
        out = empty((1,), acc_dtype, usm_type="device", device=x.ctx.device)
        if not x2.is_c_contiguous():
            raise NotImplementedError("full reduction needs a contiguous array")
        lib.nmhipReduce(x.ctx.handle, op, _code(x.dtype), x2.ptr, n0, n1,
                        n1, 1, -1, out.ptr)
        res = out.asnumpy()[0]
        return x.dtype.type(res) if result_dtype is None else result_dtype(res)
    out = empty((n1 if axis == 0 else n0,), acc_dtype, usm_type=x.usm_type,
                device=x.ctx.device)
    lib.nmhipReduce(x.ctx.handle, op, _code(x.dtype), x2.ptr, n0, n1, s0, s1,
                    axis, out.ptr)
    return out


def sum(x, axis=None):
    """numpy.sum (reference: numpy/funcs.py:222-227)."""
    return _reduce(lowered.SUM, x, axis)


def prod(x, axis=None):
    return _reduce(lowered.PROD, x, axis)


def amin(x, axis=None):
    return _reduce(lowered.MIN, x, axis)


def amax(x, axis=None):
    return _reduce(lowered.MAX, x, axis)


def sqrt_sum_squares(x, out=None):
    """``np.sqrt(np.sum(x * x))`` of a contiguous float32 array in one launch;
    returns a 1-element device array (the 0-d result of the reference)."""
    x = asarray(x)
    if x.dtype != np.float32 or not x.is_c_contiguous():
        raise ValueError("sqrt_sum_squares needs a contiguous float32 array")
    if out is None:
        out = empty((1,), np.float32, usm_type="device", device=x.ctx.device)
    lib.nmhipNorm2F32(x.ctx.handle, x.ptr, x.size, out.ptr)
    return out


def l2_norm_rows(a, out=None):
    """``np.sqrt(np.square(a).sum(axis=1))`` of a row-major float32 matrix,
    fused (the body of the reference's ``test_l2_norm``,
    numba_mlir/numba_mlir/mlir/tests/test_gpu.py:2198-2223)."""
    a = asarray(a)
    if a.dtype != np.float32 or a.ndim != 2 or (a.shape[1] > 1 and
                                                a.elem_strides[1] != 1):
        raise ValueError("l2_norm_rows needs a row-major float32 matrix")
    if out is None:
        out = empty((a.shape[0],), np.float32, usm_type=a.usm_type,
                    device=a.ctx.device)
    lib.nmhipNorm2RowsF32(a.ctx.handle, a.ptr, a.shape[0], a.shape[1],
                          a.elem_strides[0], out.ptr)
    return out


def gemm(a, b, c, alpha, beta):
    """``c[:] = beta * c + alpha * np.dot(a, b)`` through
    ``mkl_gemm_<dtype>_device`` (reference: numpy/funcs.py:866-876)."""
    a, b = asarray(a), asarray(b)
    if a.ndim != 2 or b.ndim != 2 or c.ndim != 2:
        raise ValueError("gemm needs 2-D arrays")
    if a.dtype != b.dtype or a.dtype != c.dtype:
        raise TypeError("gemm operands must share a dtype")
    if a.dtype not in (np.float32, np.float64):
        # (the reference binds mkl_gemm for these two only, numpy/funcs.py:848-864)
        raise TypeError(f"gemm is implemented for float32 and float64, not {a.dtype}")
    m, k = a.shape
    k2, n = b.shape
    if k != k2 or c.shape != (m, n):
        raise ValueError("gemm shape mismatch")
    for arr in (a, b, c):
        # _check_mkl_strides (numpy/funcs.py:752-756): the compiler copies an
        # operand with no unit stride or a non-positive stride first.
        s = arr.elem_strides
        if min(s) <= 0 and arr.size > 1 and min(arr.shape) > 1:
            raise NotImplementedError("negative or zero strides need a copy")
        if s[0] != 1 and s[1] != 1:
            raise NotImplementedError("no unit stride: operand needs a copy")
    lib.nmhipGemm(a.ctx.handle, _code(a.dtype), a.ptr, _i64x2(*a.elem_strides),
                  b.ptr, _i64x2(*b.elem_strides), c.ptr,
                  _i64x2(*c.elem_strides), m, n, k, float(alpha), float(beta))
    return c


def dot(a, b, out=None):
    """numpy.dot of 2-D arrays: alpha = 1, beta = 0
    (reference: numpy/funcs.py:803-812, 879-888)."""
    a, b = asarray(a), asarray(b)
    if out is None:
        out = empty((a.shape[0], b.shape[1]), a.dtype, usm_type=a.usm_type,
                    device=a.ctx.device)
    return gemm(a, b, out, 1, 0)


def pairwise_distance(X1, X2, D):
    """The pairwise-distance ``@kernel`` over global size
    ``(X1.shape[0], X2.shape[0])`` with the row-remapped float64 twin
    (body: reference numba_mlir/numba_mlir/mlir/tests/test_gpu.py:1397-1408)."""
    X1, X2 = asarray(X1), asarray(X2)
    for x in (X1, X2, D):
        if x.dtype != np.float64 or x.ndim != 2 or not x.is_c_contiguous():
            raise ValueError("pairwise_distance needs C-contiguous float64 "
                             "2-D arrays")
    if X1.shape[1] != 3 or X2.shape[1] != 3:
        raise ValueError("the remapped twin is specialised for 3 columns")
    if D.shape != (X1.shape[0], X2.shape[0]):
        raise ValueError("D has the wrong shape")
    lib.nmhipPairwiseF64(D.ctx.handle, X1.ptr, X2.ptr, D.ptr, X1.shape[0],
                         X2.shape[0])
    return D
