"""TEST INFRASTRUCTURE -- not part of the product.

Python face of the CPU oracle: ctypes wrappers over ``oracle.c`` (the C
restatement of the reference's ``@njit(parallel=True)`` CPU path, each
function citing the reference file:line it follows) plus float64 ground
truths used to bound float32 results.

Parity status of each function ("pinned by" = the independent check in
``tests/test_oracle.py`` a plausible mistake would fail):

  add                 pinned: bit-equal to numpy a + b on the reference's
                      broadcast fixtures (tests/test_numpy.py:483-514)
  black_scholes       pinned at tolerance: closed-form price via
                      scipy.stats.norm.cdf in float64, put-call parity
  sum_axis1_f32       pinned: exact on arange fixtures
                      (tests/test_gpu.py:2068-2098), float64 truth bound
  sum_axis0_i32       pinned: equals numpy int64 sum exactly
  norm2_f32           pinned: exact on integer inputs, float64 truth bound
  pairwise            pinned: closed form on the reference's arange fixture
                      (tests/test_gpu.py:1413-1418), scipy cdist
  gemm_f32            pinned: exact on the reference's integer fixtures
                      (tests/test_gpu.py:2101-2193), golden 3x3 of
                      mlir/test/L0_RUNNER/linalg_gemmf.mlir:8-19
  suggest_block_size  pinned: hand-computed table
  kernel_sim          pinned: closed-form index results
                      (tests/test_gpu.py:580-803)

The exact bits of the reference's float32 reductions and transcendentals
depend on its thread count, vector width and libm and cannot be reproduced
without running it: those comparisons are at tolerance only.
"""

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")


def build():
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.orc_max_threads.restype = ci
    for name in ("orc_add_f64", "orc_add_f32", "orc_add_i64", "orc_add_i32"):
        getattr(lib, name).restype = None
        getattr(lib, name).argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i64, ci]
    lib.orc_black_scholes_f32.restype = None
    lib.orc_black_scholes_f32.argtypes = [vp, vp, vp, ctypes.c_float,
                                          ctypes.c_float, vp, vp, i64, ci, ci]
    lib.orc_sum_axis1_f32.restype = None
    lib.orc_sum_axis1_f32.argtypes = [vp, i64, i64, i64, i64, vp, ci]
    lib.orc_sum_axis0_i32.restype = None
    lib.orc_sum_axis0_i32.argtypes = [vp, i64, i64, i64, i64, vp, ci]
    lib.orc_norm2_f32.restype = ctypes.c_float
    lib.orc_norm2_f32.argtypes = [vp, i64, ci]
    for name in ("orc_pairwise_f64", "orc_pairwise_f32"):
        getattr(lib, name).restype = None
        getattr(lib, name).argtypes = [vp, vp, vp, i64, i64, i64, ci]
    lib.orc_gemm_f32.restype = None
    lib.orc_gemm_f32.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i64, i64,
                                 i64, i64, ctypes.c_float, ctypes.c_float, ci]
    lib.orc_gemm_f32_acc64.restype = None
    lib.orc_gemm_f32_acc64.argtypes = [vp, i64, i64, vp, i64, i64, vp, i64, i64,
                                       i64, ci]
    lib.orc_suggest_block_size.restype = None
    lib.orc_suggest_block_size.argtypes = [ctypes.c_uint32, vp, vp,
                                           ctypes.c_size_t]
    return lib


_lib = _load()


def _p(arr):
    return arr.ctypes.data_as(ctypes.c_void_p)


def _estrides(arr):
    return tuple(s // arr.itemsize for s in arr.strides)


def max_threads():
    return int(_lib.orc_max_threads())


# ---------------------------------------------------------------------------
def add(a, b, threads=0):
    """numpy.add with broadcasting for rank <= 2 operands of one dtype."""
    a, b = np.asarray(a), np.asarray(b)
    assert a.dtype == b.dtype
    shape = np.broadcast_shapes(a.shape, b.shape)
    fn = {np.dtype(np.float64): _lib.orc_add_f64,
          np.dtype(np.float32): _lib.orc_add_f32,
          np.dtype(np.int64): _lib.orc_add_i64,
          np.dtype(np.int32): _lib.orc_add_i32}[a.dtype]
    shape2 = (1,) * (2 - len(shape)) + tuple(shape)
    ab = np.broadcast_to(a, shape).reshape(shape2) if a.size else a
    # broadcast_to gives stride 0 on broadcast dims; reshape of such a view
    # may copy, so derive the strides by hand instead.
    def strides2(x):
        shp = (1,) * (2 - x.ndim) + x.shape
        st = (0,) * (2 - x.ndim) + _estrides(x)
        return [0 if n == 1 else s for n, s in zip(shp, st)]
    del ab
    out = np.empty(shape2, a.dtype)
    if out.size:
        sa, sb = strides2(a), strides2(b)
        fn(_p(a), sa[0], sa[1], _p(b), sb[0], sb[1], _p(out), shape2[0],
           shape2[1], threads)
    return out.reshape(shape)


def black_scholes(price, strike, t, rate, volatility, wide=True, threads=0):
    n = price.size
    call = np.empty(n, np.float32)
    put = np.empty(n, np.float32)
    _lib.orc_black_scholes_f32(_p(price), _p(strike), _p(t),
                               float(np.float32(rate)),
                               float(np.float32(volatility)), _p(call), _p(put),
                               n, 1 if wide else 0, threads)
    return call, put


def black_scholes_truth(price, strike, t, rate, volatility):
    """Closed-form Black-Scholes in float64 from the float32 inputs:
    call = P N(d1) - S exp(-rT) N(d2), put by parity."""
    from scipy.stats import norm
    P, S, T = (np.asarray(x, np.float64) for x in (price, strike, t))
    r = float(np.float32(rate))
    sig = float(np.float32(volatility))
    srt = sig * np.sqrt(T)
    d1 = (np.log(P / S) + (r + 0.5 * sig * sig) * T) / srt
    d2 = d1 - srt
    disc = S * np.exp(-r * T)
    call = P * norm.cdf(d1) - disc * norm.cdf(d2)
    put = disc * norm.cdf(-d2) - P * norm.cdf(-d1)
    return call, put


def sum_axis1_f32(x, threads=0):
    x = np.asarray(x)
    assert x.dtype == np.float32 and x.ndim == 2
    out = np.empty(x.shape[0], np.float32)
    s = _estrides(x)
    _lib.orc_sum_axis1_f32(_p(x), x.shape[0], x.shape[1], s[0], s[1], _p(out),
                           threads)
    return out


def sum_axis0_i32(x, threads=0):
    x = np.asarray(x)
    assert x.dtype == np.int32 and x.ndim == 2
    out = np.empty(x.shape[1], np.int64)
    s = _estrides(x)
    _lib.orc_sum_axis0_i32(_p(x), x.shape[0], x.shape[1], s[0], s[1], _p(out),
                           threads)
    return out


def norm2_f32(x, threads=0):
    x = np.ascontiguousarray(x, np.float32)
    return np.float32(_lib.orc_norm2_f32(_p(x), x.size, threads))


def pairwise(X1, X2, threads=0):
    X1, X2 = np.ascontiguousarray(X1), np.ascontiguousarray(X2)
    assert X1.dtype == X2.dtype and X1.shape[1] == X2.shape[1]
    D = np.empty((X1.shape[0], X2.shape[0]), X1.dtype)
    fn = _lib.orc_pairwise_f64 if X1.dtype == np.float64 else _lib.orc_pairwise_f32
    fn(_p(X1), _p(X2), _p(D), X1.shape[0], X2.shape[0], X1.shape[1], threads)
    return D


def gemm_f32(a, b, c=None, alpha=1.0, beta=0.0, threads=0):
    """c = beta * c + alpha * a @ b, float32 accumulate, k innermost."""
    a, b = np.asarray(a), np.asarray(b)
    assert a.dtype == np.float32 and b.dtype == np.float32
    m, k = a.shape
    n = b.shape[1]
    if c is None:
        c = np.zeros((m, n), np.float32)
    sa, sb, sc = _estrides(a), _estrides(b), _estrides(c)
    _lib.orc_gemm_f32(_p(a), sa[0], sa[1], _p(b), sb[0], sb[1], _p(c), sc[0],
                      sc[1], m, n, k, alpha, beta, threads)
    return c


def gemm_f32_truth(a, b, threads=0):
    a, b = np.asarray(a), np.asarray(b)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), np.float64)
    sa, sb = _estrides(a), _estrides(b)
    _lib.orc_gemm_f32_acc64(_p(a), sa[0], sa[1], _p(b), sb[0], sb[1], _p(c), m,
                            n, k, threads)
    return c


def suggest_block_size(max_wg, global_size):
    g = (ctypes.c_uint32 * len(global_size))(*global_size)
    b = (ctypes.c_uint32 * len(global_size))()
    _lib.orc_suggest_block_size(max_wg, g, b, len(global_size))
    return tuple(b)
