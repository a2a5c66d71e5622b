"""Seeded synthetic inputs of the five benchmark configurations.

Shapes, distributions and seeds are fixed so every run (tests, smoke, bench)
sees the same data.  Configuration 2 reproduces the reference's own generator
(reference: numba_mlir/numba_mlir/mlir/tests/test_numpy.py:2798-2820): legacy
``numpy.random.seed`` + ``uniform`` in float64, cast to float32.
"""

import numpy as np

RISK_FREE = np.float32(0.1)
VOLATILITY = np.float32(0.2)


def broadcast_add(rows=4096, cols=4096, seed=1001):
    rng = np.random.Generator(np.random.PCG64(seed))
    a = rng.uniform(-1.0, 1.0, (rows, cols))
    b = rng.uniform(-1.0, 1.0, (1, cols))
    return a, b


def black_scholes(nopt=2 ** 24, seed=777777):
    rs = np.random.RandomState(seed)
    dtype = np.float32
    price = rs.uniform(dtype(10.0), dtype(50.0), nopt).astype(dtype)
    strike = rs.uniform(dtype(10.0), dtype(50.0), nopt).astype(dtype)
    t = rs.uniform(dtype(1.0), dtype(2.0), nopt).astype(dtype)
    call = np.zeros(nopt, dtype=dtype)
    put = -np.ones(nopt, dtype=dtype)
    return price, strike, t, RISK_FREE, VOLATILITY, call, put


def reduce_f32(rows=16384, cols=8192, seed=1003):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.standard_normal((rows, cols), dtype=np.float32)


def reduce_i32(rows=16384, cols=8192, seed=1013):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.integers(-1000, 1000, (rows, cols), dtype=np.int32, endpoint=True)


def pairwise(npoints=8192, dims=3, seed=1004):
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.uniform(0.0, 1.0, (npoints, dims)), rng.uniform(0.0, 1.0,
                                                               (npoints, dims))


def matmul(n=4096, seed=1005):
    rng = np.random.Generator(np.random.PCG64(seed))
    a = rng.standard_normal((n, n), dtype=np.float32)
    b = rng.standard_normal((n, n), dtype=np.float32)
    return a, b
