"""GPU parity: axis and full reductions through the gpux* C-ABI."""

import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
    GOLD = json.load(f)

DIMS = GOLD["reduce_shapes"]["dims_2d"]


@pytest.fixture(scope="module")
def env(hip):
    from numba_mlir_amd.mlir import ops
    from oracle import oracle as orc
    return hip, ops, orc


def test_small_golden(env):
    hip, ops, _ = env
    g = GOLD["reduce_axis_small"]
    for dtype in (np.int32, np.float32):
        d = hip.asarray(np.array(g["arr"], dtype))
        assert ops.sum(d, axis=0).asnumpy().tolist() == g["sum_axis0"]
        assert ops.sum(d, axis=1).asnumpy().tolist() == g["sum_axis1"]
        assert ops.sum(d, axis=-1).asnumpy().tolist() == g["sum_axis1"]
        assert ops.sum(d) == g["sum_all"]


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32])
@pytest.mark.parametrize("n0", DIMS)
@pytest.mark.parametrize("n1", DIMS)
def test_reference_reduce_shapes(env, dtype, n0, n1):
    """test_cfd_reduce2 of the reference (tests/test_gpu.py:2068-2098):
    arange(1..count) reshaped, sum/prod/amin/amax, rtol 1e-5."""
    hip, ops, _ = env
    count = n0 * n1
    a = np.arange(1, count + 1, dtype=dtype).reshape(n0, n1).copy()
    d = hip.asarray(a)
    rtol = GOLD["reduce_shapes"]["rtol"]
    np.testing.assert_allclose(ops.sum(d), a.sum(), rtol=rtol)
    np.testing.assert_allclose(ops.sum(d, axis=0).asnumpy(), a.sum(axis=0), rtol=rtol)
    np.testing.assert_allclose(ops.sum(d, axis=1).asnumpy(), a.sum(axis=1), rtol=rtol)
    assert ops.amin(d) == a.min() and ops.amax(d) == a.max()
    np.testing.assert_array_equal(ops.amin(d, axis=0).asnumpy(), a.min(axis=0))
    np.testing.assert_array_equal(ops.amax(d, axis=1).asnumpy(), a.max(axis=1))
    if count <= 30:          # the reference skips larger products (overflow)
        np.testing.assert_allclose(ops.prod(d), np.prod(a), rtol=rtol)
        np.testing.assert_allclose(ops.prod(d, axis=0).asnumpy(),
                                   np.prod(a, axis=0), rtol=rtol)


@pytest.mark.parametrize("size", GOLD["reduce_shapes"]["sizes_1d"])
def test_reference_reduce_1d(env, size):
    """test_cfd_reduce1 (tests/test_gpu.py:2045-2062): arange float32, rtol 1e-5."""
    hip, ops, _ = env
    a = np.arange(size, dtype=np.float32)
    got = ops.sum(hip.asarray(a))
    np.testing.assert_allclose(got, a.astype(np.float64).sum(), rtol=1e-5)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_min_max_skip_nans_as_the_reference_fold_does(env, dtype):
    """The reference folds select(x < acc, x, acc) from +inf (builtin/funcs.py:
    145-146, numpy/funcs.py:283-303): a NaN never wins, whatever its position;
    all-NaN and empty inputs give the starting value.  numpy.fmin / fmax
    reduced from the same starting value are that fold's closed form."""
    hip, ops, _ = env
    rng = np.random.default_rng(11)
    for shape in ((7,), (300,), (70000,), (5, 9), (129, 1000), (2000, 33)):
        a = rng.standard_normal(shape).astype(dtype)
        flat = a.reshape(-1)
        for where in (0, flat.size // 2, flat.size - 1):     # first, middle, last
            b = flat.copy()
            b[where] = np.nan
            b = b.reshape(shape)
            d = hip.asarray(b)
            assert ops.amin(d) == np.fmin.reduce(b, axis=None, initial=np.inf)
            assert ops.amax(d) == np.fmax.reduce(b, axis=None, initial=-np.inf)
            if b.ndim == 2:
                for axis in (0, 1):
                    np.testing.assert_array_equal(
                        ops.amin(d, axis=axis).asnumpy(),
                        np.fmin.reduce(b, axis=axis, initial=np.inf))
                    np.testing.assert_array_equal(
                        ops.amax(d, axis=axis).asnumpy(),
                        np.fmax.reduce(b, axis=axis, initial=-np.inf))
    every = hip.asarray(np.full((4, 6), np.nan, dtype))
    assert ops.amin(every) == np.inf and ops.amax(every) == -np.inf
    np.testing.assert_array_equal(ops.amin(every, axis=1).asnumpy(), np.full(4, np.inf, dtype))
    none = hip.asarray(np.zeros((0, 3), dtype))
    assert ops.amin(none) == np.inf and ops.amax(none) == -np.inf
    np.testing.assert_array_equal(ops.amax(none, axis=0).asnumpy(), np.full(3, -np.inf, dtype))


def test_int_dtype_promotion(env):
    hip, ops, _ = env
    a = np.full((70000, 8), 2 ** 31 - 1, np.int32)
    out = ops.sum(hip.asarray(a), axis=0).asnumpy()
    assert out.dtype == np.int64 and out.tolist() == [70000 * (2 ** 31 - 1)] * 8
    assert hip.get_context().last_kernel() == "nmk_sum_axis0_i32_i64"


@pytest.mark.parametrize("shape", [(64, 256), (100, 260), (16384, 8192),
                                   (1000, 1028), (4097, 512), (65, 4)])
def test_sum_axis0_i32_bit_exact(env, shape):
    hip, ops, orc = env
    rng = np.random.Generator(np.random.PCG64(1013))
    x = rng.integers(-1000, 1000, shape, dtype=np.int32, endpoint=True)
    d = hip.asarray(x)
    for _ in range(2):       # second call reuses scratch and self-reset tickets
        got = ops.sum(d, axis=0).asnumpy()
        assert got.dtype == np.int64
        assert np.array_equal(got, orc.sum_axis0_i32(x))
    assert hip.get_context().last_kernel() == "nmk_sum_axis0_i32_i64"


# Tolerance for float32 sums: |gpu - truth| <= 1e-4 * sum|x| (float64 truth).
# The reference states rel 1e-4/1e-5 on positive data; for zero-mean data the
# sum itself can be arbitrarily close to 0, so the bound is relative to the
# sum of magnitudes.
# (rows of one 16 KiB batch run the kernel capped at four waves a SIMD, many
# rows of two or three whole batches the one capped at three)
@pytest.mark.parametrize("shape, kernel", [
    ((4, 8192), "nmk_sum_axis1_wide_f32"), ((333, 1000), "nmk_sum_axis1_f32"),
    ((16384, 8192), "nmk_sum_axis1_wide_w3_f32"), ((7, 5), "nmk_sum_axis1_f32"),
    ((1024, 4100), "nmk_sum_axis1_wide_f32"), ((600, 4096), "nmk_sum_axis1_wide_w4_f32"),
    ((4100, 12288), "nmk_sum_axis1_wide_w3_f32"), ((4100, 16384), "nmk_sum_axis1_wide_f32")])
def test_sum_axis1_f32(env, shape, kernel):
    hip, ops, orc = env
    rng = np.random.Generator(np.random.PCG64(1003))
    x = rng.standard_normal(shape, dtype=np.float32)
    got = ops.sum(hip.asarray(x), axis=1).asnumpy()
    assert hip.get_context().last_kernel() == kernel
    x64 = x.astype(np.float64)
    truth, mag = x64.sum(axis=1), np.abs(x64).sum(axis=1)
    assert (np.abs(got - truth) <= 1e-4 * mag).all()
    if shape[0] * shape[1] <= 1 << 22:
        # the oracle (sequential float32 rows) obeys the same bound
        assert (np.abs(orc.sum_axis1_f32(x) - truth) <= 1e-4 * mag).all()
    # positive data: plain relative tolerance, as the reference states it
    y = np.abs(x)
    got = ops.sum(hip.asarray(y), axis=1).asnumpy()
    np.testing.assert_allclose(got, y.astype(np.float64).sum(axis=1), rtol=1e-5)


@pytest.mark.parametrize("n", [0, 1, 5, 4096, 4099, 1 << 20, 16384 * 8192])
def test_sqrt_sum_squares(env, n):
    hip, ops, orc = env
    rng = np.random.Generator(np.random.PCG64(1003))
    x = rng.standard_normal(n, dtype=np.float32)
    d = hip.asarray(x)
    got = [float(ops.sqrt_sum_squares(d).asnumpy()[0]) for _ in range(2)]
    assert got[0] == got[1]          # fixed combination order
    truth = float(np.sqrt((x.astype(np.float64) ** 2).sum()))
    assert abs(got[0] - truth) <= 1e-5 * truth + 0.0
    if 0 < n <= 1 << 20:
        assert abs(float(orc.norm2_f32(x)) - truth) <= 1e-4 * truth


def test_sqrt_sum_squares_exact(env):
    hip, ops, _ = env
    assert ops.sqrt_sum_squares(hip.asarray(np.array([3, 4], np.float32))).asnumpy()[0] == 5
    x = np.zeros(1 << 16, np.float32)
    x[::1024] = 2
    assert ops.sqrt_sum_squares(hip.asarray(x)).asnumpy()[0] == 16


def test_strided_and_transposed_inputs(env):
    hip, ops, _ = env
    rng = np.random.default_rng(8)
    a = rng.integers(-50, 50, (45, 67)).astype(np.int64)
    dt = hip.asarray(np.ascontiguousarray(a.T)).T
    np.testing.assert_array_equal(ops.sum(dt, axis=0).asnumpy(), a.sum(axis=0))
    np.testing.assert_array_equal(ops.sum(dt, axis=1).asnumpy(), a.sum(axis=1))
    f = rng.standard_normal((45, 67))
    np.testing.assert_allclose(ops.amax(hip.asarray(f), axis=1).asnumpy(), f.max(axis=1))
    np.testing.assert_allclose(ops.sum(hip.asarray(f), axis=0).asnumpy(), f.sum(axis=0),
                               rtol=1e-12)


# Shapes that take every route of the generic kernels: rows long enough for a
# block each (with and without whole 128-bit words), column strips on words
# (a last strip that is not full) and on single elements, a contiguous run in
# block chunks with a ragged end, and the same from a base inside a word.
_ROUTES = [
    ("rows, a block each, words", (600, 4100), False),
    ("rows, a block each, odd leading dimension", (520, 4099), False),
    ("rows, a wave each", (37, 1500), False),
    ("few long rows", (5, 70000), False),
    ("columns on words", (4100, 516), False),
    ("columns on single elements", (4100, 515), False),
    ("many short rows, a group of lanes each", (70001, 16), False),
    ("many rows of three", (50000, 3), False),
    ("many rows of 64, base inside a word", (5000, 64), True),
    ("many short columns, a lane each", (7, 70001), False),
    ("one run in chunks", (1, 1000003), False),
    ("one run in chunks, base inside a word", (1, 1000003), True),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
@pytest.mark.parametrize("what,shape,offset", _ROUTES, ids=[r[0] for r in _ROUTES])
def test_generic_reductions_on_every_route(env, dtype, what, shape, offset):
    """sum / prod / amin / amax over each axis and over everything: minima,
    maxima and integer sums exact, float sums and products to 1e-5 of a
    float64 fold (values in [0.5, 1.5): sums cannot cancel; products over
    values next to 1)."""
    hip, ops, _ = env
    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    count = shape[0] * shape[1]
    if np.issubdtype(dtype, np.integer):
        flat = rng.integers(-1000, 1000, count + 1).astype(dtype)
    else:
        flat = rng.uniform(0.5, 1.5, count + 1).astype(dtype)
    a = flat[1:].reshape(shape) if offset else flat[:count].reshape(shape)
    d = hip.asarray(flat)
    d = (d[1:] if offset else d[:count]).reshape(shape)
    exact = np.issubdtype(dtype, np.integer)
    wide = a.astype(np.int64 if exact else np.float64)
    for axis in (None, 0, 1):
        got = {name: fn(d, axis=axis) for name, fn in
               (("sum", ops.sum), ("amin", ops.amin), ("amax", ops.amax))}
        got = {k: (v.asnumpy() if hasattr(v, "asnumpy") else v) for k, v in got.items()}
        np.testing.assert_array_equal(got["amin"], a.min(axis=axis))
        np.testing.assert_array_equal(got["amax"], a.max(axis=axis))
        if exact:
            np.testing.assert_array_equal(got["sum"], wide.sum(axis=axis))
        else:
            np.testing.assert_allclose(got["sum"], wide.sum(axis=axis), rtol=1e-5)
    # products: factors within 2^-10 of 1 so that a million of them stay in
    # range (float32 rounds every partial product: 2.5 million of them drift
    # by up to sqrt(n) * 2^-24)
    if not exact:
        f = (1.0 + rng.uniform(-1.0, 1.0, count + 1) * 2.0 ** -10).astype(dtype)
        fa = f[1:].reshape(shape) if offset else f[:count].reshape(shape)
        fd = hip.asarray(f)
        fd = (fd[1:] if offset else fd[:count]).reshape(shape)
        # (float32 over millions of factors drifts by parts in a thousand with
        # the grouping alone -- NumPy's own float32 product of the same
        # factors taken four at a time does: the float64 fold is no yardstick
        # for it)
        for axis in ((None, 0, 1) if dtype is np.float64 or count < 100000 else (0, 1)):
            got = ops.prod(fd, axis=axis)
            got = got.asnumpy() if hasattr(got, "asnumpy") else got
            np.testing.assert_allclose(got, np.prod(fa.astype(np.float64), axis=axis), rtol=1e-3)
    else:
        f = rng.choice(np.array([1, -1, 1, 1, 2], dtype), count + 1)
        f[rng.integers(0, count, count // 64)] = 1
        fa = f[1:].reshape(shape) if offset else f[:count].reshape(shape)
        fd = hip.asarray(f)
        fd = (fd[1:] if offset else fd[:count]).reshape(shape)
        for axis in (0, 1):       # (int64 wraps the same way in NumPy)
            got = ops.prod(fd, axis=axis).asnumpy()
            np.testing.assert_array_equal(got, np.prod(fa.astype(np.int64), axis=axis))


def test_release_acquire_handoff_gives_the_same_bits(env):
    """The reduction kernels hand per-block partial results to the launch's
    last block through agent-scope accesses ordered by a wait for the stores'
    acknowledgement.  The same kernels built with the hand-off the language's
    memory model prescribes (release on the ticket, acquire in the last block:
    the "reduce_release" code object) combine in the same fixed order, so the
    three benchmark reductions at full size, and the generic kernels, must give
    identical bits from both code objects."""
    hip, ops, _ = env
    from numba_mlir_amd.mlir import lowered
    plain, release = lowered.kernel_blob("reduce"), lowered.kernel_blob("reduce_release")
    assert plain != release                     # the build flag took effect
    rng = np.random.Generator(np.random.PCG64(1003))
    x = rng.standard_normal((16384, 8192), dtype=np.float32)
    xi = np.random.Generator(np.random.PCG64(1013)).integers(
        -1000, 1000, (16384, 8192), dtype=np.int32, endpoint=True)
    d_x, d_xi = hip.asarray(x), hip.asarray(xi)
    d_x64 = hip.asarray(x[:2048].astype(np.float64))

    def results():
        out = [ops.sum(d_x, axis=1).asnumpy(),
               ops.sqrt_sum_squares(d_x.reshape((x.size,))).asnumpy(),
               ops.sum(d_xi, axis=0).asnumpy()]
        names = [hip.get_context().last_kernel()]
        out += [ops.sum(d_x, axis=0).asnumpy(), np.asarray(ops.amax(d_x)),
                ops.prod(d_x64, axis=0).asnumpy(), np.asarray(ops.sum(d_x64))]
        return out, names

    try:
        base, names0 = results()
        lowered.set_tuning("handoff_release", 1)
        other, names1 = results()
    finally:
        lowered.set_tuning("handoff_release", 0)
    assert names0 == names1 == ["nmk_sum_axis0_i32_i64"]
    for a, b in zip(base, other):
        assert a.dtype == b.dtype and a.shape == b.shape
        assert a.tobytes() == b.tobytes()
    # and the integer one is the exact column sum either way
    assert np.array_equal(other[2], xi.sum(axis=0, dtype=np.int64))
