"""GPU: shapes at the edges of the launch geometry -- very long and very
thin arrays, degenerate dimensions, flipped, strided, transposed and
zero-stride views, one-element arrays -- through the library kernels and the
fused maps, against NumPy."""

import numpy as np
import pytest

from numba_mlir_amd.decorators import njit

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env(hip):
    from numba_mlir_amd.mlir import ops
    return hip, ops


def _host(x):
    return x.asnumpy() if hasattr(x, "asnumpy") else x


def test_few_rows_of_many_columns(env):
    hip, ops = env
    d = hip.asarray(np.ones((8, 2 ** 25), np.float32))
    cols = ops.sum(d, axis=0)
    assert cols.shape == (2 ** 25,)
    assert float(ops.amin(cols)) == 8.0 and float(ops.amax(cols)) == 8.0
    assert ops.sum(d, axis=1).asnumpy().tolist() == [2.0 ** 25] * 8


@pytest.mark.parametrize("shape", [(2 ** 22, 1), (1, 2 ** 22)])
def test_a_dimension_of_one(env, shape):
    hip, ops = env
    x = np.arange(2 ** 22, dtype=np.int32).reshape(shape)
    d = hip.asarray(x)
    for axis in (0, 1):
        assert np.array_equal(ops.sum(d, axis=axis).asnumpy(), x.sum(axis=axis, dtype=np.int64))
        assert np.array_equal(ops.amax(d, axis=axis).asnumpy(), x.max(axis=axis))
    assert int(ops.amax(d)) == 2 ** 22 - 1
    f = x.astype(np.float32)
    assert np.array_equal(ops.add(hip.asarray(f), hip.asarray(f)).asnumpy(), f + f)


def test_reductions_over_tall_strided_views(env):
    hip, ops = env
    x = np.random.default_rng(0).standard_normal((3_000_000, 3))
    d = hip.asarray(x)[:, :2]
    assert np.array_equal(ops.amax(d, axis=0).asnumpy(), x[:, :2].max(axis=0))
    assert np.array_equal(ops.amax(d, axis=1).asnumpy(), x[:, :2].max(axis=1))


def _root_plus_one(a):
    return np.sqrt(np.abs(a)) + 1.0


def test_flipped_strided_and_transposed_views(env):
    hip, ops = env
    x = np.random.default_rng(1).standard_normal((1000, 700))
    d = hip.asarray(x)
    f = njit(_root_plus_one)
    for view_d, view_h in ((d[::-1], x[::-1]), (d[:, ::-1], x[:, ::-1]),
                           (d[::2, ::3], x[::2, ::3]), (d.T, x.T),
                           (d[::-2, 5:600:7], x[::-2, 5:600:7])):
        for axis in (0, 1):
            np.testing.assert_allclose(ops.sum(view_d, axis=axis).asnumpy(),
                                       view_h.sum(axis=axis), rtol=1e-12, atol=1e-11)
            assert np.array_equal(ops.amax(view_d, axis=axis).asnumpy(), view_h.max(axis=axis))
        assert np.array_equal(ops.add(view_d, view_d).asnumpy(), view_h + view_h)
        np.testing.assert_allclose(f(view_d).asnumpy(), np.sqrt(np.abs(view_h)) + 1.0,
                                   rtol=1e-15)


def test_zero_stride_operands(env):
    hip, ops = env
    x = np.random.default_rng(2).standard_normal((1, 700))
    b = hip.asarray(x).broadcast_to((900, 700))
    hb = np.broadcast_to(x, (900, 700))
    np.testing.assert_allclose(ops.sum(b, axis=0).asnumpy(), hb.sum(axis=0), rtol=1e-12, atol=1e-11)
    np.testing.assert_allclose(ops.sum(b, axis=1).asnumpy(), hb.sum(axis=1), rtol=1e-12, atol=1e-11)
    y = np.random.default_rng(3).standard_normal((900, 700))
    assert np.array_equal(ops.add(b, hip.asarray(y)).asnumpy(), hb + y)


def _outer_sum(x, y):
    return x + y


def test_column_against_row(env):
    hip, _ = env
    a = np.random.default_rng(4).standard_normal((3000, 1))
    b = np.random.default_rng(5).standard_normal((1, 2000))
    assert np.array_equal(njit(_outer_sum)(hip.asarray(a), hip.asarray(b)).asnumpy(), a + b)


@pytest.mark.parametrize("shape", [(1, 1), (1, 3), (3, 1), (2, 2), (5, 7), (1, 129), (129, 1)])
def test_tiny_shapes(env, shape):
    hip, ops = env
    x = np.random.default_rng(6).standard_normal(shape).astype(np.float32)
    d = hip.asarray(x)
    for axis in (None, 0, 1):
        np.testing.assert_allclose(_host(ops.sum(d, axis=axis)),
                                   x.astype(np.float64).sum(axis=axis), rtol=1e-5, atol=1e-6)
        assert np.array_equal(_host(ops.amin(d, axis=axis)), x.min(axis=axis))
    c = hip.asarray(np.zeros((shape[0], shape[0]), np.float32))
    ops.gemm(d, hip.asarray(np.ascontiguousarray(x.T)), c, 1.0, 0.0)
    np.testing.assert_allclose(c.asnumpy(), x @ x.T, rtol=1e-5, atol=1e-6)


def test_gemm_with_one_long_dimension(env):
    hip, ops = env
    rng = np.random.default_rng(7)
    a = rng.standard_normal((8, 2_000_000)).astype(np.float32)
    b = rng.standard_normal((2_000_000, 8)).astype(np.float32)
    c = hip.asarray(np.zeros((8, 8), np.float32))
    ops.gemm(hip.asarray(a), hip.asarray(b), c, 1.0, 0.0)
    truth = a.astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64)
    assert (np.abs(c.asnumpy() - truth) <= 1e-5 * scale).all()
    a = rng.standard_normal((8, 16)).astype(np.float32)
    b = rng.standard_normal((16, 3_000_000)).astype(np.float32)
    c = hip.asarray(np.zeros((8, 3_000_000), np.float32))
    ops.gemm(hip.asarray(a), hip.asarray(b), c, 1.0, 0.0)
    np.testing.assert_allclose(c.asnumpy(), a @ b, rtol=1e-4, atol=1e-4)


def _row_sums_of_squares(a):
    return np.sum(a * a, axis=1)


def _column_sums_of_squares(a):
    return np.sum(a * a, axis=0)


def test_fused_axis_sums_of_a_tall_matrix(env):
    hip, _ = env
    x = np.random.default_rng(8).uniform(0.5, 1.5, (5_000_000, 3)).astype(np.float32)
    d = hip.asarray(x)
    np.testing.assert_allclose(njit(_row_sums_of_squares)(d).asnumpy(),
                               (x.astype(np.float64) ** 2).sum(axis=1), rtol=1e-5)
    np.testing.assert_allclose(njit(_column_sums_of_squares)(d).asnumpy(),
                               (x.astype(np.float64) ** 2).sum(axis=0), rtol=1e-4)


def _tall_body(a, b, c):
    return a - 2.0 * b + c


def _tall_store(a, b, c, out):
    out[:] = a * b + c


@pytest.mark.parametrize("cols", [1, 3, 8, 16, 33, 63, 64])
@pytest.mark.parametrize("rows", [64, 1000, 100003])
def test_tall_results_of_a_few_columns(env, rows, cols):
    """A fused map over [rows, cols] with a column and a row operand (which
    keeps the two dimensions apart): with fewer than 64 columns the blocks
    have lanes along the rows too, so a wave works on whole neighbouring rows
    instead of one short one."""
    hip, _ = env
    rng = np.random.default_rng(rows + cols)
    a = rng.standard_normal((rows, 1))
    b = rng.standard_normal((rows, cols))
    c = rng.standard_normal(cols)
    f = njit(_tall_body)
    got = f(hip.asarray(a), hip.asarray(b), hip.asarray(c))
    assert np.array_equal(_host(got), a - 2.0 * b + c)
    block = f.last_launch["block"]
    if cols < 64 and cols > 1:
        assert block[:2] == (cols, min(256 // cols, rows)), block
    out = hip.asarray(np.zeros((rows, cols), np.float32))
    g = njit(_tall_store)
    a32, b32, c32 = a.astype(np.float32), b.astype(np.float32), c.astype(np.float32)
    g(hip.asarray(a32), hip.asarray(b32), hip.asarray(c32), out)
    assert np.array_equal(out.asnumpy(), a32 * b32 + c32)


def test_a_tall_kernel_grid_of_a_few_columns(env):
    """The same layout for an @kernel body launched over (rows, 8) with a
    block chosen by the runtime."""
    hip, _ = env
    from numba_mlir_amd import kernel as kapi

    def body(x, y, out):
        i = kapi.get_global_id(0)
        j = kapi.get_global_id(1)
        out[i, j] = x[i, j] * 3 + y[j] - i

    rows, cols = 50001, 8
    x = np.arange(rows * cols, dtype=np.int64).reshape(rows, cols)
    y = np.arange(cols, dtype=np.int64) * 7
    out = hip.asarray(np.zeros((rows, cols), np.int64))
    k = kapi.kernel(body)[(rows, cols), ()]
    k(hip.asarray(x), hip.asarray(y), out)
    assert k.last_launch["block"][:2] == (8, 32)
    assert np.array_equal(out.asnumpy(), x * 3 + y - np.arange(rows)[:, None])
