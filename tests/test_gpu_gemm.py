"""GPU parity: np.dot / __internal_gemm through mkl_gemm_<dtype>_device."""

import itertools
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
    GOLD = json.load(f)


@pytest.fixture(scope="module")
def env(hip):
    from numba_mlir_amd.mlir import math_runtime, ops
    from oracle import oracle as orc
    return hip, ops, orc, math_runtime


def _kernel(mrt):
    """Name of the last gemm kernel without the marker of how K was shared
    out (split into slices, or even shares of the slabs of all tiles: that
    depends only on how many tiles the shape has)."""
    return mrt.last_kernel().replace("_splitk", "").replace("_even", "").replace("+packed", "")


def _printed(x):
    return np.array([float("%.6g" % v) for v in np.ravel(x)]).reshape(np.shape(x))


def _to_dev(hip, a):
    """Device copy that keeps the host array's layout (C, F or a transposed view)."""
    if a.flags["C_CONTIGUOUS"]:
        return hip.asarray(a)
    assert a.T.flags["C_CONTIGUOUS"]
    return hip.asarray(np.ascontiguousarray(a.T)).T


def test_dot_golden(env):
    hip, ops, _, _ = env
    g = GOLD["dot_2d"]
    a, b = np.array(g["a"], np.float32), np.array(g["b"], np.float32)
    got = ops.dot(hip.asarray(a), hip.asarray(b)).asnumpy()
    assert np.array_equal(got, np.array(g["out"], np.float32))
    # test_dot's flipped variants are copies made by the compiler before the
    # call; here: their materialised equivalents
    for aa, bb in ((a[::-1].copy(), b), (a, b[:, ::-1].copy())):
        got = ops.dot(hip.asarray(aa), hip.asarray(bb)).asnumpy()
        assert np.array_equal(got, np.dot(aa, bb))


def test_linalg_gemmf_golden(env):
    hip, ops, _, _ = env
    g = GOLD["linalg_gemmf"]
    c = hip.asarray(np.array(g["c0"], np.float32))
    ops.gemm(hip.asarray(np.array(g["a"], np.float32)),
             hip.asarray(np.array(g["b"], np.float32)), c, 1.0, 1.0)
    assert np.array_equal(_printed(c.asnumpy()), np.array(g["printed"]))


def _fixture_cases():
    sq = [np.zeros((4, 4), np.float32), np.ones((4, 4), np.float32),
          np.arange(16).reshape(4, 4).astype(np.float32)]
    rect = [np.zeros((4, 6), np.float32), np.ones((4, 6), np.float32),
            np.arange(24).reshape(4, 6).astype(np.float32)]
    rect_t = [a.T for a in rect]
    ab = GOLD["internal_gemm"]["alpha_beta"]
    return list(itertools.product(sq, sq, sq, ab, ab)) + \
        list(itertools.product(rect, rect_t, sq, ab, ab))


def test_internal_gemm_fixture_grid(env):
    """test_internal_gemm (tests/test_gpu.py:2141-2193): assert_equal."""
    hip, ops, orc, _ = env
    for a, b, c, alpha, beta in _fixture_cases():
        expect = (beta * c + alpha * np.dot(a, b)).astype(np.float32)
        d_c = hip.asarray(c.copy())
        ops.gemm(_to_dev(hip, a), _to_dev(hip, b), d_c, alpha, beta)
        got = d_c.asnumpy()
        assert np.array_equal(got, expect)
        assert np.array_equal(got, orc.gemm_f32(a, b, c.copy(), alpha, beta))


@pytest.mark.parametrize("ta,tb,tc", list(itertools.product([False, True], repeat=3)))
@pytest.mark.parametrize("m,n,k", [(33, 29, 47), (128, 128, 16), (1, 1, 1), (64, 1, 300),
                                   (256, 384, 64), (4096, 3072, 32), (4096, 3072, 48),
                                   (3072, 4096, 96), (300, 260, 100), (257, 129, 17),
                                   (1000, 1000, 1000), (131, 4100, 40), (1500, 2000, 52)])
def test_layouts_against_float64(env, ta, tb, tc, m, n, k):
    """Every stride pattern the entry point accepts (row/column major A, B, C)."""
    hip, ops, orc, mrt = env
    rng = np.random.default_rng(m * 1000 + n * 10 + k)
    a = rng.standard_normal((m, k), dtype=np.float32)
    b = rng.standard_normal((k, n), dtype=np.float32)
    c0 = rng.standard_normal((m, n), dtype=np.float32)
    lay = lambda x, t: np.asfortranarray(x) if t else x
    d_c = _to_dev(hip, lay(c0, tc))
    ops.gemm(_to_dev(hip, lay(a, ta)), _to_dev(hip, lay(b, tb)), d_c, 0.5, 2.0)
    got = d_c.asnumpy()
    mt, nt, kt = m - m % 128, n - n % 128, k - k % 16
    if (mt, nt, kt) == (m, n, k):
        # every layout of a tile-aligned problem runs on the matrix cores
        assert _kernel(mrt) in ("sgemm_mfma_128x128", "sgemm_mfma_256x256")
    elif -(-m // 128) * -(-n // 128) < 16:
        assert mrt.last_kernel() == "sgemm_generic"
    else:
        # whole tiles on the matrix cores, the edges on the strided kernel
        # (when the leading dimensions allow 128-bit loads)
        assert _kernel(mrt) in ("sgemm_generic", "sgemm_mfma_128x128+edges",
                                     "sgemm_mfma_256x256+edges", "sgemm_mfma_128x128_ragged")
    truth = 2.0 * c0 + 0.5 * (a.astype(np.float64) @ b.astype(np.float64))
    bound = 1e-5 * (2.0 * np.abs(c0) + 0.5 * (np.abs(a).astype(np.float64) @ np.abs(b))) + 1e-30
    assert (np.abs(got - truth) <= bound).all()


def _check_scaled(got, a, b, c0, alpha, beta, rel):
    truth = beta * c0.astype(np.float64) + alpha * (a.astype(np.float64) @ b.astype(np.float64))
    scale = abs(beta) * np.abs(c0) + abs(alpha) * (np.abs(a).astype(np.float64) @ np.abs(b))
    assert (np.abs(got - truth) <= rel * scale + 1e-30).all()


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("m,n,k", [(2000, 1500, 1000), (1540, 1420, 2004), (1412, 1536, 20),
                                   (4100, 4200, 36), (516, 520, 4)])
def test_ragged_shapes_on_tiles_that_read_zeros_outside(env, dtype, m, n, k, ta, tb):
    """Shapes that are not whole tiles but whose 128-bit words are whole run
    in one launch of tiles that read zeros beyond the operands and store only
    inside C: every layout, alpha and beta applied once to every element."""
    hip, ops, orc, mrt = env
    rng = np.random.default_rng(m + n + k)
    a = rng.standard_normal((m, k)).astype(dtype)
    b = rng.standard_normal((k, n)).astype(dtype)
    c0 = rng.standard_normal((m, n)).astype(dtype)
    lay = lambda x, t: np.asfortranarray(x) if t else x
    d_c = _to_dev(hip, c0)
    ops.gemm(_to_dev(hip, lay(a, ta)), _to_dev(hip, lay(b, tb)), d_c, 1.5, -0.5)
    assert _kernel(mrt).endswith("_mfma_128x128_ragged")
    _check_scaled(d_c.asnumpy(), a, b, c0, 1.5, -0.5, 1e-5 if dtype == np.float32 else 1e-13)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_ragged_k_alone_keeps_the_tiles(env, dtype):
    """Whole tiles in M and N, a K that is not whole slabs: the tiles as they
    are, the rest of K added by the strided kernel."""
    hip, ops, orc, mrt = env
    m, n, k = 1536, 2048, 100
    rng = np.random.default_rng(6)
    a = rng.standard_normal((m, k)).astype(dtype)
    b = rng.standard_normal((k, n)).astype(dtype)
    c0 = rng.standard_normal((m, n)).astype(dtype)
    d_c = hip.asarray(c0)
    ops.gemm(hip.asarray(a), hip.asarray(b), d_c, 1.5, -0.5)
    assert _kernel(mrt).endswith("_mfma_128x128+edges")
    _check_scaled(d_c.asnumpy(), a, b, c0, 1.5, -0.5, 1e-5 if dtype == np.float32 else 1e-13)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_operands_off_the_word_grid_are_repacked(env, dtype):
    """Operands whose rows do not begin or end on a 128-bit word (views of
    wider arrays, odd extents, a base inside a word) are copied once into
    word-aligned rows padded with zeros and run on the guarded tiles."""
    hip, ops, orc, mrt = env
    m, n, k = 1540, 2052, 1001
    rng = np.random.default_rng(5)
    a_wide = rng.standard_normal((m, k + 3)).astype(dtype)
    b = rng.standard_normal((k, n)).astype(dtype)
    c0 = rng.standard_normal((m, n)).astype(dtype)
    d_a = hip.asarray(a_wide)[:, :k]
    d_c = hip.asarray(c0)
    ops.gemm(d_a, hip.asarray(b), d_c, 1.5, -0.5)
    assert mrt.last_kernel().endswith("+packed") and "_mfma_128x128_ragged" in mrt.last_kernel()
    _check_scaled(d_c.asnumpy(), a_wide[:, :k], b, c0, 1.5, -0.5,
                  1e-5 if dtype == np.float32 else 1e-13)
    tol = 1e-5 if dtype == np.float32 else 1e-13
    lay = lambda x, t: np.asfortranarray(x) if t else x
    for (m, n, k), ta, tb, tc in (((1001, 1003, 1005), False, False, False),
                                  ((1001, 1003, 1005), True, False, True),
                                  ((777, 1025, 2049), True, True, False),
                                  ((513, 2047, 300), False, False, False),
                                  ((2047, 2049, 2051), False, False, False)):
        a = rng.standard_normal((m, k)).astype(dtype)
        b = rng.standard_normal((k, n)).astype(dtype)
        c0 = rng.standard_normal((m, n)).astype(dtype)
        d_c = _to_dev(hip, lay(c0, tc))
        ops.gemm(_to_dev(hip, lay(a, ta)), _to_dev(hip, lay(b, tb)), d_c, 1.5, -0.5)
        assert mrt.last_kernel().endswith("+packed"), mrt.last_kernel()
        _check_scaled(d_c.asnumpy(), a, b, c0, 1.5, -0.5, tol)
    # whole tiles, but the first operand starts one element into a word
    m = n = k = 1024
    a = rng.standard_normal((m, k)).astype(dtype)
    b = rng.standard_normal((k, n)).astype(dtype)
    flat = np.zeros(m * k + 1, dtype)
    flat[1:] = a.ravel()
    d_a = hip.asarray(flat)[1:].reshape(m, k)
    d_c = hip.asarray(np.full((m, n), np.nan, dtype))
    ops.gemm(d_a, hip.asarray(b), d_c, 1.0, 0.0)
    assert mrt.last_kernel().endswith("+packed")
    _check_scaled(d_c.asnumpy(), a, b, np.zeros((m, n), dtype), 1.0, 0.0, tol)


def test_copies_above_a_gigabyte_are_given_back(env):
    """The device keeps its gemm workspace between calls, but not more than
    1 GiB of it: a product whose padded copies need more (1.2 GB here) frees
    the block when it returns.  Rows of the result against float64."""
    import ctypes
    hip, ops, _, mrt = env
    hiprt = ctypes.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hiprt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    m, n, k = 12290, 12294, 12289
    rng = np.random.default_rng(11)
    a = rng.standard_normal((m, k), dtype=np.float32)
    b = rng.standard_normal((k, n), dtype=np.float32)
    d_a, d_b = hip.asarray(a), hip.asarray(b)
    d_c = hip.asarray(np.zeros((m, n), np.float32))
    ops.gemm(d_a, d_b, d_c, 1.0, 0.0)        # (whatever an earlier test left is freed too)
    before = free_bytes()
    for _ in range(2):
        ops.gemm(d_a, d_b, d_c, 1.0, 0.0)
        assert mrt.last_kernel() == "sgemm_mfma_256x256+packed"
        assert free_bytes() >= before - (64 << 20)
    got = d_c.asnumpy()
    rows = np.array([0, 1, 255, 256, 6000, m - 2, m - 1])
    truth = a[rows].astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(a[rows]).astype(np.float64) @ np.abs(b).astype(np.float64)
    assert (np.abs(got[rows] - truth) <= 1e-5 * scale).all()
    cols = np.array([0, 255, 256, n - 1])
    truth = a.astype(np.float64) @ b[:, cols].astype(np.float64)
    scale = np.abs(a).astype(np.float64) @ np.abs(b[:, cols]).astype(np.float64)
    assert (np.abs(got[:, cols] - truth) <= 1e-5 * scale).all()


# Tolerance for float32 matmul: |gpu - truth| <= 1e-4 * (|a| @ |b|) elementwise
# against a float64 ground truth, and relative 1e-4 in the Frobenius norm.
def _check(got, a, b):
    truth = a.astype(np.float64) @ b.astype(np.float64)
    bound = 1e-4 * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64))
    assert (np.abs(got - truth) <= bound).all()
    assert np.linalg.norm(got - truth) <= 1e-4 * np.linalg.norm(truth)


@pytest.mark.parametrize("m,n,k", [(128, 128, 16), (256, 384, 512), (128, 256, 4096),
                                   (1024, 1024, 1024), (384, 128, 48),
                                   (4096, 3072, 64), (3584, 3584, 16)])
def test_mfma_kernel(env, m, n, k):
    hip, ops, orc, mrt = env
    rng = np.random.Generator(np.random.PCG64(1005))
    a = rng.standard_normal((m, k), dtype=np.float32)
    b = rng.standard_normal((k, n), dtype=np.float32)
    got = ops.dot(hip.asarray(a), hip.asarray(b)).asnumpy()
    expect_kernel = "sgemm_mfma_256x256" if (m % 256 == 0 and n % 256 == 0 and
                                             (m // 256) * (n // 256) >= 192) \
        else "sgemm_mfma_128x128"
    assert _kernel(mrt) == expect_kernel
    _check(got, a, b)
    if m * n * k <= 1 << 27:
        # against the oracle's float32 contraction (k innermost)
        ref = orc.gemm_f32(a, b)
        bound = 2e-4 * (np.abs(a).astype(np.float64) @ np.abs(b))
        assert (np.abs(got - ref) <= bound).all()
    # alpha/beta epilogue on the MFMA path
    c0 = rng.standard_normal((m, n), dtype=np.float32)
    d_c = hip.asarray(c0.copy())
    ops.gemm(hip.asarray(a), hip.asarray(b), d_c, 0.5, -1.5)
    truth = -1.5 * c0 + 0.5 * (a.astype(np.float64) @ b.astype(np.float64))
    bound = 1e-4 * (1.5 * np.abs(c0) + 0.5 * (np.abs(a).astype(np.float64) @ np.abs(b)))
    assert (np.abs(d_c.asnumpy() - truth) <= bound).all()


def test_beta_zero_ignores_c(env):
    hip, ops, _, _ = env
    a = np.ones((128, 16), np.float32); b = np.ones((16, 128), np.float32)
    c = hip.asarray(np.full((128, 128), np.nan, np.float32))
    ops.gemm(hip.asarray(a), hip.asarray(b), c, 1.0, 0.0)
    assert (c.asnumpy() == 16).all()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_empty_extents(env, dtype):
    """No rows or no columns: nothing to write.  No inner dimension: the
    product is zero, so C becomes beta * C (and plain zeros for beta == 0,
    whatever C held)."""
    hip, ops, _, mrt = env
    for m, n in ((0, 5), (5, 0), (0, 0)):
        c = hip.asarray(np.zeros((m, n), dtype))
        ops.gemm(hip.asarray(np.ones((m, 7), dtype)), hip.asarray(np.ones((7, n), dtype)),
                 c, 1.0, 0.0)
        assert c.asnumpy().shape == (m, n)
    for m, n in ((5, 9), (130, 257)):
        c0 = np.arange(m * n, dtype=dtype).reshape(m, n)
        c = hip.asarray(c0)
        ops.gemm(hip.asarray(np.ones((m, 0), dtype)), hip.asarray(np.ones((0, n), dtype)),
                 c, 1.0, 2.0)
        assert np.array_equal(c.asnumpy(), 2 * c0)
        c = hip.asarray(np.full((m, n), np.nan, dtype))
        ops.gemm(hip.asarray(np.ones((m, 0), dtype)), hip.asarray(np.ones((0, n), dtype)),
                 c, 1.0, 0.0)
        assert np.array_equal(c.asnumpy(), np.zeros((m, n), dtype))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_tall_and_skinny(env, dtype):
    """2.2 million rows times an 8 x 8 matrix, and 9 million rows times a
    40 x 130 one: more rows of tiles than a launch has along y."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(17)
    for m, k, n in ((2_200_000, 8, 8), (9_000_000, 40, 130) if dtype is np.float32
                    else (4_500_000, 40, 130)):
        a = rng.standard_normal((m, k)).astype(dtype)
        b = rng.standard_normal((k, n)).astype(dtype)
        c = hip.asarray(np.full((m, n), np.nan, dtype))
        ops.gemm(hip.asarray(a), hip.asarray(b), c, 1.0, 0.0)
        got = c.asnumpy()
        for rows in (slice(0, 4096), slice(m // 2, m // 2 + 4096), slice(m - 4096, m)):
            truth = a[rows].astype(np.float64) @ b.astype(np.float64)
            scale = np.abs(a[rows]).astype(np.float64) @ np.abs(b).astype(np.float64)
            assert (np.abs(got[rows] - truth) <= (1e-5 if dtype is np.float32 else 1e-13)
                    * scale).all(), (m, k, n, mrt.last_kernel())
        assert np.isfinite(got).all()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("m,k,n", [(4096, 1, 1), (5000, 3, 3), (100_003, 8, 8), (70_001, 16, 5),
                                   (33_333, 32, 32), (65_537, 7, 29)])
def test_tall_times_small(env, dtype, m, k, n):
    """Coordinates times a small matrix (K, N <= 32): the streaming kernel.
    Row-major, a view of wider rows, a transposed small operand, alpha and
    beta; every element against float64."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(m + k + n)
    wide = rng.standard_normal((m, k + 3)).astype(dtype)
    b = rng.standard_normal((k, n)).astype(dtype)
    c0 = rng.standard_normal((m, n + 2)).astype(dtype)
    tol = 1e-5 if dtype == np.float32 else 1e-13
    for a_view, b_dev in ((hip.asarray(np.ascontiguousarray(wide[:, :k])), hip.asarray(b)),
                          (hip.asarray(wide)[:, :k], hip.asarray(np.asfortranarray(b)))):
        d_c = hip.asarray(c0)[:, :n]
        ops.gemm(a_view, b_dev, d_c, 1.5, -0.5)
        assert mrt.last_kernel() == ("sgemm_skinny" if dtype == np.float32 else "dgemm_skinny")
        _check_scaled(d_c.asnumpy(), wide[:, :k], b, c0[:, :n], 1.5, -0.5, tol)
        d_c = hip.asarray(np.full((m, n), np.nan, dtype))
        ops.gemm(a_view, b_dev, d_c, 1.0, 0.0)
        _check_scaled(d_c.asnumpy(), wide[:, :k], b, np.zeros((m, n), dtype), 1.0, 0.0, tol)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("m,k,n", [(1, 1, 4096), (3, 3, 5000), (8, 8, 100_003), (5, 16, 70_001),
                                   (32, 32, 33_333), (29, 7, 65_537)])
def test_small_times_long(env, dtype, m, k, n):
    """A small matrix times a long one (M, K <= 32): a lane per column.
    Row-major, views of wider rows, a transposed small operand, alpha and
    beta; every element against float64."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(m + k + n)
    a = rng.standard_normal((m, k)).astype(dtype)
    wide = rng.standard_normal((k, n + 5)).astype(dtype)
    c0 = rng.standard_normal((m, n + 3)).astype(dtype)
    tol = 1e-5 if dtype == np.float32 else 1e-13
    for a_dev, b_view in ((hip.asarray(a), hip.asarray(np.ascontiguousarray(wide[:, :n]))),
                          (hip.asarray(np.asfortranarray(a)), hip.asarray(wide)[:, :n])):
        d_c = hip.asarray(c0)[:, :n]
        ops.gemm(a_dev, b_view, d_c, 1.5, -0.5)
        assert mrt.last_kernel() == ("sgemm_wide" if dtype == np.float32 else "dgemm_wide")
        _check_scaled(d_c.asnumpy(), a, wide[:, :n], c0[:, :n], 1.5, -0.5, tol)
        d_c = hip.asarray(np.full((m, n), np.nan, dtype))
        ops.gemm(a_dev, b_view, d_c, 1.0, 0.0)
        _check_scaled(d_c.asnumpy(), a, wide[:, :n], np.zeros((m, n), dtype), 1.0, 0.0, tol)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("long,k,thin", [(1500, 100, 1), (1025, 33, 3), (2000, 1001, 8),
                                         (5000, 4099, 5), (1100, 70_000, 2), (40_000, 260, 4),
                                         (100, 70_000, 2), (64, 8192, 1), (700, 20_001, 8)])
def test_long_times_thin(env, dtype, long, k, thin):
    """A long matrix times a thin one (a vector, or up to eight of them) and a
    thin one times a long one, K > 32: the long operand is read once, by rows
    when it has unit stride along k, by columns otherwise (a long extent of
    64 to 1023 too where K is 8192 or more: K goes in slices over many blocks
    then).  Every layout of
    the three operands, rows that are and are not whole 128-bit words (views
    of wider rows), alpha and beta, a C of NaNs under beta = 0; every element
    against float64."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(long + k + thin)
    tol = 1e-5 if dtype == np.float32 else 1e-13
    prefix = "s" if dtype == np.float32 else "d"
    for m, n in ((long, thin), (thin, long)):
        a = rng.standard_normal((m, k)).astype(dtype)
        b = rng.standard_normal((k, n)).astype(dtype)
        c0 = rng.standard_normal((m, n)).astype(dtype)
        for fa in (False, True):
            for fb in (False, True):
                # the long operand decides: by rows when its unit stride is k's
                long_by_rows = (not fa) if m == long else fb
                want = prefix + ("gemm_thin_rows" if long_by_rows else "gemm_thin_cols")
                for fc in (False, True):
                    d_a = _to_dev(hip, a.T.copy().T if fa else a)
                    d_b = _to_dev(hip, b.T.copy().T if fb else b)
                    d_c = _to_dev(hip, c0.T.copy().T if fc else c0)
                    ops.gemm(d_a, d_b, d_c, 1.5, -0.5)
                    assert mrt.last_kernel() == want, (m, n, fa, fb, fc)
                    _check_scaled(d_c.asnumpy(), a, b, c0, 1.5, -0.5, tol)
        # views of rows three and four elements wider, and beta = 0 over NaNs
        for pad in (3, 4):
            wide_a = rng.standard_normal((m, k + pad)).astype(dtype)
            wide_b = rng.standard_normal((k, n + pad)).astype(dtype)
            d_a, d_b = hip.asarray(wide_a)[:, :k], hip.asarray(wide_b)[:, :n]
            d_c = hip.asarray(np.full((m, n), np.nan, dtype))
            ops.gemm(d_a, d_b, d_c, 1.0, 0.0)
            assert "gemm_thin" in mrt.last_kernel()
            _check_scaled(d_c.asnumpy(), wide_a[:, :k], wide_b[:, :n], np.zeros((m, n), dtype),
                          1.0, 0.0, tol)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("thin", [9, 12, 16])
def test_up_to_sixteen_vectors_against_columns(env, dtype, thin):
    """Nine to sixteen rows times a long matrix with unit stride along its
    long dimension (and the transposed problem) stay on the column kernel;
    with unit stride along k they go to the tiles."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(thin)
    k, long = 1000, 3004
    a = rng.standard_normal((thin, k)).astype(dtype)
    b = rng.standard_normal((k, long)).astype(dtype)
    c0 = rng.standard_normal((thin, long)).astype(dtype)
    tol = 1e-5 if dtype == np.float32 else 1e-13
    name = ("s" if dtype == np.float32 else "d") + "gemm_thin_cols"
    d_c = hip.asarray(c0)
    ops.gemm(hip.asarray(a), hip.asarray(b), d_c, 1.5, -0.5)
    assert mrt.last_kernel() == name
    _check_scaled(d_c.asnumpy(), a, b, c0, 1.5, -0.5, tol)
    # (b.T a.T): the long operand first, its unit stride still along `long`
    d_t = hip.asarray(np.ascontiguousarray(c0.T))
    ops.gemm(hip.asarray(b).T, hip.asarray(a).T, d_t, 1.5, -0.5)
    assert mrt.last_kernel() == name
    _check_scaled(d_t.asnumpy(), b.T, a.T, c0.T, 1.5, -0.5, tol)
    # unit stride along k: not this kernel's
    d_c = hip.asarray(c0)
    ops.gemm(hip.asarray(a), hip.asarray(np.ascontiguousarray(b.T)).T, d_c, 1.5, -0.5)
    assert "thin" not in mrt.last_kernel()
    _check_scaled(d_c.asnumpy(), a, b, c0, 1.5, -0.5, tol)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_thin_and_small_products_of_views_that_start_inside_a_word(env, dtype):
    """Operands that are views starting one element into a row: nothing is
    aligned to a 128-bit word, every kernel of these families reads by
    elements."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(31)
    tol = 1e-5 if dtype == np.float32 else 1e-13
    for m, k, n in ((2000, 1003, 3), (3, 1003, 2000), (5, 20_000, 7), (300, 9000, 1)):
        wa = rng.standard_normal((m, k + 2)).astype(dtype)
        wb = rng.standard_normal((k, n + 2)).astype(dtype)
        wc = rng.standard_normal((m, n + 2)).astype(dtype)
        d_a, d_b = hip.asarray(wa)[:, 1:k + 1], hip.asarray(wb)[:, 1:n + 1]
        d_w = hip.asarray(wc)
        ops.gemm(d_a, d_b, d_w[:, 1:n + 1], 1.5, -0.5)
        assert "thin" in mrt.last_kernel() or "inner" in mrt.last_kernel(), mrt.last_kernel()
        got = d_w.asnumpy()
        _check_scaled(got[:, 1:n + 1], wa[:, 1:k + 1], wb[:, 1:n + 1], wc[:, 1:n + 1],
                      1.5, -0.5, tol)
        # the columns of C beside the view are untouched
        assert np.array_equal(got[:, 0], wc[:, 0]) and np.array_equal(got[:, n + 1], wc[:, n + 1])
        # the transposed long operand
        d_at = hip.asarray(np.ascontiguousarray(wa.T))[1:k + 1].T
        d_w = hip.asarray(wc)
        ops.gemm(d_at, d_b, d_w[:, 1:n + 1], 1.0, 0.0)
        _check_scaled(d_w.asnumpy()[:, 1:n + 1], wa[:, 1:k + 1], wb[:, 1:n + 1],
                      np.zeros((m, n), dtype), 1.0, 0.0, tol)


@pytest.mark.parametrize("seed", range(6))
def test_shapes_drawn_round_the_limits_between_kernels(env, seed):
    """Extents drawn next to the limits at which one kernel hands over to
    another (thin extents of 8 and 16, long ones of 64, 1024 and 4096, K of
    32, 2048, 4096 and 8192, tile counts of 16 and 256), every layout,
    both types: whichever kernel serves, every element against float64."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(1000 + seed)
    small = [1, 2, 3, 4, 5, 7, 8, 9, 12, 15, 16, 17, 31, 32, 33]
    long = [63, 64, 65, 127, 129, 500, 1023, 1024, 1025, 4095, 4096, 4100]
    depth = [31, 32, 33, 40, 255, 2047, 2048, 2050, 4095, 4096, 4097, 8191, 8192, 8200, 20_000]
    for _ in range(16):
        kind = rng.integers(0, 4)
        if kind == 0:
            m, n = rng.choice(long), rng.choice(small)
        elif kind == 1:
            m, n = rng.choice(small), rng.choice(long)
        elif kind == 2:
            m, n = rng.choice(small), rng.choice(small)
        else:
            m, n = rng.choice(long[:8]), rng.choice(long[:8])
        k = int(rng.choice(depth))
        m, n = int(m), int(n)
        dtype = np.float32 if rng.integers(0, 2) else np.float64
        fa, fb, fc = (bool(rng.integers(0, 2)) for _ in range(3))
        alpha, beta = ((1.0, 0.0), (1.5, -0.5))[int(rng.integers(0, 2))]
        a = rng.standard_normal((m, k)).astype(dtype)
        b = rng.standard_normal((k, n)).astype(dtype)
        c0 = rng.standard_normal((m, n)).astype(dtype)
        d_a = _to_dev(hip, a.T.copy().T if fa else a)
        d_b = _to_dev(hip, b.T.copy().T if fb else b)
        d_c = _to_dev(hip, c0.T.copy().T if fc else c0)
        ops.gemm(d_a, d_b, d_c, alpha, beta)
        case = (m, k, n, np.dtype(dtype).name, fa, fb, fc, alpha, beta, mrt.last_kernel())
        truth = beta * c0.astype(np.float64) + alpha * (a.astype(np.float64) @ b.astype(np.float64))
        scale = abs(beta) * np.abs(c0) + abs(alpha) * (np.abs(a).astype(np.float64) @ np.abs(b))
        rel = 1e-5 if dtype == np.float32 else 1e-13
        assert (np.abs(d_c.asnumpy() - truth) <= rel * scale + 1e-30).all(), case


def test_thin_products_do_not_mix_in_what_lies_beyond(env):
    """An infinity in the long operand's padding, or in the thin one's, stays
    out of the sums (a product with zero would make it a NaN)."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(11)
    m, k = 3000, 1030
    wide = rng.standard_normal((m, k + 2)).astype(np.float32)
    wide[:, k:] = np.inf
    v = rng.standard_normal((k + 1, 1)).astype(np.float32)
    v[k] = np.inf
    d_c = hip.asarray(np.zeros((m, 1), np.float32))
    ops.gemm(hip.asarray(wide)[:, :k], hip.asarray(v)[:k], d_c, 1.0, 0.0)
    assert mrt.last_kernel() == "sgemm_thin_rows"
    _check_scaled(d_c.asnumpy(), wide[:, :k], v[:k], np.zeros((m, 1), np.float32), 1.0, 0.0, 1e-5)
    d_r = hip.asarray(np.zeros((1, m), np.float32))
    row = hip.asarray(np.ascontiguousarray(v.T))[:, :k]
    ops.gemm(row, _to_dev(hip, wide.T)[:k], d_r, 1.0, 0.0)
    assert "gemm_thin" in mrt.last_kernel()
    _check_scaled(d_r.asnumpy(), v[:k].T, wide[:, :k].T, np.zeros((1, m), np.float32), 1.0, 0.0,
                  1e-5)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("k,m,n", [(1 << 18, 8, 8), (300_001, 8, 1), (1 << 20, 3, 3), (5000, 4, 8),
                                   (70_000, 5, 2), (4096, 1, 1)])
def test_small_products_of_long_operands(env, dtype, k, m, n):
    """X.T @ Y for tall X and Y of a few columns (a Gram matrix, the right-hand
    side of normal equations): slices of K on many blocks, partial sums added
    in a fixed order.  Transposed views of row-major operands (rows read as
    words where m and n are 4 or 8), row-major ones, views of wider rows,
    alpha and beta, C in both layouts; every element against float64, and
    twice the same bits."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(k + m + n)
    x = rng.standard_normal((k, m + 1)).astype(dtype)
    y = rng.standard_normal((k, n + 1)).astype(dtype)
    c0 = rng.standard_normal((m, n)).astype(dtype)
    tol = 1e-5 if dtype == np.float32 else 1e-13
    name = "sgemm_inner" if dtype == np.float32 else "dgemm_inner"
    xs, ys = np.ascontiguousarray(x[:, :m]), np.ascontiguousarray(y[:, :n])
    cases = [(hip.asarray(xs).T, hip.asarray(ys)),                          # rows of m and n
             (hip.asarray(x)[:, :m].T, hip.asarray(y)[:, :n]),              # of wider rows
             (hip.asarray(np.ascontiguousarray(xs.T)), hip.asarray(ys)),    # X.T row-major
             (hip.asarray(xs).T, hip.asarray(np.ascontiguousarray(ys.T)).T)]
    for d_a, d_b in cases:
        for fc in (False, True):
            d_c = _to_dev(hip, c0.T.copy().T if fc else c0)
            ops.gemm(d_a, d_b, d_c, 1.5, -0.5)
            assert mrt.last_kernel() == name
            first = d_c.asnumpy()
            _check_scaled(first, xs.T, ys, c0, 1.5, -0.5, tol)
            d_c = _to_dev(hip, c0.T.copy().T if fc else c0)
            ops.gemm(d_a, d_b, d_c, 1.5, -0.5)
            assert np.array_equal(d_c.asnumpy(), first)
    d_c = hip.asarray(np.full((m, n), np.nan, dtype))
    ops.gemm(cases[0][0], cases[0][1], d_c, 1.0, 0.0)
    _check_scaled(d_c.asnumpy(), xs.T, ys, np.zeros((m, n), dtype), 1.0, 0.0, tol)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("m,k,n", [(16, 1 << 18, 16), (32, 100_003, 20), (100, 50_000, 60),
                                   (128, 1 << 17, 128), (300, 1 << 15, 300), (10, 4099, 12)])
def test_few_tiles_with_a_long_k(env, dtype, m, k, n):
    """Results of a few tiles from long operands: K is cut into as many
    slices as fill the GPU, on the strided kernel for the smallest results
    and on the guarded tiles from a quarter of a tile on."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(m + k + n)
    x = rng.standard_normal((k, m)).astype(dtype)
    b = rng.standard_normal((k, n)).astype(dtype)
    c0 = rng.standard_normal((m, n)).astype(dtype)
    tol = 1e-5 if dtype == np.float32 else 1e-13
    for d_a, a in ((hip.asarray(x).T, x.T), (hip.asarray(np.ascontiguousarray(x.T)), x.T)):
        d_c = hip.asarray(c0)
        ops.gemm(d_a, hip.asarray(b), d_c, 1.5, -0.5)
        assert "_splitk" in mrt.last_kernel(), mrt.last_kernel()
        assert ("generic" in mrt.last_kernel()) == (m * n < 4096)
        _check_scaled(d_c.asnumpy(), a, b, c0, 1.5, -0.5, tol)


def test_identity_and_linearity_full_size(env):
    """Configuration 5 (4096^3): rows checked against float64, plus
    size-independent properties: A @ I == A exactly, and linearity."""
    hip, ops, _, mrt = env
    from numba_mlir_amd import workloads
    A, B = workloads.matmul()
    d_A, d_B = hip.asarray(A), hip.asarray(B)
    C = ops.dot(d_A, d_B).asnumpy()
    assert mrt.last_kernel().startswith("sgemm_mfma")
    # every element against the float64 product, in blocks of 512 rows
    B64, absB = B.astype(np.float64), np.abs(B).astype(np.float64)
    err2 = ref2 = 0.0
    for r0 in range(0, 4096, 512):
        rows = slice(r0, r0 + 512)
        truth = A[rows].astype(np.float64) @ B64
        bound = 1e-4 * (np.abs(A[rows]).astype(np.float64) @ absB)
        diff = C[rows] - truth
        assert (np.abs(diff) <= bound).all(), r0
        err2 += float((diff * diff).sum())
        ref2 += float((truth * truth).sum())
    assert err2 <= (1e-4) ** 2 * ref2
    eye = hip.asarray(np.eye(4096, dtype=np.float32))
    assert np.array_equal(ops.dot(d_A, eye).asnumpy(), A)
    assert np.array_equal(ops.dot(eye, d_B).asnumpy(), B)
    # numpy's own float32 sgemm as a second reference, every element
    np.testing.assert_allclose(C, np.dot(A, B), rtol=0, atol=1e-4 * 64 * 3)


@pytest.mark.parametrize("ta,tb,tc", list(itertools.product([False, True], repeat=3)))
@pytest.mark.parametrize("m,n,k", [(128, 128, 16), (256, 384, 80), (1024, 1024, 1024)])
def test_float64_mfma(env, ta, tb, tc, m, n, k):
    """mkl_gemm_float64_device on the fp64 matrix cores, every layout; the
    tolerance is rel 1e-5 (float64 bar), met with a wide margin."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(m + n + k)
    a, b = rng.standard_normal((m, k)), rng.standard_normal((k, n))
    c0 = rng.standard_normal((m, n))
    lay = lambda x, t: np.asfortranarray(x) if t else x
    d_c = _to_dev(hip, lay(c0, tc))
    ops.gemm(_to_dev(hip, lay(a, ta)), _to_dev(hip, lay(b, tb)), d_c, 1.25, -0.5)
    assert _kernel(mrt) == "dgemm_mfma_128x128"
    got = d_c.asnumpy()
    truth = -0.5 * c0 + 1.25 * (a @ b)
    bound = 1e-13 * (0.5 * np.abs(c0) + 1.25 * (np.abs(a) @ np.abs(b)))
    assert (np.abs(got - truth) <= bound).all()
    np.testing.assert_allclose(got, truth, rtol=1e-5, atol=1e-9)


def test_float64_gemm(env):
    hip, ops, _, mrt = env
    rng = np.random.default_rng(4)
    a, b = rng.standard_normal((70, 90)), rng.standard_normal((90, 50))
    got = ops.dot(hip.asarray(a), hip.asarray(b)).asnumpy()
    np.testing.assert_allclose(got, a @ b, rtol=1e-12, atol=1e-12)


# ---- split K: few tiles, long K ------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("ta,tb,tc", [(False, False, False), (True, False, False),
                                      (False, True, True), (True, True, False)])
@pytest.mark.parametrize("m,n,k", [(1024, 1024, 1024), (128, 256, 4096), (512, 384, 2000),
                                   (1000, 1000, 1000), (640, 516, 1028), (1280, 1280, 272)])
def test_split_k(env, dtype, ta, tb, tc, m, n, k):
    """Shapes with too few tiles to fill the GPU cut K into slices whose
    partial products are added in slice order: every layout, alpha and beta
    applied once, K that is not a whole number of slices or slabs, and the
    same bits on a second run."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    a = rng.standard_normal((m, k)).astype(dtype)
    b = rng.standard_normal((k, n)).astype(dtype)
    c0 = rng.standard_normal((m, n)).astype(dtype)
    lay = lambda x, t: np.asfortranarray(x) if t else x
    d_a, d_b = _to_dev(hip, lay(a, ta)), _to_dev(hip, lay(b, tb))
    runs = []
    for _ in range(2):
        d_c = _to_dev(hip, lay(c0, tc))
        ops.gemm(d_a, d_b, d_c, 1.5, -0.5)
        assert "_splitk" in mrt.last_kernel() or "_even" in mrt.last_kernel(), mrt.last_kernel()
        runs.append(d_c.asnumpy())
    assert np.array_equal(runs[0], runs[1])
    _check_scaled(runs[0], a, b, c0, 1.5, -0.5, 1e-5 if dtype == np.float32 else 1e-13)


def test_split_k_beta_zero_ignores_c(env):
    hip, ops, _, mrt = env
    a = np.ones((256, 2048), np.float32)
    b = np.ones((2048, 256), np.float32)
    c = hip.asarray(np.full((256, 256), np.nan, np.float32))
    ops.gemm(hip.asarray(a), hip.asarray(b), c, 1.0, 0.0)
    assert "_splitk" in mrt.last_kernel()
    assert (c.asnumpy() == 2048).all()


# ---- even shares: the K slabs of all tiles dealt out to the resident blocks ------

@pytest.mark.parametrize("dtype,m,n,k,kernel", [
    # 576 tiles of 256 x 256, eight slabs each: a share is 2.25 tiles (the end
    # of one, a whole one, the beginning of the next)
    (np.float32, 6144, 6144, 256, "sgemm_mfma_256x256_even"),
    # 64 tiles on 256 blocks: every tile in four pieces
    (np.float32, 2048, 2048, 1024, "sgemm_mfma_256x256_even"),
    # (fewer than 64 large tiles: the small ones, here in four slices of K)
    (np.float32, 1024, 1024, 4096, "sgemm_mfma_128x128_splitk"),
    (np.float32, 2048, 2048, 2048 + 16, "sgemm_mfma_256x256_even"),   # slabs of 16
    (np.float32, 1536, 1408, 2056, "sgemm_mfma_128x128_even+edges"),  # the rest of K beside
    (np.float32, 1500, 1500, 1200, "sgemm_mfma_128x128_ragged_even"),
    (np.float32, 1000, 1100, 1200, "sgemm_mfma_128x128_ragged_splitk"),  # 72 tiles x 7 on 512 blocks
    (np.float32, 2000, 2300, 2600, "sgemm_mfma_128x128_ragged_even"),
    # from 192 padded tiles on, ragged float32 shapes run on the large tile over
    # zero-padded copies of both operands: 210 tiles in even shares, 256 as they are
    (np.float32, 3560, 3800, 1020, "sgemm_mfma_256x256_even+packed"),
    (np.float32, 4000, 4000, 530, "sgemm_mfma_256x256+packed"),
    (np.float64, 3072, 3072, 512, "dgemm_mfma_128x128_even"),         # 1.125 rounds
    (np.float64, 1536, 1536, 2048, "dgemm_mfma_128x128_even"),        # 144 tiles: 3 slices fill 0.84
    (np.float64, 1500, 1500, 1200, "dgemm_mfma_128x128_ragged_even"),
    # equal slices of K go first where they fill the blocks: 64 tiles x 8, 72 x 7
    (np.float64, 1024, 1024, 4096, "dgemm_mfma_128x128_splitk"),
    (np.float64, 1000, 1100, 1200, "dgemm_mfma_128x128_ragged_splitk"),  # the reference's preset
    (np.float32, 1152, 1152, 1152, "sgemm_mfma_128x128_splitk"),
    # float64 from 256 padded tiles on: the same tile over zero-padded copies
    (np.float64, 2500, 2750, 3000, "dgemm_mfma_128x128_even+packed"),
    (np.float64, 2040, 4090, 600, "dgemm_mfma_128x128+packed"),
])
@pytest.mark.parametrize("ta,tb,tc", [(False, False, False), (True, False, True),
                                      (False, True, False)])
def test_even_shares(env, dtype, m, n, k, kernel, ta, tb, tc):
    """Whole tiles that would leave most CUs idle (too few, or a nearly empty
    last round): the blocks take equal shares of all K slabs, pieces of tiles
    meet in the workspace and are added in K order.  Every element against
    float64, alpha and beta applied once, the same bits on a second run."""
    hip, ops, _, mrt = env
    rng = np.random.default_rng(m + 3 * n + 7 * k)
    a = rng.standard_normal((m, k)).astype(dtype)
    b = rng.standard_normal((k, n)).astype(dtype)
    c0 = rng.standard_normal((m, n)).astype(dtype)
    lay = lambda x, t: np.asfortranarray(x) if t else x
    d_a, d_b = _to_dev(hip, lay(a, ta)), _to_dev(hip, lay(b, tb))
    runs = []
    for _ in range(2):
        d_c = _to_dev(hip, lay(c0, tc))
        ops.gemm(d_a, d_b, d_c, 1.5, -0.5)
        if not tc:       # (a column-major C swaps the operands: another tile count)
            assert mrt.last_kernel() == kernel
        runs.append(d_c.asnumpy())
    assert np.array_equal(runs[0], runs[1])
    _check_scaled(runs[0], a, b, c0, 1.5, -0.5, 1e-5 if dtype == np.float32 else 1e-13)


def test_even_shares_beta_zero_ignores_c_and_the_no_alloc_entry_keeps_slices(env):
    hip, ops, _, mrt = env
    a = np.ones((2048, 1024), np.float32)
    b = np.ones((1024, 2048), np.float32)
    c = hip.asarray(np.full((2048, 2048), np.nan, np.float32))
    ops.gemm(hip.asarray(a), hip.asarray(b), c, 1.0, 0.0)
    assert "_even" in mrt.last_kernel()
    assert (c.asnumpy() == 1024).all()


def test_calls_from_two_threads_take_turns_on_the_workspace(env):
    """Two host threads, each with a queue of its own, multiply at the same
    time through the raw C-ABI (ctypes drops the GIL for the call): products
    that go through the device's one workspace must not mix."""
    import ctypes
    import threading
    hip, ops, _, mrt = env
    from numba_mlir_amd.mlir import gpu_runtime

    class Memref2(ctypes.Structure):
        _fields_ = [("userData", ctypes.c_void_p), ("data", ctypes.c_void_p),
                    ("offset", ctypes.c_size_t), ("dims", ctypes.c_size_t * 2),
                    ("strides", ctypes.c_size_t * 2)]

    def memref(arr):
        r = Memref2()
        r.userData, r.data, r.offset = None, arr.ptr, 0
        r.dims[0], r.dims[1] = arr.shape
        r.strides[0], r.strides[1] = arr.elem_strides
        return r

    lib = mrt.runtime_hip_lib
    gemm = lib.mkl_gemm_float32_device
    gemm.restype = None
    gemm.argtypes = [ctypes.c_void_p, ctypes.POINTER(Memref2), ctypes.POINTER(Memref2),
                     ctypes.c_float, ctypes.c_float, ctypes.POINTER(Memref2)]
    rt = gpu_runtime.runtime_lib
    shapes = [(1024, 1024, 2048), (640, 768, 4096)]      # both share K out over the blocks
    work = []
    for seed, (m, n, k) in enumerate(shapes):
        rng = np.random.default_rng(seed)
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = rng.standard_normal((k, n)).astype(np.float32)
        work.append((a, b, hip.asarray(a), hip.asarray(b),
                     hip.asarray(np.zeros((m, n), np.float32)), rt.gpuxQueueCreate(None)))
    errors = []

    def run(item):
        a, b, d_a, d_b, d_c, queue = item
        try:
            for _ in range(25):
                gemm(queue, memref(d_a), memref(d_b), 1.0, 0.0, memref(d_c))
        except Exception as exc:      # noqa: BLE001
            errors.append(exc)

    threads = [threading.Thread(target=run, args=(item,)) for item in work]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors
    for a, b, d_a, d_b, d_c, queue in work:
        truth = a.astype(np.float64) @ b.astype(np.float64)
        scale = np.abs(a).astype(np.float64) @ np.abs(b)
        assert (np.abs(d_c.asnumpy() - truth) <= 1e-4 * scale).all()
        rt.gpuxQueueDestroy(queue)
