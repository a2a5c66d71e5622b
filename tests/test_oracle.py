"""Pins the CPU oracle (oracle/) before anything is compared against it.

Every check here is independent of the oracle's own formula: vectors the
reference's tests hold (tests/golden/reference_vectors.json), closed forms,
library routines, brute force, invariants.
"""

import json
import math
import os

import numpy as np
import pytest

from oracle import oracle as orc
from oracle.kernel_sim import kernel_sim

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
    GOLD = json.load(f)


def _printed(x):
    """What MLIR's printMemrefF32 shows: 6 significant digits."""
    return np.array([float("%.6g" % v) for v in np.ravel(x)]).reshape(np.shape(x))


# -- add / broadcast ----------------------------------------------------------
def test_add_golden_addf():
    g = GOLD["addf"]
    out = orc.add(np.array(g["a"], np.float32), np.array(g["b"], np.float32))
    assert np.array_equal(_printed(out), np.array(g["printed"]))


def test_add_golden_linalg_addf():
    g = GOLD["linalg_addf"]
    out = orc.add(np.array(g["a"], np.float32), np.array(g["b"], np.float32))
    assert np.array_equal(out, np.array(g["out"], np.float32))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_fused_map_golden_linalg_test(dtype):
    """linalg_test_f32.mlir / _f64.mlir: the nineteen one-op linalg.generic
    steps of @foo, each rounded in the tensor's type, print 500 x 1.00002."""
    g = GOLD["linalg_test"]
    a = np.full(g["n"], g["a"], dtype)
    s = [dtype(v) for v in g["s"]]
    v11, v13, v15 = s[0] + s[1], s[4] - s[3], -s[2]
    t19 = a - s[0]
    t27 = np.exp(v15 * t19) + a
    t35 = s[3] + v13 / t27
    out = v11 + t35 * (a - s[0])
    assert out.dtype == dtype
    assert np.array_equal(_printed(out), np.full(g["n"], g["printed"]))
    # the correction term is what the print shows: 4 / (e^12 + 1)
    # (t35 * -4 is near -8, where float32 numbers are 1e-6 apart)
    assert abs(float(out[0]) - (1 + 4 / (np.exp(12.0) + 1))) < (2e-6 if dtype is np.float32 else 1e-14)


@pytest.mark.parametrize("i", range(6))
@pytest.mark.parametrize("j", range(6))
def test_add_broadcast_fixtures(i, j):
    arrs = [np.array(a, np.int64) for a in GOLD["broadcast_arrays"]["arrays"]]
    a, b = arrs[i], arrs[j]
    out = orc.add(a, b)
    expect = np.add(a, b)
    assert out.shape == expect.shape and np.array_equal(out, expect)


def test_add_f64_bit_exact_and_thread_independent():
    rng = np.random.default_rng(5)
    a = rng.uniform(-1, 1, (257, 131))
    b = rng.uniform(-1, 1, (1, 131))
    expect = a + b
    for threads in (1, 3, 8):
        out = orc.add(a, b, threads)
        assert out.tobytes() == expect.tobytes()
    # a transposed operand (non-unit strides) goes through the same loop
    out = orc.add(np.asfortranarray(a), b)
    assert out.tobytes() == expect.tobytes()


# -- Black-Scholes -------------------------------------------------------------
def _bs_inputs(n):
    from numba_mlir_amd import workloads
    return workloads.black_scholes(n)


def test_black_scholes_generator_matches_reference_recipe():
    # legacy seed + three uniform draws in float64, cast to float32
    price, strike, t, rate, vol, call, put = _bs_inputs(1000)
    rs = np.random.RandomState(777777)
    p2 = rs.uniform(10.0, 50.0, 1000).astype(np.float32)
    assert np.array_equal(price, p2)
    assert rate == np.float32(0.1) and vol == np.float32(0.2)
    assert (call == 0).all() and (put == -1).all()
    assert 10 <= price.min() and price.max() <= 50 and 1 <= t.min() <= t.max() <= 2


def test_black_scholes_against_closed_form():
    n = GOLD["black_scholes"]["nopt"]
    price, strike, t, rate, vol, _, _ = _bs_inputs(n)
    tc, tp = orc.black_scholes_truth(price, strike, t, rate, vol)
    for wide in (True, False):
        c, p = orc.black_scholes(price, strike, t, rate, vol, wide)
        # the reference's own bar between its two evaluations
        np.testing.assert_allclose(c, tc, atol=GOLD["black_scholes"]["atol"])
        np.testing.assert_allclose(p, tp, atol=GOLD["black_scholes"]["atol"])
    # float64-literal typing keeps relative accuracy even in the tails
    c, p = orc.black_scholes(price, strike, t, rate, vol, True)
    np.testing.assert_allclose(c, tc, rtol=5e-5, atol=1e-12)
    np.testing.assert_allclose(p, tp, rtol=5e-5, atol=1e-12)


def test_black_scholes_put_call_parity():
    price, strike, t, rate, vol, _, _ = _bs_inputs(1 << 16)
    c, p = orc.black_scholes(price, strike, t, rate, vol, True)
    disc = strike.astype(np.float64) * np.exp(-float(rate) * t.astype(np.float64))
    np.testing.assert_allclose(c.astype(np.float64) - p, price - disc,
                               rtol=0, atol=2e-5)


def test_black_scholes_sign_and_operand_sensitivity():
    # swapping price and strike, or flipping the rate's sign, must change the
    # answer well beyond the tolerance: guards the truth against a transposed
    # operand or a dropped minus.
    price, strike, t, rate, vol, _, _ = _bs_inputs(4096)
    c, _ = orc.black_scholes(price, strike, t, rate, vol, True)
    c_swapped, _ = orc.black_scholes(strike, price, t, rate, vol, True)
    c_neg, _ = orc.black_scholes(price, strike, t, -rate, vol, True)
    assert np.abs(c - c_swapped).max() > 1.0
    assert np.abs(c - c_neg).max() > 0.1
    # at-the-money, zero rate: call = P * (2 N(sigma sqrt(T) / 2) - 1)
    P = np.full(8, 30.0, np.float32)
    T = np.full(8, 1.5, np.float32)
    c0, p0 = orc.black_scholes(P, P, T, 0.0, vol, True)
    expect = 30.0 * math.erf(float(np.float32(vol)) * math.sqrt(1.5) / 2 / math.sqrt(2))
    np.testing.assert_allclose(c0, expect, rtol=1e-6)
    np.testing.assert_allclose(p0, expect, rtol=1e-6)


# -- reductions ---------------------------------------------------------------
def test_reduce_small_golden():
    g = GOLD["reduce_axis_small"]
    a32 = np.array(g["arr"], np.float32)
    ai = np.array(g["arr"], np.int32)
    assert orc.sum_axis1_f32(a32).tolist() == g["sum_axis1"]
    out = orc.sum_axis0_i32(ai)
    assert out.dtype == np.int64 and out.tolist() == g["sum_axis0"]


@pytest.mark.parametrize("n0", GOLD["reduce_shapes"]["dims_2d"])
@pytest.mark.parametrize("n1", GOLD["reduce_shapes"]["dims_2d"])
def test_reduce_arange_shapes(n0, n1):
    count = n0 * n1
    a = np.arange(1, count + 1, dtype=np.float32).reshape(n0, n1)
    # arange sums are exact in float32 below 2^24: closed form per row
    rows = np.array([n1 * (2 * (r * n1 + 1) + (n1 - 1)) / 2 for r in range(n0)])
    assert np.array_equal(orc.sum_axis1_f32(a), rows.astype(np.float32))
    ai = np.arange(1, count + 1, dtype=np.int32).reshape(n0, n1)
    cols = np.array([n0 * (c + 1) + n1 * n0 * (n0 - 1) // 2 for c in range(n1)])
    assert np.array_equal(orc.sum_axis0_i32(ai), cols)


def test_sum_axis0_int64_no_overflow():
    x = np.full((70000, 3), 2 ** 31 - 1, np.int32)
    assert orc.sum_axis0_i32(x).tolist() == [70000 * (2 ** 31 - 1)] * 3
    x = np.full((70000, 3), -2 ** 31, np.int32)
    assert orc.sum_axis0_i32(x).tolist() == [-70000 * 2 ** 31] * 3


def test_float_reductions_within_rounding_bound():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((300, 4099), dtype=np.float32)
    truth = x.astype(np.float64).sum(axis=1)
    got = orc.sum_axis1_f32(x)
    # sequential float32 sum: |err| <= n * eps * sum|x|
    bound = 4099 * 2.0 ** -24 * np.abs(x).astype(np.float64).sum(axis=1)
    assert (np.abs(got - truth) <= bound).all()
    # Full reduction: per-thread sequential float32 accumulators.  With n
    # positive terms the relative error of the sum is below n * 2^-24 (it is
    # what a reference run with few threads would show as well), so the bound
    # is loose on 1.2M terms and tight on a short input.
    sq = float((x.astype(np.float64) ** 2).sum())
    for threads in (1, 4, 8):
        got2 = float(orc.norm2_f32(x, threads)) ** 2
        assert abs(got2 - sq) <= x.size * 2.0 ** -24 * sq
    y = x[:40, :500]
    t2 = math.sqrt(float((y.astype(np.float64) ** 2).sum()))
    for threads in (1, 4, 8):
        assert abs(float(orc.norm2_f32(y, threads)) - t2) <= 1e-4 * t2


def test_norm2_exact_cases():
    assert orc.norm2_f32(np.array([3, 4], np.float32)) == 5
    assert orc.norm2_f32(np.array([2, 3, 6], np.float32)) == 7
    x = np.zeros(4096, np.float32)
    x[::64] = 2          # 64 values of 2 -> sqrt(256) = 16
    for threads in (1, 2, 8):
        assert orc.norm2_f32(x, threads) == 16
    assert orc.norm2_f32(np.zeros(0, np.float32)) == 0


# -- pairwise -----------------------------------------------------------------
def test_pairwise_reference_fixture_closed_form():
    g = GOLD["pairwise"]
    n, d = g["npoints"], g["dims"]
    a = np.arange(n * d, dtype=np.float32).reshape(n, d)
    b = a + 5
    D = orc.pairwise(a, b)
    i, j = np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
    expect = math.sqrt(3.0) * np.abs(3.0 * (i - j) - 5.0)
    np.testing.assert_allclose(D, expect, rtol=g["rtol"])
    D64 = orc.pairwise(a.astype(np.float64), b.astype(np.float64))
    np.testing.assert_allclose(D64, expect, rtol=1e-14)


def test_pairwise_against_cdist_and_brute_force():
    from scipy.spatial.distance import cdist
    rng = np.random.default_rng(3)
    X, Y = rng.uniform(0, 1, (37, 3)), rng.uniform(0, 1, (53, 3))
    D = orc.pairwise(X, Y)
    np.testing.assert_allclose(D, cdist(X, Y), rtol=1e-14)
    brute = np.empty_like(D)
    for i in range(37):
        for j in range(53):
            d = 0.0
            for k in range(3):
                tmp = X[i, k] - Y[j, k]
                d += tmp * tmp
            brute[i, j] = math.sqrt(d)
    assert D.tobytes() == brute.tobytes()      # same op order: bit-equal
    assert not np.allclose(D[:37, :37], orc.pairwise(Y, X)[:37, :37])  # argument order matters


# -- gemm ---------------------------------------------------------------------
def test_gemm_golden_dot():
    g = GOLD["dot_2d"]
    out = orc.gemm_f32(np.array(g["a"], np.float32), np.array(g["b"], np.float32))
    assert np.array_equal(out, np.array(g["out"], np.float32))


def test_gemm_golden_linalg_gemmf():
    g = GOLD["linalg_gemmf"]
    c = np.array(g["c0"], np.float32)
    out = orc.gemm_f32(np.array(g["a"], np.float32), np.array(g["b"], np.float32),
                       c, 1.0, 1.0)
    assert np.array_equal(_printed(out), np.array(g["printed"]))


def test_gemv_golden_as_gemm_column():
    g = GOLD["linalg_gemvf"]
    a = np.array(g["a"], np.float32)
    x = np.array(g["x"], np.float32).reshape(3, 1)
    y = np.array(g["y0"], np.float32).reshape(3, 1).copy()
    out = orc.gemm_f32(a, x, y, 1.0, 1.0)
    assert np.array_equal(_printed(out.ravel()), np.array(g["printed"]))


def _gemm_fixture_arrays():
    sq = [np.zeros((4, 4), np.float32), np.ones((4, 4), np.float32),
          np.arange(16).reshape(4, 4).astype(np.float32)]
    rect = [np.zeros((4, 6), np.float32), np.ones((4, 6), np.float32),
            np.arange(24).reshape(4, 6).astype(np.float32)]
    return sq, rect, [a.T for a in rect]


def test_gemm_internal_gemm_fixture_grid():
    import itertools
    sq, rect, rect_t = _gemm_fixture_arrays()
    ab = GOLD["internal_gemm"]["alpha_beta"]
    cases = list(itertools.product(sq, sq, sq, ab, ab)) + \
        list(itertools.product(rect, rect_t, sq, ab, ab))
    for a, b, c, alpha, beta in cases:
        expect = beta * c + alpha * np.dot(a, b)      # __internal_gemm's body
        got = orc.gemm_f32(a, b, c.copy(), alpha, beta)
        assert np.array_equal(got, expect.astype(np.float32))


def test_gemm_random_against_float64_and_layouts():
    rng = np.random.default_rng(9)
    a = rng.standard_normal((33, 47), dtype=np.float32)
    b = rng.standard_normal((47, 29), dtype=np.float32)
    truth = a.astype(np.float64) @ b.astype(np.float64)
    np.testing.assert_allclose(orc.gemm_f32_truth(a, b), truth, rtol=1e-13,
                               atol=1e-13)
    bound = 47 * 2.0 ** -23 * (np.abs(a).astype(np.float64) @ np.abs(b))
    for aa in (a, np.asfortranarray(a)):
        for bb in (b, np.asfortranarray(b)):
            got = orc.gemm_f32(aa, bb)
            assert (np.abs(got - truth) <= bound).all()
    assert not np.allclose(orc.gemm_f32(a, b), orc.gemm_f32(a, b[::-1]))


# -- block-size suggestion ------------------------------------------------------
@pytest.mark.parametrize("global_size,expect", [
    ((1,), (1,)), ((7,), (7,)), ((1, 1), (1, 1)), ((7, 13), (7, 13)),
    ((1, 1, 1), (1, 1, 1)), ((7, 13, 23), (7, 13, 2)),
    ((4096, 4096), (256, 1)), ((8192, 8192), (256, 1)),
    ((16777216,), (256,)), ((100, 3), (100, 2)), ((300, 5, 5), (256, 1, 1)),
])
def test_suggest_block_size_table(global_size, expect):
    assert orc.suggest_block_size(256, global_size) == expect


def test_suggest_block_size_non_pow2_limit():
    # maxWg is rounded down to a power of two first
    assert orc.suggest_block_size(300, (1000,)) == (256,)
    assert orc.suggest_block_size(1024, (7, 13, 23)) == (7, 13, 8)


# -- kernel simulator -----------------------------------------------------------
def get_global_id(k): raise NotImplementedError
def get_local_id(k): raise NotImplementedError
def get_group_id(k): raise NotImplementedError
def get_global_size(k): raise NotImplementedError
def get_local_size(k): raise NotImplementedError


@pytest.mark.parametrize("shape", [tuple(s) for s in GOLD["kernel_shapes"]["shapes"]])
@pytest.mark.parametrize("lsize", [(), (1, 1, 1), (2, 4, 8)])
def test_kernel_sim_index_closed_forms(shape, lsize):
    def func(c):
        idx = tuple(get_global_id(k) for k in range(c.ndim))
        v = 0
        for k in range(c.ndim):
            v += (get_global_id(k) + 7 * get_local_id(k) + 31 * get_group_id(k)
                  + 1000 * get_local_size(k) + 100000 * get_global_size(k)) * 3 ** k
        c[idx] = v

    ls = tuple(lsize[:len(shape)])
    res = np.zeros(shape, np.int64)
    kernel_sim(func)[shape, ls](res)
    eff = ls if ls else (1,) * len(shape)
    expect = np.zeros(shape, np.int64)
    for idx in np.ndindex(*shape):
        v = 0
        for k, g in enumerate(idx):
            v += (g + 7 * (g % eff[k]) + 31 * (g // eff[k]) + 1000 * eff[k]
                  + 100000 * shape[k]) * 3 ** k
        expect[idx] = v
    assert np.array_equal(res, expect)
    # the stubs are restored afterwards
    with pytest.raises(NotImplementedError):
        get_global_id(0)


def test_kernel_sim_visits_every_item_once_in_group_order():
    order = []

    def func(c):
        order.append((get_global_id(0), get_global_id(1)))

    kernel_sim(func)[(5, 3), (2, 2)](None)
    assert sorted(order) == [(i, j) for i in range(5) for j in range(3)]
    # first group is ids {0,1} x {0,1} in row-major order
    assert order[:4] == [(0, 0), (0, 1), (1, 0), (1, 1)]
    assert len(order) == 15


# -- kernel simulator: barriers, local/private arrays, group ops, atomics ------
from numba_mlir_amd import kernel as _K  # stubs only; nothing here runs a GPU

_STUBS = {
    "get_global_id": _K.get_global_id, "get_local_id": _K.get_local_id,
    "get_group_id": _K.get_group_id, "get_global_size": _K.get_global_size,
    "get_local_size": _K.get_local_size, "barrier": _K.barrier,
    "mem_fence": _K.mem_fence, "atomic_add": _K.atomic.add,
    "atomic_sub": _K.atomic.sub, "local_array": _K.local.array,
    "private_array": _K.private.array,
    "group_reduce_add": _K.group.reduce_add, "group_reduce_mul": _K.group.reduce_mul,
    "group_reduce_min": _K.group.reduce_min, "group_reduce_max": _K.group.reduce_max,
}


@pytest.mark.parametrize("blocksize", [1, 10, 17, 64])
def test_kernel_sim_local_memory_and_barrier(blocksize):
    local_array, barrier, gid = _K.local.array, _K.barrier, _K.get_global_id

    def func(A):
        lm = local_array(shape=blocksize, dtype=np.float32)
        i = gid(0)
        lm[i] = A[i]
        barrier(_K.LOCAL_MEM_FENCE)
        A[i] += lm[blocksize - 1 - i]

    arr = np.arange(blocksize).astype(np.float32)
    res = arr.copy()
    kernel_sim(func, _STUBS)[blocksize, blocksize](res)
    # closed form: i + (blocksize - 1 - i)
    assert np.array_equal(res, np.full(blocksize, blocksize - 1, np.float32))


@pytest.mark.parametrize("global_size,local_size", [(1, 1), (4, 2), (27, 7), (101, 33)])
def test_kernel_sim_group_reduce_closed_form(global_size, local_size):
    gid = _K.get_global_id
    for name, fold in (("add", sum), ("max", max), ("min", min)):
        op = getattr(_K.group, "reduce_" + name)

        def func(a, b):
            i = gid(0)
            b[i] = op(a[i])

        a = np.arange(global_size, dtype=np.int64)
        b = np.zeros(global_size, np.int64)
        kernel_sim(func, _STUBS)[(global_size,), (local_size,)](a, b)
        expect = np.empty_like(b)
        for start in range(0, global_size, local_size):
            stop = min(start + local_size, global_size)
            expect[start:stop] = fold(range(start, stop))
        assert np.array_equal(b, expect)


def test_kernel_sim_atomics_and_barrier_order():
    atomic_add, atomic_sub, barrier, gid = _K.atomic.add, _K.atomic.sub, _K.barrier, _K.get_global_id

    def func(a, b):
        i = gid(0)
        off = i // 7
        atomic_add(a, off, i)
        barrier(_K.GLOBAL_MEM_FENCE)
        b[i] = a[off]

    n = 27
    a = np.zeros(4, np.int64)
    b = np.zeros(n, np.int64)
    kernel_sim(func, _STUBS)[n, 7](a, b)
    groups = [sum(range(s, min(s + 7, n))) for s in range(0, n, 7)]
    assert a.tolist() == groups
    assert b.tolist() == [groups[i // 7] for i in range(n)]   # all adds land before reads

    def func2(a, b):
        i = gid(0)
        atomic_sub(b, i % 2, a[i])

    a = np.arange(1, 10, dtype=np.int32)
    b = np.zeros(2, np.int32)
    kernel_sim(func2, _STUBS)[a.shape, ()](a, b)
    assert b.tolist() == [-(1 + 3 + 5 + 7 + 9), -(2 + 4 + 6 + 8)]


def test_kernel_sim_private_arrays_are_per_item():
    private_array, barrier, gid = _K.private.array, _K.barrier, _K.get_global_id

    def func(A):
        i = gid(0)
        p = private_array(shape=(10, 10), dtype=np.float32)
        for j in range(10):
            for k in range(10):
                p[j, k] = i
        barrier(_K.LOCAL_MEM_FENCE)
        A[i] = p[i % 10, i % 10] * 2

    res = np.zeros(17, np.float32)
    kernel_sim(func, _STUBS)[17, 17](res)
    assert np.array_equal(res, 2 * np.arange(17, dtype=np.float32))
