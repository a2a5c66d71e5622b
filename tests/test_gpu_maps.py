"""GPU parity: elementwise/broadcast maps and the fused Black-Scholes map,
through the gpux* C-ABI, against the CPU oracle."""

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
    from numba_mlir_amd.mlir import ops
    from oracle import oracle as orc
    return hip, ops, orc


def _bits(a):
    return np.ascontiguousarray(a).tobytes()


@pytest.mark.parametrize("i", range(6))
@pytest.mark.parametrize("j", range(6))
def test_broadcast_fixtures_bit_exact(env, i, j):
    """The reference's own broadcast cases (tests/test_numpy.py:483-514)."""
    hip, ops, orc = env
    arrs = [np.array(a, np.int64) for a in GOLD["broadcast_arrays"]["arrays"]]
    a, b = arrs[i], arrs[j]
    got = ops.add(hip.asarray(a), hip.asarray(b)).asnumpy()
    expect = orc.add(a, b)
    assert got.shape == expect.shape and got.dtype == expect.dtype
    assert np.array_equal(got, expect)
    assert np.array_equal(got, np.add(a, b))


@pytest.mark.parametrize("dtype", [np.float64, np.float32, np.int32, np.int64])
def test_golden_linalg_addf(env, dtype):
    hip, ops, _ = env
    g = GOLD["linalg_addf"]
    a, b = np.array(g["a"], dtype), np.array(g["b"], dtype)
    got = ops.add(hip.asarray(a), hip.asarray(b)).asnumpy()
    assert np.array_equal(got, np.array(g["out"], dtype))


@pytest.mark.parametrize("shape,expect_kernel", [
    ((4096, 4096), "nmk_map2_rowbcast_add_f64"),     # benchmark configuration
    ((1000, 4098), "nmk_map2_rowbcast_add_f64"),     # ragged rows / column tail
    ((3, 2), "nmk_map2_rowbcast_add_f64"),
    ((7, 4097), "nmk_map2_strided_add_f64"),         # odd column count
    ((5, 1), "nmk_map2_strided_add_f64"),
])
def test_row_broadcast_add_f64_bit_exact(env, shape, expect_kernel):
    hip, ops, orc = env
    rng = np.random.Generator(np.random.PCG64(1001))
    a = rng.uniform(-1, 1, shape)
    b = rng.uniform(-1, 1, (1, shape[1]))
    d_a, d_b = hip.asarray(a), hip.asarray(b)
    got = ops.add(d_a, d_b).asnumpy()
    assert hip.get_context().last_kernel() == expect_kernel
    assert _bits(got) == _bits(orc.add(a, b))
    # broadcast operand on the left (add commutes bit-exactly)
    got = ops.add(d_b, d_a).asnumpy()
    assert _bits(got) == _bits(orc.add(a, b))
    # rank-1 row operand
    got = ops.add(d_a, hip.asarray(b[0])).asnumpy()
    assert _bits(got) == _bits(a + b[0])


def test_config1_workload_matches_oracle(env):
    hip, ops, orc = env
    from numba_mlir_amd import workloads
    a, b = workloads.broadcast_add()
    assert a.shape == (4096, 4096) and b.shape == (1, 4096) and a.dtype == np.float64
    got = ops.add(hip.asarray(a), hip.asarray(b)).asnumpy()
    assert _bits(got) == _bits(orc.add(a, b))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [4, 1024, 1 << 20, (1 << 20) + 4, 1027])
def test_contiguous_maps(env, dtype, n):
    hip, ops, _ = env
    rng = np.random.default_rng(n)
    a = rng.standard_normal(n).astype(dtype)
    b = rng.standard_normal(n).astype(dtype)
    d_a, d_b = hip.asarray(a), hip.asarray(b)
    for fn, ref in ((ops.add, np.add), (ops.subtract, np.subtract),
                    (ops.divide, np.divide), (ops.multiply, np.multiply)):
        got = fn(d_a, d_b).asnumpy()
        assert _bits(got) == _bits(ref(a, b))
    kern = hip.get_context().last_kernel()
    vec = 16 // np.dtype(dtype).itemsize
    assert ("contig" in kern) == (n % vec == 0)


def test_column_broadcast_and_transposed_operands(env):
    hip, ops, _ = env
    rng = np.random.default_rng(2)
    a = rng.standard_normal((37, 53))
    col = rng.standard_normal((37, 1))
    d_a = hip.asarray(a)
    assert _bits(ops.add(d_a, hip.asarray(col)).asnumpy()) == _bits(a + col)
    assert _bits(ops.subtract(hip.asarray(col), d_a).asnumpy()) == _bits(col - a)
    at = hip.asarray(np.ascontiguousarray(a.T)).T      # strided view of a
    assert at.shape == a.shape and not at.is_c_contiguous()
    assert _bits(ops.multiply(at, d_a).asnumpy()) == _bits(a * a)


def test_division_of_floats_is_correctly_rounded(env):
    """Row-broadcast (either side), strided and special operands of the
    hand-written division; integers are left to the generated kernels."""
    hip, ops, _ = env
    rng = np.random.default_rng(3)
    for dtype in (np.float32, np.float64):
        a = rng.standard_normal((64, 1024)).astype(dtype)
        row = (rng.standard_normal((1, 1024)) + 3).astype(dtype)
        d_a, d_row = hip.asarray(a), hip.asarray(row)
        assert _bits(ops.divide(d_a, d_row).asnumpy()) == _bits(a / row)
        assert "rowbcast_div" in hip.get_context().last_kernel()
        assert _bits(ops.divide(d_row, d_a).asnumpy()) == _bits(row / a)   # does not commute
        assert "strided_div" in hip.get_context().last_kernel()
        odd = np.array([0, -0.0, 1, np.inf, -np.inf, np.nan, 1e-40, 3], dtype)
        with np.errstate(all="ignore"):
            expect = odd[:, None] / odd[None, :]
        got = ops.divide(hip.asarray(odd.reshape(8, 1)), hip.asarray(odd.reshape(1, 8))).asnumpy()
        assert _bits(got) == _bits(expect)
    with pytest.raises(NotImplementedError):
        ops.divide(hip.asarray(np.arange(4)), hip.asarray(np.arange(4)))


def test_empty_inputs(env):
    hip, ops, _ = env
    a = np.zeros((0, 8)); b = np.zeros((1, 8))
    assert ops.add(hip.asarray(a), hip.asarray(b)).asnumpy().shape == (0, 8)
    assert ops.add(hip.asarray(np.zeros(0)), hip.asarray(np.zeros(0))).asnumpy().shape == (0,)


# -- Black-Scholes -------------------------------------------------------------
# Tolerance: |gpu - oracle| <= 1e-4 * |oracle| + 1e-7 for the reference typing
# (float64 literals).  The absolute term covers float32 denormal-range outputs;
# prices are O(1..40).
BS_RTOL, BS_ATOL = 1e-4, 1e-7


def _run_bs(hip, ops, n, wide):
    from numba_mlir_amd import workloads
    price, strike, t, rate, vol, call, put = workloads.black_scholes(n)
    d = [hip.asarray(x) for x in (price, strike, t, call, put)]
    ops.black_scholes(d[0], d[1], d[2], rate, vol, d[3], d[4],
                      float64_literals=wide)
    return (price, strike, t, rate, vol), d[3].asnumpy(), d[4].asnumpy()


@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 524288, 524291])
def test_black_scholes_reference_typing(env, n):
    hip, ops, orc = env
    inp, call, put = _run_bs(hip, ops, n, True)
    assert hip.get_context().last_kernel() == "nmk_black_scholes_f32_w64"
    rc, rp = orc.black_scholes(*inp, wide=True)
    np.testing.assert_allclose(call, rc, rtol=BS_RTOL, atol=BS_ATOL)
    np.testing.assert_allclose(put, rp, rtol=BS_RTOL, atol=BS_ATOL)


def test_black_scholes_special_values(env):
    """Zero, infinite and NaN inputs take the same IEEE paths as the oracle."""
    hip, ops, orc = env
    inf, nan = np.inf, np.nan
    price = np.array([30, 0, 30, 0, inf, 30, nan, 30, 30, 1e-30, 50, 10], np.float32)
    strike = np.array([30, 30, 0, 0, 30, inf, 30, nan, 30, 30, 10, 50], np.float32)
    t = np.array([1.5, 1, 1, 1, 1, 1, 1, 1, 0, 1, 2, 1], np.float32)
    d = [hip.asarray(x) for x in (price, strike, t, np.zeros(12, np.float32),
                                  np.zeros(12, np.float32))]
    ops.black_scholes(d[0], d[1], d[2], np.float32(0.1), np.float32(0.2), d[3], d[4])
    with np.errstate(all="ignore"):
        rc, rp = orc.black_scholes(price, strike, t, 0.1, 0.2, wide=True)
    call, put = d[3].asnumpy(), d[4].asnumpy()
    assert np.array_equal(np.isnan(call), np.isnan(rc))
    assert np.array_equal(np.isnan(put), np.isnan(rp))
    ok = ~np.isnan(rc)
    np.testing.assert_allclose(call[ok], rc[ok], rtol=BS_RTOL, atol=BS_ATOL)
    ok = ~np.isnan(rp)
    np.testing.assert_allclose(put[ok], rp[ok], rtol=BS_RTOL, atol=BS_ATOL)


def test_black_scholes_out_of_range_operands(env):
    """Operands outside the everyday range (huge, tiny, denormal, negative, a
    long-dated option whose discount factor underflows) go through the general
    routines and still match the oracle."""
    hip, ops, orc = env
    price = np.array([1e38, 1e-38, 1e-42, 30, 30, -30, 30, 2.0 ** 60, 2.0 ** -61, 30, 1e20],
                     np.float32)
    strike = np.array([1e38, 1e-38, 1e-42, 1e38, 1e-38, 30, -30, 2.0 ** 59, 2.0 ** -60, 30, 1e-20],
                      np.float32)
    t = np.array([1, 1, 1, 1, 1, 1, 1, 1.5, 1.5, 1000, 1], np.float32)
    n = len(price)
    for wide in (True, False):
        d = [hip.asarray(x) for x in (price, strike, t, np.zeros(n, np.float32),
                                      np.zeros(n, np.float32))]
        ops.black_scholes(d[0], d[1], d[2], np.float32(0.1), np.float32(0.2), d[3], d[4],
                          float64_literals=wide)
        with np.errstate(all="ignore"):
            rc, rp = orc.black_scholes(price, strike, t, 0.1, 0.2, wide=wide)
        call, put = d[3].asnumpy(), d[4].asnumpy()
        assert np.array_equal(np.isnan(call), np.isnan(rc)), (wide, call, rc)
        assert np.array_equal(np.isnan(put), np.isnan(rp)), (wide, put, rp)
        ok = np.isfinite(rc)
        np.testing.assert_allclose(call[ok], rc[ok], rtol=1e-4, atol=1e-30)
        assert np.array_equal(call[~ok & ~np.isnan(rc)], rc[~ok & ~np.isnan(rc)])
        ok = np.isfinite(rp)
        np.testing.assert_allclose(put[ok], rp[ok], rtol=1e-4, atol=2e-5 if not wide else 1e-30)
        assert np.array_equal(put[~ok & ~np.isnan(rp)], rp[~ok & ~np.isnan(rp)])


def test_black_scholes_plain_and_careful_bodies_agree(env):
    """One odd lane sends its whole wave through the careful body (library
    routines, NaN care).  float32 typing: the everyday forms repeat the library
    routines' operations, so every other option of the wave comes out
    bit-identical to the run without the odd lane.  float64 typing: the plain
    body takes the hardware reciprocal, log2 and exp2 directly (within 2 units
    in the last place of the library's float32 results), so the two runs may
    differ by what a relative change of 3e-7 in exp(b) S moves a price: under
    2e-5 absolute on prices up to 40, far inside the tolerance."""
    hip, ops, orc = env
    n = 1 << 16
    (price, strike, t, rate, vol), call0, put0 = _run_bs(hip, ops, n, True)
    for wide in (True, False):
        d = [hip.asarray(x) for x in (price, strike, t, np.zeros(n, np.float32),
                                      np.zeros(n, np.float32))]
        ops.black_scholes(d[0], d[1], d[2], rate, vol, d[3], d[4], float64_literals=wide)
        base_c, base_p = d[3].asnumpy(), d[4].asnumpy()
        p2, s2, t2 = price.copy(), strike.copy(), t.copy()
        odd = np.arange(7, n, 97)          # at least one lane in every wave
        p2[odd[0::3]] = 0.0
        s2[odd[1::3]] = np.inf
        t2[odd[2::3]] = 900.0              # exp(-90) is below the everyday range
        d = [hip.asarray(x) for x in (p2, s2, t2, np.zeros(n, np.float32),
                                      np.zeros(n, np.float32))]
        ops.black_scholes(d[0], d[1], d[2], rate, vol, d[3], d[4], float64_literals=wide)
        c2, u2 = d[3].asnumpy(), d[4].asnumpy()
        keep = np.ones(n, bool)
        keep[odd] = False
        if wide:
            np.testing.assert_allclose(c2[keep], base_c[keep], rtol=1e-6, atol=2e-5)
            np.testing.assert_allclose(u2[keep], base_p[keep], rtol=1e-6, atol=2e-5)
            # and both runs meet the bar against the oracle
            rc, rp = orc.black_scholes(price, strike, t, rate, vol, wide=True)
            for got_c, got_p in ((base_c, base_p), (c2, u2)):
                np.testing.assert_allclose(got_c[keep], rc[keep], rtol=BS_RTOL, atol=BS_ATOL)
                np.testing.assert_allclose(got_p[keep], rp[keep], rtol=BS_RTOL, atol=BS_ATOL)
        else:
            assert np.array_equal(c2[keep], base_c[keep])
            assert np.array_equal(u2[keep], base_p[keep])
        with np.errstate(all="ignore"):
            rc, rp = orc.black_scholes(p2[odd], s2[odd], t2[odd], rate, vol, wide=wide)
        np.testing.assert_allclose(c2[odd], rc, rtol=1e-4, atol=2e-5)
        np.testing.assert_allclose(u2[odd], rp, rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("rate,vol", [
    (0.1, 0.2), (0.49, 0.2), (0.51, 0.2), (0.7, 0.3), (-0.3, 0.2), (-0.6, 0.2),
    (0.0, 0.2), (40.0, 0.2), (0.1, 1e-20), (0.1, 1e18), (0.1, 0.0), (0.1, -0.2),
    (np.nan, 0.2), (0.1, np.nan), (np.inf, 0.2), (0.1, np.inf), (1e30, 0.2)])
def test_black_scholes_scalar_ranges(env, rate, vol):
    """The plain body is taken only while |rate t| <= 1 and the scalars are
    ordinary; rates around that limit, zero, negative, huge, infinite and NaN
    scalars all match the oracle (same NaN pattern, same prices)."""
    hip, ops, orc = env
    from numba_mlir_amd import workloads
    n = 4096
    price, strike, t, _, _, call, put = workloads.black_scholes(n)
    rate, vol = np.float32(rate), np.float32(vol)
    d = [hip.asarray(x) for x in (price, strike, t, call, put)]
    ops.black_scholes(d[0], d[1], d[2], rate, vol, d[3], d[4])
    with np.errstate(all="ignore"):
        rc, rp = orc.black_scholes(price, strike, t, rate, vol, wide=True)
    got_c, got_p = d[3].asnumpy(), d[4].asnumpy()
    for got, ref in ((got_c, rc), (got_p, rp)):
        assert np.array_equal(np.isnan(got), np.isnan(ref)), (rate, vol)
        fin = np.isfinite(ref)
        np.testing.assert_allclose(got[fin], ref[fin], rtol=BS_RTOL,
                                   atol=BS_ATOL + 4e-6 * float(np.abs(ref[fin]).max(initial=0)))
        rest = ~fin & ~np.isnan(ref)
        assert np.array_equal(got[rest], ref[rest])


def test_black_scholes_float32_typing(env):
    hip, ops, orc = env
    inp, call, put = _run_bs(hip, ops, 524288, False)
    assert hip.get_context().last_kernel() == "nmk_black_scholes_f32_w32"
    rc, rp = orc.black_scholes(*inp, wide=False)
    # float32 throughout: the tails cancel catastrophically on both sides, so
    # only an absolute bound is meaningful (prices up to ~40, eps 6e-8).
    np.testing.assert_allclose(call, rc, rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(put, rp, rtol=1e-4, atol=2e-5)
    # and the reference's own bar against the other typing
    wc, wp = orc.black_scholes(*inp, wide=True)
    np.testing.assert_allclose(call, wc, atol=GOLD["black_scholes"]["atol"])
    np.testing.assert_allclose(put, wp, atol=GOLD["black_scholes"]["atol"])


@pytest.mark.parametrize("wide", [True, False])
def test_black_scholes_block_counts_set_by_hand(env, wide):
    """Which block takes which options (two trips 128 pieces apart by default,
    whole grids apart for a block count set by hand, a power of two or not)
    does not change a price: on everyday operands every wave runs the same
    arithmetic."""
    from numba_mlir_amd.mlir import lowered
    hip, ops, _ = env
    n = 700003
    _, call, put = _run_bs(hip, ops, n, wide)
    try:
        for blocks in (1, 3, 100, 128, 1000, 4096):
            lowered.set_tuning("bs_blocks", blocks)
            _, c2, p2 = _run_bs(hip, ops, n, wide)
            assert c2.tobytes() == call.tobytes() and p2.tobytes() == put.tobytes(), blocks
    finally:
        lowered.set_tuning("bs_blocks", 0)


def test_black_scholes_full_size(env):
    """2^24 options: oracle parity plus put-call parity and the closed form."""
    hip, ops, orc = env
    inp, call, put = _run_bs(hip, ops, 2 ** 24, True)
    rc, rp = orc.black_scholes(*inp, wide=True)
    np.testing.assert_allclose(call, rc, rtol=BS_RTOL, atol=BS_ATOL)
    np.testing.assert_allclose(put, rp, rtol=BS_RTOL, atol=BS_ATOL)
    price, strike, t, rate, vol = inp
    disc = strike.astype(np.float64) * np.exp(-float(rate) * t.astype(np.float64))
    np.testing.assert_allclose(call.astype(np.float64) - put, price - disc,
                               rtol=0, atol=2e-5)
    tc, tp = orc.black_scholes_truth(*inp)
    np.testing.assert_allclose(call, tc, rtol=5e-5, atol=1e-12)
    np.testing.assert_allclose(put, tp, rtol=5e-5, atol=1e-12)
    assert (call >= 0).all() and (put >= -1e-6).all()   # r - P + Se cancels


def test_more_than_two_to_the_31_elements(env):
    """Element counts and byte offsets past 2^31 (8 GiB of int32 an array): the
    map and the reductions index in 64 bits.  Checked on the device: the ends
    of the result, and its sums."""
    hip, ops, _ = env
    n = 2 ** 31 + 8
    host = np.ones(n, np.int32)
    host[-8:] = 7
    a = hip.asarray(host)
    del host
    out = ops.add(a, a)
    assert out.shape == (n,)
    assert out[:8].asnumpy().tolist() == [2] * 8
    assert out[n - 16:].asnumpy().tolist() == [2] * 8 + [14] * 8
    # (a full reduction accumulates in int64 and is cast back to the array's
    # type, numpy/funcs.py:183-185: the total modulo 2^32)
    total = ops.sum(out)
    assert total.dtype == np.int32
    assert int(total) == int(np.int64(2 * (n - 8) + 14 * 8).astype(np.int32)) == 112
    assert int(ops.amax(out)) == 14 and int(ops.amin(out)) == 2
    wide = out.reshape((n // 8, 8))
    assert ops.sum(wide, axis=0).asnumpy().tolist() == [2 * (n // 8 - 1) + 14] * 8
    # (268 million rows of eight: more blocks than one dimension of a launch holds)
    rows = ops.sum(wide, axis=1)
    assert rows.shape == (n // 8,) and int(ops.amax(rows)) == 112 and int(ops.amin(rows)) == 16
    assert rows[n // 8 - 2:].asnumpy().tolist() == [16, 112]
    del rows, wide, out, a
    tall = hip.asarray(np.ones((2 ** 27 + 3, 8), np.float32))
    sums = ops.sum(tall, axis=1)
    assert float(ops.amin(sums)) == 8.0 and float(ops.amax(sums)) == 8.0
    norms = ops.l2_norm_rows(tall)
    assert abs(float(ops.amin(norms)) - 8 ** 0.5) < 1e-6 and abs(float(ops.amax(norms)) - 8 ** 0.5) < 1e-6


def test_tall_strided_operands(env):
    """Views of ten million rows (two of three columns): more blocks of rows
    than a launch has along y."""
    hip, ops, _ = env
    rng = np.random.default_rng(23)
    a = rng.standard_normal((10_000_000, 3)).astype(np.float32)
    b = rng.standard_normal((10_000_000, 3)).astype(np.float32)
    got = ops.add(hip.asarray(a)[:, :2], hip.asarray(b)[:, :2]).asnumpy()
    assert np.array_equal(got, a[:, :2] + b[:, :2])
