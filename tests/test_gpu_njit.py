"""GPU parity: ``njit`` over device arrays -- library lowering, one parallel
loop, elementwise fusion -- against NumPy / the oracle."""

import numpy as np
import pytest

import njit_cases as cases
from numba_mlir_amd.decorators import njit

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env(hip):
    from numba_mlir_amd import workloads
    from numba_mlir_amd.mlir import ops
    from oracle import oracle as orc
    return hip, ops, orc, workloads


def _bs_inputs(hip, workloads, n):
    price, strike, t, rate, vol, call, put = workloads.black_scholes(n)
    dev = [hip.asarray(x) for x in (price, strike, t)]
    return (price, strike, t, rate, vol), dev, hip.asarray(call), hip.asarray(put)


@pytest.mark.parametrize("n", [1, 1000, 524288])
def test_black_scholes_whole_array_body(env, n):
    """The reference's fused-loop test (test_numpy.py:2796-2866): the body over
    whole arrays becomes one kernel; results against the oracle at the path's
    tolerance and against the reference's own bar."""
    hip, ops, orc, workloads = env
    inp, dev, call, put = _bs_inputs(hip, workloads, n)
    f = njit(cases.black_scholes_arrays)
    f(dev[0], dev[1], dev[2], inp[3], inp[4], call, put)
    assert f.last_launch["path"] == "elementwise"
    rc, rp = orc.black_scholes(*inp, wide=True)
    np.testing.assert_allclose(call.asnumpy(), rc, rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(put.asnumpy(), rp, rtol=1e-4, atol=1e-7)
    # and against the hand-written kernel of the same formula
    c2, p2 = hip.asarray(np.zeros(n, np.float32)), hip.asarray(np.zeros(n, np.float32))
    ops.black_scholes(dev[0], dev[1], dev[2], inp[3], inp[4], c2, p2)
    np.testing.assert_allclose(call.asnumpy(), c2.asnumpy(), rtol=2e-6, atol=1e-6)
    np.testing.assert_allclose(put.asnumpy(), p2.asnumpy(), rtol=2e-6, atol=2e-6)


def test_black_scholes_body_unaligned_views_and_ragged_ends(env):
    """The fused map gives a lane four adjacent options in 128-bit words when
    every array starts on a 16-byte boundary; a view that starts one element
    further on, and the last n % 4 options, are computed one option a lane.
    Both orders of evaluation give every option the same price."""
    hip, ops, orc, workloads = env
    n = 4099
    price, strike, t, rate, vol, _, _ = workloads.black_scholes(n + 1)
    f = njit(cases.black_scholes_arrays)
    got = []
    for first in (0, 1):
        dev = [hip.asarray(x)[first:first + n] for x in (price, strike, t)]
        call = hip.asarray(np.zeros(n + 1, np.float32))[first:first + n]
        put = hip.asarray(np.zeros(n + 1, np.float32))[first:first + n]
        f(dev[0], dev[1], dev[2], rate, vol, call, put)
        assert f.last_launch["path"] == "elementwise"
        rc, rp = orc.black_scholes(price[first:first + n], strike[first:first + n],
                                   t[first:first + n], rate, vol, wide=True)
        np.testing.assert_allclose(call.asnumpy(), rc, rtol=1e-4, atol=1e-7)
        np.testing.assert_allclose(put.asnumpy(), rp, rtol=1e-4, atol=1e-7)
        got.append((call.asnumpy(), put.asnumpy()))
    # options 1 .. n-1 of the first run are options 0 .. n-2 of the second
    np.testing.assert_allclose(got[0][0][1:], got[1][0][:-1], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(got[0][1][1:], got[1][1][:-1], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("form", ["arrays", "loop"])
def test_black_scholes_body_odd_operands(env, form):
    """Zeros, infinities, NaNs, negative, huge, tiny and denormal operands and
    a discount factor that underflows: the wave computes its options again
    with the general routines and matches the oracle; the everyday options
    that share a wave with an odd one keep their prices.  Both forms of the
    body: whole arrays, and one prange loop that stores call[i], put[i]."""
    hip, ops, orc, workloads = env
    if form == "arrays":
        compiled = njit(cases.black_scholes_arrays)
    else:
        loop = njit(parallel=True)(cases.black_scholes_loop)
        compiled = lambda p, s, t, rate, vol, call, put: loop(len(p), p, s, t, rate, vol, call, put)
    inf, nan = np.inf, np.nan
    price = np.array([30, 0, 30, 0, inf, 30, nan, 30, 30, 1e-30, 50, 10, 1e38, 1e-38, 1e-42,
                      30, 30, -30, 30, 2.0 ** 60, 2.0 ** -61, 30, 1e20], np.float32)
    strike = np.array([30, 30, 0, 0, 30, inf, 30, nan, 30, 30, 10, 50, 1e38, 1e-38, 1e-42,
                       1e38, 1e-38, 30, -30, 2.0 ** 59, 2.0 ** -60, 30, 1e-20], np.float32)
    t = np.array([1.5, 1, 1, 1, 1, 1, 1, 1, 0, 1, 2, 1, 1, 1, 1, 1, 1, 1, 1, 1.5, 1.5, 1000, 1],
                 np.float32)
    f = compiled
    n = len(price)
    d = [hip.asarray(x) for x in (price, strike, t, np.zeros(n, np.float32),
                                  np.zeros(n, np.float32))]
    f(d[0], d[1], d[2], np.float32(0.1), np.float32(0.2), d[3], d[4])
    with np.errstate(all="ignore"):
        rc, rp = orc.black_scholes(price, strike, t, 0.1, 0.2, wide=True)
    call, put = d[3].asnumpy(), d[4].asnumpy()
    for got, ref in ((call, rc), (put, rp)):
        assert np.array_equal(np.isnan(got), np.isnan(ref)), (got, ref)
        ok = np.isfinite(ref)
        np.testing.assert_allclose(got[ok], ref[ok], rtol=1e-4, atol=1e-7)
        assert np.array_equal(got[~ok & ~np.isnan(ref)], ref[~ok & ~np.isnan(ref)])
    # one odd option in every wave
    n = 1 << 16
    price, strike, t, rate, vol, _, _ = workloads.black_scholes(n)
    runs = []
    p2, s2, t2 = price.copy(), strike.copy(), t.copy()
    odd = np.arange(7, n, 97)
    p2[odd[0::3]] = 0.0
    s2[odd[1::3]] = np.inf
    t2[odd[2::3]] = 900.0
    for p, s, tt in ((price, strike, t), (p2, s2, t2)):
        d = [hip.asarray(x) for x in (p, s, tt, np.zeros(n, np.float32),
                                      np.zeros(n, np.float32))]
        f(d[0], d[1], d[2], rate, vol, d[3], d[4])
        runs.append((d[3].asnumpy(), d[4].asnumpy()))
    keep = np.ones(n, bool)
    keep[odd] = False
    # (the two forms repeat the same operations but for the quotient, which
    # the plain form rounds differently in about one case in 10^7)
    np.testing.assert_allclose(runs[1][0][keep], runs[0][0][keep], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(runs[1][1][keep], runs[0][1][keep], rtol=1e-6, atol=1e-6)
    assert np.mean(runs[1][0][keep] == runs[0][0][keep]) > 0.999
    with np.errstate(all="ignore"):
        rc, rp = orc.black_scholes(p2[odd], s2[odd], t2[odd], rate, vol, wide=True)
    np.testing.assert_allclose(runs[1][0][odd], rc, rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(runs[1][1][odd], rp, rtol=1e-4, atol=2e-5)


def test_black_scholes_prange_body(env):
    hip, ops, orc, workloads = env
    n = 100003
    inp, dev, call, put = _bs_inputs(hip, workloads, n)
    f = njit(parallel=True)(cases.black_scholes_loop)
    f(n, dev[0], dev[1], dev[2], inp[3], inp[4], call, put)
    assert f.last_launch["path"] == "parallel loop"
    rc, rp = orc.black_scholes(*inp, wide=True)
    np.testing.assert_allclose(call.asnumpy(), rc, rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(put.asnumpy(), rp, rtol=1e-4, atol=1e-7)


def test_numpy_arguments_round_trip(env):
    """Host arrays are copied in and out, as calling the jitted function on
    NumPy arrays behaves in the reference."""
    hip, ops, orc, workloads = env
    price, strike, t, rate, vol, call, put = workloads.black_scholes(4096)
    njit(cases.black_scholes_arrays)(price, strike, t, rate, vol, call, put)
    rc, rp = orc.black_scholes(price, strike, t, rate, vol, wide=True)
    np.testing.assert_allclose(call, rc, rtol=1e-4, atol=1e-7)
    np.testing.assert_allclose(put, rp, rtol=1e-4, atol=1e-7)
    out = njit(cases.add)(np.arange(6.0).reshape(2, 3), np.ones((1, 3)))
    np.testing.assert_array_equal(out, np.arange(6.0).reshape(2, 3) + 1)


def test_broadcast_add_goes_to_the_hand_written_kernel(env):
    hip, ops, orc, workloads = env
    a, b = workloads.broadcast_add(512, 1024)
    f = njit(parallel=True)(cases.add)
    out = f(hip.asarray(a), hip.asarray(b))
    assert f.last_launch == {"path": "library", "kernel": "nmk_map2_rowbcast_add_f64"}
    assert np.array_equal(out.asnumpy(), a + b)
    # operands the map kernels do not cover are fused instead
    x = np.arange(24, dtype=np.int16).reshape(2, 3, 4)
    out = f(hip.asarray(x), hip.asarray(x[:1]))
    assert f.last_launch["path"] == "elementwise"
    assert np.array_equal(out.asnumpy(), x + x[:1])
    out = f(hip.asarray(np.arange(5, dtype=np.int32)), hip.asarray(np.arange(5.0)))
    assert out.dtype == np.float64 and np.array_equal(out.asnumpy(), 2.0 * np.arange(5))


@pytest.mark.parametrize("shapes", [((40, 50), (40, 50), (40, 50)),
                                    ((40, 1), (1, 50), (40, 50)),
                                    ((50,), (40, 50), (1, 1)),
                                    ((3, 4, 5), (4, 1), (5,))])
def test_elementwise_fusion_with_broadcasting(env, shapes):
    hip, ops, orc, workloads = env
    rng = np.random.default_rng(11)
    a, b, c = (rng.uniform(-2, 2, s) for s in shapes)
    f = njit(cases.fused_map)
    out = f(hip.asarray(a), hip.asarray(b), hip.asarray(c), 1.5)
    assert f.last_launch["path"] == "elementwise"
    np.testing.assert_allclose(out.asnumpy(), cases.fused_map(a, b, c, 1.5), rtol=1e-13)
    assert out.shape == np.broadcast_shapes(*shapes)


def test_elementwise_fusion_over_strided_views(env):
    hip, ops, orc, workloads = env
    rng = np.random.default_rng(12)
    base = rng.uniform(-2, 2, (3, 64, 96))
    dev = hip.asarray(base)
    views = [dev[k, ::2, 1::3] for k in range(3)]
    host = [base[k, ::2, 1::3] for k in range(3)]
    f = njit(cases.fused_map)
    out = f(*views, 0.5)
    np.testing.assert_allclose(out.asnumpy(), cases.fused_map(*host, 0.5), rtol=1e-13)
    out = f(views[0].T, views[1].T, views[2].T, 0.5)
    np.testing.assert_allclose(out.asnumpy(), cases.fused_map(*[h.T for h in host], 0.5),
                               rtol=1e-13)


def test_stores_into_several_outputs(env):
    hip, ops, orc, workloads = env
    x = np.arange(-50, 50, dtype=np.int32)
    y = np.arange(100, 0, -1, dtype=np.int32)
    out_f, out_i = hip.asarray(np.zeros(100)), hip.asarray(np.zeros(100, np.int64))
    njit(cases.fused_store)(hip.asarray(x), hip.asarray(y), out_f, out_i)
    ref_f, ref_i = np.zeros(100), np.zeros(100, np.int64)
    cases.fused_store(x.astype(np.int64), y.astype(np.int64), ref_f, ref_i)
    np.testing.assert_allclose(out_f.asnumpy(), ref_f, rtol=1e-15)
    np.testing.assert_array_equal(out_i.asnumpy(), ref_i)
    with pytest.raises(ValueError, match="broadcast shape"):
        njit(cases.fused_store)(hip.asarray(x), hip.asarray(y), out_f,
                                hip.asarray(np.zeros(1, np.int64)))


def test_prange_loops(env):
    hip, ops, orc, workloads = env
    rng = np.random.default_rng(13)
    x, y = rng.standard_normal(10007).astype(np.float32), rng.standard_normal(10007).astype(np.float32)
    out = hip.asarray(np.zeros(10007, np.float32))
    njit(parallel=True)(cases.saxpy_loop)(np.float32(2.5), hip.asarray(x), hip.asarray(y), out)
    np.testing.assert_array_equal(out.asnumpy(), np.float32(2.5) * x + y)
    m = rng.standard_normal((101, 7))
    out = hip.asarray(np.zeros(101))
    njit(parallel=True)(cases.strided_loop)(hip.asarray(m), out)
    ref = np.zeros(101)
    cases.strided_loop(m, ref)
    np.testing.assert_allclose(out.asnumpy(), ref, rtol=1e-13)


SCALARS = [True, False, -3, -2, -1, 0, 1, 2, 3, -2.5, -1.0, -0.5, -0.0, 0.0, 0.5, 1.0, 2.5]


def test_reference_parfor_and_array_statement_tests(env):
    """test_gpu.py:1518-1700: prange loops over device and shared arrays, a
    scalar argument or captured value of every kind, b[:] = a * 2, c[:] = a + b,
    nested prange with the shape unpacked before the loop."""
    hip, ops, orc, workloads = env
    a = np.arange(1024, dtype=np.float32)
    b = np.arange(1024, dtype=np.float32) * 3
    da, db = hip.asarray(a), hip.asarray(b, usm_type="shared")
    out = hip.asarray(np.zeros(1024, np.float32))
    njit(cases.parfor_add)(da, db, out)
    np.testing.assert_array_equal(out.asnumpy(), a + b)
    for val in SCALARS:
        ref = np.zeros(1024, np.float32)
        cases.parfor_scalar(a, b, ref, val)
        njit(cases.parfor_scalar)(da, db, out, val)
        np.testing.assert_array_equal(out.asnumpy(), ref)

        def captured(a, b, c):
            for i in cases.prange(len(a)):
                c[i] = a[i] + b[i] + val

        njit(captured)(da, db, out)
        np.testing.assert_array_equal(out.asnumpy(), ref)
    njit(cases.scale_into)(da, out)
    np.testing.assert_array_equal(out.asnumpy(), a * 2)
    njit(cases.add_into)(da, db, out)
    np.testing.assert_array_equal(out.asnumpy(), a + b)
    njit(cases.fill)(out)
    np.testing.assert_array_equal(out.asnumpy(), np.full(1024, 42, np.float32))
    grid = hip.asarray(np.zeros((2, 3), np.float32))
    for options in ({}, {"gpu_use_64bit_index": True}, {"fastmath": True}):
        f = njit(cases.nested_prange, **options)
        f(grid)
        np.testing.assert_array_equal(grid.asnumpy(), [[0, 1, 2], [3, 4, 5]])
    # the perfect nest is a 2-d grid with the inner loop on x ...
    big = hip.asarray(np.zeros((300, 1000), np.float32))
    f(big)
    # (flat blocks, four rows of the outer loop per lane)
    assert f.last_launch["grid"][1] == 75 and f.last_launch["block"][1] == 1
    np.testing.assert_array_equal(big.asnumpy(),
                                  np.arange(300000, dtype=np.float32).reshape(300, 1000))
    # ... unless the outer loop is too long for grid y: then it alone is the grid
    tall = hip.asarray(np.zeros((70000, 4), np.float32))
    f(tall)
    assert f.last_launch["grid"][1] == 1
    np.testing.assert_array_equal(tall.asnumpy(),
                                  np.arange(280000, dtype=np.float32).reshape(70000, 4))


def test_prange_reductions(env):
    """Scalars a prange loop only updates with += / *= are reductions: lanes,
    blocks, then the host fold their shares; the return runs on the host."""
    hip, ops, orc, workloads = env
    rng = np.random.default_rng(14)
    x = rng.standard_normal(1000003).astype(np.float32)
    got = njit(parallel=True)(cases.sum_of_squares)(hip.asarray(x))
    # x[i] * x[i] is a float32 product; the accumulator is float64
    np.testing.assert_allclose(got, np.sqrt((x * x).astype(np.float64).sum()), rtol=1e-12)
    mean, above = njit(parallel=True)(cases.mean_and_count)(hip.asarray(x), 0.5)
    np.testing.assert_allclose(mean, x.astype(np.float64).mean(), rtol=1e-9, atol=1e-12)
    assert above == int((x > 0.5).sum())
    a = rng.integers(-1000, 1000, 70001).astype(np.int32)
    b = rng.integers(-1000, 1000, 70001).astype(np.int32)
    f = njit(parallel=True)(cases.int_dot)
    assert f(hip.asarray(a), hip.asarray(b)) == 10 + int((a.astype(np.int64) * b).sum())
    assert f(hip.asarray(a[:0]), hip.asarray(b[:0])) == 10       # empty loop: start value
    # repeated launches fold in the same order: same bits
    g = njit(parallel=True)(cases.sum_of_squares)
    dx = hip.asarray(x)
    assert len({g(dx) for _ in range(5)}) == 1
    p = rng.uniform(0.9, 1.1, 5000)
    np.testing.assert_allclose(njit(parallel=True)(cases.product)(hip.asarray(p)),
                               2.0 * np.prod(p), rtol=1e-12)


def test_reductions_and_contractions_go_to_the_library(env):
    hip, ops, orc, workloads = env
    x = workloads.reduce_f32(256, 4096)
    xi = workloads.reduce_i32(256, 512)
    f = njit(cases.row_sums)
    got = f(hip.asarray(x))
    assert f.last_launch == {"path": "library", "kernel": "nmk_sum_axis1_wide_w4_f32"}
    np.testing.assert_allclose(got.asnumpy(), x.astype(np.float64).sum(axis=1), rtol=1e-4,
                               atol=1e-3)
    f = njit(cases.col_sums)
    got = f(hip.asarray(xi))
    assert f.last_launch["kernel"] == "nmk_sum_axis0_i32_i64"
    assert np.array_equal(got.asnumpy(), xi.sum(axis=0, dtype=np.int64))
    f = njit(cases.norm)
    got = f(hip.asarray(x))
    assert f.last_launch["kernel"] == "nmk_norm2_f32"
    assert isinstance(got, np.float32)
    np.testing.assert_allclose(got, np.sqrt((x.astype(np.float64) ** 2).sum()), rtol=1e-5)
    # the reference's reduce tests (test_gpu.py:2045-2098): sizes, shapes, forms
    for size in (7, 16, 64, 65, 256, 512, 1024 * 1024):
        v = np.arange(size, dtype=np.float32)
        np.testing.assert_allclose(njit(lambda a: a.sum())(hip.asarray(v)), v.sum(), rtol=1e-5)
    forms = [                                  # one lambda per source line
        lambda a: a.sum(),
        lambda a: a.sum(axis=0),
        lambda a: a.sum(axis=1),
        lambda a: np.prod(a),
        lambda a: np.prod(a, axis=0),
        lambda a: np.prod(a, axis=1),
        lambda a: np.amin(a),
        lambda a: np.amax(a),
    ]
    for k, form in enumerate(forms):
        for shape in ((7, 16), (25, 64), (65, 7)):
            for dtype in (np.int32, np.int64, np.float32):
                count = shape[0] * shape[1]
                if count > 30 and 3 <= k <= 5:
                    continue                   # products overflow (skipped there too)
                v = np.arange(1, count + 1, dtype=dtype).reshape(shape).copy()
                f = njit(form)
                got = f(hip.asarray(v))
                assert f.last_launch["path"] == "library"
                got = got.asnumpy() if hasattr(got, "asnumpy") else got
                np.testing.assert_allclose(got, form(v), rtol=1e-5)
    a, b = workloads.matmul(256)
    for fn in (cases.matmul, cases.dot):
        got = njit(fn)(hip.asarray(a), hip.asarray(b))
        np.testing.assert_allclose(got.asnumpy(), orc.gemm_f32_truth(a, b), rtol=1e-4,
                                   atol=1e-3)


def test_compiled_functions_call_each_other(env):
    """An njit function called from a prange loop or a kernel is inlined as a
    device function of its scalar arguments."""
    hip, ops, orc, workloads = env
    from numba_mlir_amd import kernel as K
    smooth = njit(cases._smoothstep)
    x = np.linspace(-0.5, 1.5, 1001)

    def loop(x, out):
        for i in cases.prange(len(x)):
            out[i] = smooth(x[i], 0.25, 0.75)

    def body(x, out):
        i = K.get_global_id(0)
        out[i] = smooth(x[i], 0.25, 0.75) * 2.0

    ref = np.array([cases._smoothstep(v, 0.25, 0.75) for v in x])
    out = hip.asarray(np.zeros_like(x))
    njit(parallel=True)(loop)(hip.asarray(x), out)
    np.testing.assert_allclose(out.asnumpy(), ref, rtol=1e-15)
    K.kernel(body)[len(x), K.DEFAULT_LOCAL_SIZE](hip.asarray(x), out)
    np.testing.assert_allclose(out.asnumpy(), 2.0 * ref, rtol=1e-15)
    # whole-array form: the same function maps over arrays
    f = njit(lambda x: smooth(x, 0.25, 0.75))
    np.testing.assert_allclose(f(hip.asarray(x)).asnumpy(), ref, rtol=1e-15)


def test_unsupported_functions_are_reported(env):
    hip, ops, orc, workloads = env
    from numba_mlir_amd.kernel import KernelCompileError
    x = hip.asarray(np.arange(8.0))
    with pytest.raises(KernelCompileError, match="after the parallel loop"):
        njit(parallel=True)(cases.statements_after_loop)(x, hip.asarray(np.zeros(8)))
    with pytest.raises(ValueError, match="at least one device array"):
        njit(cases.add)(1.0, 2.0)


@pytest.mark.parametrize("n", [1, 255, 1024, 4097, 100003])
def test_prange_loops_with_reads_loaded_ahead(env, n):
    """Loops whose unconditional reads are loaded ahead of the body, beside
    conditional reads and a loop that skips iterations (which load nothing
    ahead): results as the Python loops give them, at sizes with whole and
    ragged rounds."""
    hip, ops, orc, workloads = env
    rng = np.random.default_rng(n)
    a, b, c, out0 = (rng.standard_normal(n) for _ in range(4))
    want = out0.copy()
    x = a + want
    y = np.where(x > 0, b, 0.0)
    y = np.where(y > 1.0, c, y)
    want = x + y
    d_out = hip.asarray(out0.copy())
    njit(parallel=True)(cases.loop_reads)(n, hip.asarray(a), hip.asarray(b), hip.asarray(c), d_out)
    np.testing.assert_array_equal(d_out.asnumpy(), want)
    d_out = hip.asarray(out0.copy())
    njit(parallel=True)(cases.loop_leaves_early)(n, hip.asarray(a), d_out)
    want = out0.copy()
    want[::2] = a[::2]
    np.testing.assert_array_equal(d_out.asnumpy(), want)


def test_enqueued_launches_are_covered_by_synchronize(env):
    """Launches put on the queue without waiting (the benchmark's timing path)
    are finished when the context's synchronize() returns; their events stay
    with the caller until retired."""
    hip, ops, orc, workloads = env
    from numba_mlir_amd.mlir import device_array as da
    ctx = da.get_context()
    a = np.arange(1 << 20, dtype=np.float64)
    d_a = hip.asarray(a)
    outs = [hip.asarray(np.zeros_like(a)) for _ in range(6)]
    f = njit(cases.scale_into)
    f(d_a, outs[0])
    plan = f.last_plan
    events = [plan.enqueue([d_a, o]) for o in outs]
    assert ctx.pending[-len(events):] == events
    ctx.synchronize()
    for o in outs:
        np.testing.assert_array_equal(o.asnumpy(), a * 2)
    for e in events:
        plan.retire(e)
    assert not any(e in ctx.pending for e in events)
    # arguments that do not fit the prepared launch are refused, not launched
    with pytest.raises(ValueError, match="differ in type, shape or strides"):
        plan.enqueue([d_a, hip.asarray(np.zeros(a.size, np.float32))])
    with pytest.raises(ValueError, match="differ in type, shape or strides"):
        plan.enqueue([hip.asarray(a[:100]), outs[0]])
    # a launch translated for arrays that do not overlap refuses ones that do
    assert plan.compiled.noalias
    with pytest.raises(ValueError, match="do not\\s+overlap"):
        plan.enqueue([d_a, d_a])
    g = njit(lambda a, b: a * 2 + b)          # a generated kernel that returns an array
    small = hip.asarray(np.arange(64, dtype=np.int32))
    g(small, small)
    with pytest.raises(ValueError, match="result array must have dtype"):
        g.last_plan.enqueue([small, small], hip.asarray(np.zeros(64, np.int16)))
    with pytest.raises(ValueError, match="result array must have dtype"):
        g.last_plan.enqueue([small, small])


def test_repeated_calls_replay_stored_launches(env):
    """A call whose argument types, shapes and strides were seen before reuses
    the prepared launch: new addresses, new scalar values and a change of
    aliasing must all still be honoured."""
    hip, ops, orc, workloads = env
    rng = np.random.default_rng(11)
    f = njit(cases.fused_map)
    for scale in (0.5, -3.0, 7.25):
        a, b, c = (rng.standard_normal(1000) for _ in range(3))
        got = f(hip.asarray(a), hip.asarray(b), hip.asarray(c), scale)
        np.testing.assert_allclose(got.asnumpy(), cases.fused_map(a, b, c, scale), rtol=1e-12)
    assert len(f._plans) == 1
    # a different length is a different launch
    a, b, c = (rng.standard_normal(77) for _ in range(3))
    got = f(hip.asarray(a), hip.asarray(b), hip.asarray(c), 2.0)
    np.testing.assert_allclose(got.asnumpy(), cases.fused_map(a, b, c, 2.0), rtol=1e-12)
    assert len(f._plans) == 2

    g = njit(parallel=True)(cases.saxpy_loop)
    for alpha in (2.0, -1.5, 0.0):
        x, y = rng.standard_normal(5000), rng.standard_normal(5000)
        out = hip.asarray(np.zeros(5000))
        g(alpha, hip.asarray(x), hip.asarray(y), out)
        np.testing.assert_array_equal(out.asnumpy(), alpha * x + y)
    # the output aliasing an input: same shapes, another kernel variant
    x, y = rng.standard_normal(5000), rng.standard_normal(5000)
    dx = hip.asarray(x)
    g(3.0, dx, hip.asarray(y), dx)
    np.testing.assert_array_equal(dx.asnumpy(), 3.0 * x + y)
    x2 = rng.standard_normal(5000)
    out = hip.asarray(np.zeros(5000))
    g(3.0, hip.asarray(x2), hip.asarray(y), out)
    np.testing.assert_array_equal(out.asnumpy(), 3.0 * x2 + y)

    h = njit(parallel=True)(cases.sum_of_squares)
    for n in (4096, 4096, 100, 4096):
        v = rng.standard_normal(n).astype(np.float32)
        np.testing.assert_allclose(h(hip.asarray(v)), np.sqrt(np.sum(v.astype(np.float64) ** 2)),
                                   rtol=1e-6)

    k = njit(cases.add_into)
    for _ in range(3):
        a, b = rng.standard_normal(300), rng.standard_normal(300)
        dc = hip.asarray(np.zeros(300))
        k(hip.asarray(a), hip.asarray(b), dc)
        np.testing.assert_array_equal(dc.asnumpy(), a + b)
    da_ = hip.asarray(a)
    k(da_, hip.asarray(b), da_)             # in place
    np.testing.assert_array_equal(da_.asnumpy(), a + b)


def _operands(kind, rng, n=257):
    if kind == "f":
        return rng.uniform(-3, 3, n), rng.uniform(-3, 3, n)
    if kind == "p":                       # positive floats
        return rng.uniform(0.1, 9, n), rng.uniform(0.1, 9, n)
    if kind == "i":
        b = rng.integers(-9, 10, n)
        return rng.integers(-50, 50, n), np.where(b == 0, 3, b)
    if kind == "s":                       # shift counts
        return rng.integers(-1000, 1000, n), rng.integers(0, 20, n)
    return rng.integers(0, 2, n).astype(bool), rng.integers(0, 2, n).astype(bool)


@pytest.mark.parametrize("name,func,kinds", cases.NAMED_UFUNCS,
                         ids=[c[0] for c in cases.NAMED_UFUNCS])
def test_named_binary_ufuncs(env, name, func, kinds):
    """test_numpy.py:148-199 compares each registered binary function with
    NumPy over float, integer and boolean operands."""
    hip = env[0]
    rng = np.random.default_rng(5)
    f = njit(func)
    for kind in kinds:
        a, b = _operands(kind, rng)
        got = f(hip.asarray(a), hip.asarray(b)).asnumpy()
        want = func(a, b)
        assert got.dtype == want.dtype, (name, kind)
        if want.dtype.kind == "f":
            np.testing.assert_allclose(got, want, rtol=1e-13, err_msg=f"{name} {kind}")
        else:
            np.testing.assert_array_equal(got, want, err_msg=f"{name} {kind}")
        # an array against a scalar broadcasts
        got = f(hip.asarray(a), b[3]).asnumpy()
        want = func(a, b[3])
        if want.dtype.kind == "f":
            np.testing.assert_allclose(got, want, rtol=1e-13, err_msg=f"{name} {kind}")
        else:
            np.testing.assert_array_equal(got, want, err_msg=f"{name} {kind}")


@pytest.mark.parametrize("name,func,kinds", cases.NAMED_UNARY,
                         ids=[c[0] for c in cases.NAMED_UNARY])
def test_named_unary_ufuncs(env, name, func, kinds):
    """test_numpy.py:107-145 (unary functions against NumPy)."""
    hip = env[0]
    rng = np.random.default_rng(6)
    f = njit(func)
    for kind in kinds:
        a, _ = _operands(kind, rng)
        got = f(hip.asarray(a)).asnumpy()
        want = func(a)
        assert got.dtype == want.dtype, (name, kind)
        if want.dtype.kind == "f":
            np.testing.assert_allclose(got, want, rtol=1e-13, err_msg=f"{name} {kind}")
        else:
            np.testing.assert_array_equal(got, want, err_msg=f"{name} {kind}")


def test_clip(env):
    """numpy.clip (numpy/funcs.py:571-578; test_numpy.py's clip cases): scalar
    and array bounds, NaN kept."""
    hip = env[0]
    rng = np.random.default_rng(7)
    a = rng.uniform(-2, 2, 1000)
    a[::97] = np.nan
    got = njit(cases.clip_scalars)(hip.asarray(a)).asnumpy()
    np.testing.assert_array_equal(got, np.clip(a, -0.5, 0.75))
    lo, hi = rng.uniform(-1, 0, 1000), rng.uniform(0, 1, 1000)
    got = njit(cases.clip_arrays)(hip.asarray(a), hip.asarray(lo), hip.asarray(hi)).asnumpy()
    np.testing.assert_array_equal(got, np.clip(a, lo, hi))
    ai = rng.integers(-100, 100, 500).astype(np.int32)
    got = njit(cases.clip_arrays)(hip.asarray(ai), np.int32(-7), np.int32(11)).asnumpy()
    np.testing.assert_array_equal(got, np.clip(ai, -7, 11))
    assert got.dtype == np.int32


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32])
def test_mean(env, dtype):
    """numpy.mean / array.mean (numpy/funcs.py:306-328): the sum over the
    count in the array's float type, float64 for integers."""
    hip = env[0]
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((300, 170)) * 10).astype(dtype)
    rtol = 2e-6 if dtype == np.float32 else 1e-12
    dx = hip.asarray(x)
    for func, want in ((cases.mean_all, np.mean(x)), (cases.mean_rows, x.mean(axis=1)),
                       (cases.mean_cols, np.mean(x, axis=0))):
        f = njit(func)
        got = f(dx)
        assert f.last_launch["path"] == "library"
        got = got.asnumpy() if hasattr(got, "asnumpy") else got
        assert np.asarray(got).dtype == np.asarray(want).dtype
        np.testing.assert_allclose(got, want, rtol=rtol, atol=1e-6 if dtype == np.float32 else 0)


def test_bodies_mixing_maps_reductions_and_products(env):
    """Straight-line bodies are split at their reductions and matrix products:
    maps run as fused kernels, the rest on the hand-written kernels
    (test_l2_norm, test_gpu.py:2198-2223, is the first case)."""
    hip = env[0]
    rng = np.random.default_rng(21)

    def run(func, *host, rtol=1e-12):
        f = njit(func)
        dev = [hip.asarray(h) if isinstance(h, np.ndarray) else h for h in host]
        got = f(*dev)
        assert f.last_launch["path"] == "staged"
        want = func(*[h.copy() if isinstance(h, np.ndarray) else h for h in host])
        if want is not None:
            got = got.asnumpy() if hasattr(got, "asnumpy") else got
            np.testing.assert_allclose(got, want, rtol=rtol)
            assert np.asarray(got).shape == np.asarray(want).shape
        return f, dev

    a64 = rng.standard_normal((65, 25))
    f, _ = run(cases.l2_norm_rows, a64)
    # the square runs inside the row sums, the root is a map of its own
    assert [s["path"] for s in f.last_launch["stages"]] == ["kernel", "elementwise"]
    # float32 row-major input: the fused row-norm kernel serves the whole body
    a32 = a64.astype(np.float32)
    for func in (cases.l2_norm_rows, cases.l2_norm_rows_product):
        g = njit(func)
        got = g(hip.asarray(a32))
        assert g.last_launch["path"] == "library"
        assert g.last_launch["kernel"].startswith("nmk_norm2_axis1")
        np.testing.assert_allclose(got.asnumpy(), func(a32), rtol=1e-5)
    x = rng.standard_normal(1000)
    run(cases.softmax, x)
    m = rng.standard_normal((200, 33))
    run(cases.standardise, m)
    run(cases.column_range, m)
    a, b, c = (rng.standard_normal(s) for s in ((40, 30), (30, 20), (20,)))
    run(cases.affine, a, b, c)
    run(cases.chain, a, b, rng.standard_normal((20, 10)))
    run(cases.cosine, x, rng.standard_normal(1000))
    run(cases.matvec, a, rng.standard_normal(30))
    w = rng.standard_normal(30)
    out = np.zeros(40)
    f, dev = run(cases.weighted_rows, a, w, out)
    want = np.zeros(40)
    cases.weighted_rows(a, w, want)
    np.testing.assert_allclose(dev[2].asnumpy(), want, rtol=1e-12)
    # a second call reuses the stage functions
    f(*dev)
    np.testing.assert_allclose(dev[2].asnumpy(), want, rtol=1e-12)
    assert len(f._stage_funcs) == 3


def test_compiled_functions_apply_others_to_whole_arrays(env):
    """test_cfd_indirect / test_cfd_reshape (test_gpu.py:1737-1768, 1934-1964):
    a compiled function whose statement is a call of another one, and a
    reshape of an argument that is then filled."""
    hip = env[0]
    inner = njit(cases.scale_into)

    def outer(a, b):
        inner(a, b)

    a = np.arange(1024, dtype=np.float32)
    da, db = hip.asarray(a), hip.asarray(np.zeros_like(a))
    f = njit(outer)
    f(da, db)
    assert f.last_launch["path"] == "staged"
    np.testing.assert_array_equal(db.asnumpy(), a * 2)

    fill = njit(cases.reshape_fill)

    def outer2(a):
        fill(a)

    x = np.arange(17 * 23 * 56, dtype=np.float32).reshape(23, 56, 17).copy()
    dx = hip.asarray(x)
    njit(outer2)(dx)
    np.testing.assert_array_equal(dx.asnumpy(), np.full_like(x, 42))

    m = np.random.default_rng(3).standard_normal((30, 50))
    got = njit(cases.transposed_sum)(hip.asarray(m))
    np.testing.assert_allclose(got.asnumpy(), cases.transposed_sum(m), rtol=1e-12)


@pytest.mark.parametrize("func", [cases.dot_out_positional, cases.dot_out_keyword])
def test_dot_into_an_existing_array(env, func):
    """test_cfd_dot (test_gpu.py:2101-2138): the reference's exact fixture."""
    hip = env[0]
    a = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    b = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    dc = hip.asarray(np.zeros((2, 2), np.float32))
    f = njit(func)
    res = f(hip.asarray(a), hip.asarray(b), dc)
    assert f.last_launch["path"] == "library"
    np.testing.assert_array_equal(dc.asnumpy(), [[22, 28], [49, 64]])
    np.testing.assert_array_equal(res.asnumpy(), [[22, 28], [49, 64]])


def _matmul_operator(a, b):
    return a @ b


def _np_dot(a, b):
    return np.dot(a, b)


@pytest.mark.parametrize("func", [_matmul_operator, _np_dot])
def test_products_with_vectors(env, func):
    """A matrix times a vector, a vector times a matrix and two vectors
    (numpy/funcs.py:879-930: rank 1 operands of dot and of ``@`` take the
    rank numpy gives the result)."""
    hip = env[0]
    rng = np.random.default_rng(3)
    A = rng.standard_normal((1300, 700))
    v, w = rng.standard_normal(700), rng.standard_normal(1300)
    f = njit(func)
    got = f(hip.asarray(A), hip.asarray(v))
    assert f.last_launch["path"] == "library" and got.shape == (1300,)
    np.testing.assert_allclose(got.asnumpy(), A @ v, rtol=1e-12, atol=1e-12)
    got = f(hip.asarray(w), hip.asarray(A))
    assert got.shape == (700,)
    np.testing.assert_allclose(got.asnumpy(), w @ A, rtol=1e-12, atol=1e-12)
    got = f(hip.asarray(v), hip.asarray(v))
    assert np.shape(got) == ()
    np.testing.assert_allclose(got, v @ v, rtol=1e-12)


@pytest.mark.parametrize("name,operands", [
    ("built_arange_steps", "x"), ("built_arange_count", "x"), ("built_arange_down", "x"),
    ("built_eye", "A"), ("built_eye_square", "A"), ("built_triangles", "A"),
    ("built_outer", "uv"), ("built_concatenate_columns", "AC"),
    ("built_concatenate_three", "AR"), ("built_vstack", "AR"), ("built_hstack", "AC"),
    ("built_cov", "S"), ("built_cov_pair", "ST"), ("built_cov_columns", "C"),
    ("sliced_sums", "A"), ("sliced_differences", "A"), ("sliced_row", "A"),
    ("sliced_row_part", "A"), ("sliced_element", "A"), ("sliced_element_returned", "A"),
    ("copied_transpose", "A"), ("copied_method", "A"), ("flattened_transpose", "A"),
    ("facts_in_a_map", "A"), ("facts_after_a_reduction", "A"), ("facts_of_layout", "A"),
    ("facts_dtype", "A"), ("converted", "x"), ("converted_down", "x"),
    ("built_dstack", "AA"), ("copied_fortran", "A")])
def test_arrays_built_and_sliced_inside(env, name, operands):
    """np.arange / eye / tril / triu / outer / concatenate / hstack / vstack /
    cov / copy / flatten and basic indexing inside a compiled function: shape,
    type and values as NumPy gives them for the same function."""
    hip = env[0]
    rng = np.random.default_rng(17)
    A = rng.standard_normal((300, 200))
    pool = {"x": rng.standard_normal(5000), "A": A, "u": rng.standard_normal(300),
            "v": rng.standard_normal(200), "C": A[:, :7] * 2, "R": A[:9] * 2,
            "S": A[:6], "T": A[10:12]}
    func = getattr(cases, name)
    host = [np.ascontiguousarray(pool[k]) for k in operands]
    want = func(*host)
    got = njit(func)(*[hip.asarray(a) for a in host])
    got = got.asnumpy() if hasattr(got, "asnumpy") else got
    assert np.shape(got) == np.shape(want)
    assert np.asarray(got).dtype == np.asarray(want).dtype
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("name", ["store_slice", "store_column", "store_block_and_update_row",
                                  "update_shifted", "store_row_and_elements"])
def test_stores_into_slices(env, name):
    """x[1:5] = ..., x[:, 3] = ..., x[1:] += ...: stores into views of the
    array (array.__setitem__ with slices, numpy/funcs.py:1140-1195)."""
    hip = env[0]
    rng = np.random.default_rng(19)
    flat = name in ("store_slice", "update_shifted")
    a = rng.standard_normal(5000 if flat else (300, 200))
    b = rng.standard_normal(a.shape)
    func = getattr(cases, name)
    want = a.copy()
    func(want, b)
    d_a = hip.asarray(a)
    assert njit(func)(d_a, hip.asarray(b)) is None
    np.testing.assert_allclose(d_a.asnumpy(), want, rtol=1e-13)


def test_shapes_read_inside_a_map_that_is_not_straight_line(env):
    """A body with a branch is one fused map; where it reads an argument's
    shape or length the map walks the arrays with their own dimensions (not
    merged into one long row), and an argument that would be stretched to a
    larger shape is refused rather than seen with that shape."""
    hip = env[0]
    rng = np.random.default_rng(20)
    A = rng.standard_normal((300, 200))
    f = njit(cases.facts_under_a_branch)
    for host in (A, np.ascontiguousarray(A.T).T):
        dev = hip.asarray(np.ascontiguousarray(host.T)).T if not host.flags.c_contiguous \
            else hip.asarray(host)
        for flag in (True, False):
            np.testing.assert_allclose(f(dev, flag).asnumpy(),
                                       cases.facts_under_a_branch(host, flag), rtol=1e-13)
    assert f.last_launch["path"] == "elementwise"
    g = njit(cases.facts_of_a_stretched_operand)
    with pytest.raises(Exception, match="broadcast"):
        g(hip.asarray(A), hip.asarray(A[0].copy()), True)


@pytest.mark.parametrize("name", ["update_overlapping", "store_overlapping",
                                  "store_reversed_onto_itself"])
def test_a_store_whose_operand_overlaps_its_target(env, name):
    """x[1:] += x[:-1]: NumPy reads the right-hand side in full before it
    stores; every work-item storing while others still read would not."""
    hip = env[0]
    a = np.random.default_rng(21).standard_normal(100_000)
    func = getattr(cases, name)
    want = a.copy()
    func(want)
    d_a = hip.asarray(a)
    njit(func)(d_a)
    np.testing.assert_array_equal(d_a.asnumpy(), want)


def test_invert_of_booleans_is_logical_not(env):
    hip = env[0]
    x = np.random.default_rng(22).standard_normal(5000)
    f = njit(cases.inverted)
    got = f(hip.asarray(x > 0)).asnumpy()
    assert got.dtype == np.bool_
    np.testing.assert_array_equal(got, ~(x > 0))
    counts = (x * 100).astype(np.int64)
    np.testing.assert_array_equal(f(hip.asarray(counts)).asnumpy(), ~counts)


def test_cov_keeps_float32_and_one_variable_is_a_scalar(env):
    """The reference's cov keeps the input's floating type (numpy/funcs.py:
    1490-1527: only integers become float64) and returns a scalar for one
    1-d variable (1547-1548)."""
    hip = env[0]
    rng = np.random.default_rng(18)
    a = rng.standard_normal((5, 4000)).astype(np.float32)
    f = njit(cases.built_cov)
    got = f(hip.asarray(a)).asnumpy()
    assert got.dtype == np.float32 and got.shape == (5, 5)
    np.testing.assert_allclose(got, np.cov(a.astype(np.float64)), rtol=1e-4, atol=1e-5)
    one = f(hip.asarray(a[0].astype(np.float64)))
    assert np.shape(one) == ()
    np.testing.assert_allclose(one, np.cov(a[0].astype(np.float64)), rtol=1e-12)
    counts = rng.integers(0, 50, (3, 1000))
    got = f(hip.asarray(counts)).asnumpy()
    assert got.dtype == np.float64
    np.testing.assert_allclose(got, np.cov(counts), rtol=1e-12)


@pytest.mark.parametrize("left,right", [(np.int64, np.int64), (np.int32, np.int32),
                                        (np.float32, np.float64), (np.float64, np.int64),
                                        (np.int32, np.float32)])
def test_products_of_integers_and_of_two_types(env, left, right):
    """``@`` and np.dot of integer matrices (the reference lowers those to
    linalg.matmul, numpy/funcs.py:889-906) and of operands of two types: the
    type NumPy gives, exact for integers."""
    hip = env[0]
    rng = np.random.default_rng(23)

    def draw(shape, dtype):
        if np.dtype(dtype).kind == "i":
            return rng.integers(-5, 6, shape).astype(dtype)
        return rng.standard_normal(shape).astype(dtype)

    a, b = draw((130, 70), left), draw((70, 45), right)
    for func in (_matmul_operator, _np_dot):
        f = njit(func)
        for x, y in ((a, b), (a, b[:, 0].copy()), (a[0].copy(), b)):
            want = func(x, y)
            got = f(hip.asarray(x), hip.asarray(y)).asnumpy()
            assert got.dtype == want.dtype and got.shape == want.shape
            if want.dtype.kind == "i":
                np.testing.assert_array_equal(got, want)
            else:
                np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)


def test_gemm_refuses_other_types_with_an_exception(env):
    """ops.gemm mirrors the reference's binding, which exists for float32 and
    float64 (numpy/funcs.py:848-864): anything else is a TypeError, not an
    abort inside the runtime."""
    hip = env[0]
    from numba_mlir_amd.mlir import ops
    a = hip.asarray(np.ones((4, 4), np.int64))
    with pytest.raises(TypeError, match="float32 and float64"):
        ops.dot(a, a)


@pytest.mark.parametrize("dtype", [np.int8, np.int16, np.uint8, np.uint16, np.uint32])
def test_reductions_of_narrow_integers(env, dtype):
    """Integer types narrower than the reduction kernels take are widened to
    int64 first: along an axis the sums are NumPy's in value and type, minima
    and maxima keep the input's type, the mean does not wrap round."""
    hip = env[0]
    rng = np.random.default_rng(24)
    x = rng.integers(1, 100, (500, 40)).astype(dtype)
    d_x = hip.asarray(x)
    got = njit(lambda a: np.sum(a, axis=0))(d_x).asnumpy()
    want = np.sum(x, axis=0)
    assert got.dtype == want.dtype
    np.testing.assert_array_equal(got, want)
    got = njit(lambda a: a.max(axis=1))(d_x).asnumpy()
    assert got.dtype == x.dtype
    np.testing.assert_array_equal(got, x.max(axis=1))
    assert njit(lambda a: np.min(a))(d_x) == x.min()
    np.testing.assert_allclose(njit(lambda a: np.mean(a))(d_x), x.mean(), rtol=1e-12)
    np.testing.assert_allclose(njit(lambda a: a.mean(axis=0))(d_x).asnumpy(), x.mean(axis=0),
                               rtol=1e-12)
    # over everything the total comes back in the input's type, as for int32
    total = njit(lambda a: a.sum())(d_x)
    assert total == np.sum(x).astype(dtype)


@pytest.mark.parametrize("name,operands", [
    ("distances_to_centres", "XC"), ("softmax_rows", "X"), ("covariance_of_columns", "X"),
    ("ridge_gradient", "Xywl"), ("cosine_to_centres", "XC")])
def test_whole_array_recipes(env, name, operands):
    """Recipes of a few lines over a tall matrix -- distances to centres, a
    softmax per row, the covariance of columns, a gradient -- that mix
    reductions, reshape(-1, 1), broadcasting and products with thin and
    transposed operands: the values NumPy gives."""
    hip = env[0]
    rng = np.random.default_rng(25)
    pool = {"X": rng.standard_normal((20000, 16)), "C": rng.standard_normal((8, 16)),
            "y": rng.standard_normal(20000), "w": rng.standard_normal(16), "l": 0.1}
    func = getattr(cases, name)
    host = [pool[k] for k in operands]
    want = func(*host)
    got = njit(func)(*[hip.asarray(a) if isinstance(a, np.ndarray) else a for a in host])
    got = got.asnumpy()
    assert got.shape == want.shape and got.dtype == want.dtype
    np.testing.assert_allclose(got, want, rtol=1e-9, atol=1e-9)


def test_pairwise_as_nested_prange_loops(env):
    """test_pairwise2 (test_gpu.py:2226-2266): the distance body as two
    prange loops around a serial one, on the reference's fixture."""
    hip = env[0]
    a = np.arange(128 * 3, dtype=np.float32).reshape(128, 3)
    b = a + 5
    want = np.zeros((128, 128), np.float32)
    cases.pairwise_loop(a, b, want)
    dD = hip.asarray(np.zeros_like(want))
    f = njit(parallel=True)(cases.pairwise_loop)
    f(hip.asarray(a), hip.asarray(b), dD)
    assert f.last_launch["path"] == "parallel loop"
    np.testing.assert_allclose(dD.asnumpy(), want, rtol=1e-5)


def test_batchnorm(env):
    """test_batchnorm (test_numpy.py): allocations, reductions along the
    first axis of a 4-d array, broadcast stores and maps in one body."""
    hip = env[0]
    rng = np.random.default_rng(42)
    x = rng.random((8, 14, 14, 32), dtype=np.float32)
    f = njit(cases.batchnorm4, parallel=True)
    got = f(hip.asarray(x), 1e-5)
    assert f.last_launch["path"] == "staged"
    np.testing.assert_allclose(got.asnumpy(), cases.batchnorm(x), rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("a_shape, b_shape",
                         [((2, 3, 4), (2, 1, 4)), ((1, 2, 3), (1, 1)), ((2, 3, 4), (3, 4)),
                          ((5, 6, 7, 8), (1, 7, 8)), ((3, 4, 5, 6, 7), (5, 6, 7)),
                          ((5, 6, 7, 8), (6, 1, 8)), ((2, 3, 4, 5, 6), (3, 1, 5, 1))])
def test_broadcast_setitem(env, a_shape, b_shape):
    """test_broadcast_setitem (test_numpy.py), plus ranks above three whose
    dimensions merge, and ones that do not (one launch per leading index)."""
    import math
    hip = env[0]
    a = np.zeros(a_shape)
    b = np.arange(math.prod(b_shape)).reshape(b_shape)
    da = hip.asarray(a)
    got = njit(cases.broadcast_setitem)(da, hip.asarray(b))
    want = cases.broadcast_setitem(a.copy(), b)
    np.testing.assert_array_equal(got.asnumpy(), want)
    np.testing.assert_array_equal(da.asnumpy(), want)
    # the same operands through a map that returns a new array
    got = njit(cases.fused_map)(da, hip.asarray(b), hip.asarray(b), 0.5)
    np.testing.assert_allclose(got.asnumpy(), cases.fused_map(want, b, b, 0.5), rtol=1e-13)


@pytest.mark.parametrize("name,func", cases.OUT_FORMS, ids=[c[0] for c in cases.OUT_FORMS])
def test_functions_with_an_out_array(env, name, func):
    """test_binary_inplace (test_numpy.py): the third argument receives the
    result and is what the call returns."""
    hip = env[0]
    rng = np.random.default_rng(9)
    a, b = rng.uniform(0.5, 3, (6, 7)), rng.uniform(0.5, 3, (7,))
    want = np.zeros((6, 7))
    func(a, b, want)
    dc = hip.asarray(np.zeros((6, 7)))
    res = njit(func)(hip.asarray(a), hip.asarray(b), dc)
    np.testing.assert_allclose(dc.asnumpy(), want, rtol=1e-13)
    assert res is dc


def test_clip_with_out_and_allocations(env):
    hip = env[0]
    rng = np.random.default_rng(10)
    a, lo, hi = rng.uniform(-2, 2, 50), rng.uniform(-1, 0, 50), rng.uniform(0, 1, 50)
    out = hip.asarray(np.zeros(50))
    njit(cases.clip_out)(hip.asarray(a), hip.asarray(lo), hip.asarray(hi), out)
    np.testing.assert_array_equal(out.asnumpy(), np.clip(a, lo, hi))
    x = rng.uniform(-2, 2, (9, 11))
    got = njit(cases.zeros_ones)(hip.asarray(x))
    np.testing.assert_allclose(got.asnumpy(), cases.zeros_ones(x), rtol=1e-13)


@pytest.mark.parametrize("name,func", cases.TRANSPOSES + cases.FLIPS,
                         ids=[str(c[0]) for c in cases.TRANSPOSES + cases.FLIPS])
def test_transpose_and_flip_are_views(env, name, func):
    """test_transpose, test_flip1 (test_numpy.py): every permutation of the
    axes, flips along each axis; no data moves."""
    hip = env[0]
    a = np.arange(3 * 4 * 5).reshape(3, 4, 5)
    da = hip.asarray(a)
    got = njit(func)(da)
    np.testing.assert_array_equal(got.asnumpy(), func(a))
    if "map" not in str(name) and name != "method":
        assert got._buffer is da._buffer


def test_affine_into_an_existing_array(env):
    hip = env[0]
    rng = np.random.default_rng(13)
    a, b, c = rng.standard_normal((20, 30)), rng.standard_normal((30, 10)), \
        rng.standard_normal(10)

    def affine(a, b, c, out):
        np.add(np.dot(a, b), c, out)

    out = hip.asarray(np.zeros((20, 10)))
    njit(affine)(hip.asarray(a), hip.asarray(b), hip.asarray(c), out)
    np.testing.assert_allclose(out.asnumpy(), a @ b + c, rtol=1e-12)


def test_maps_run_inside_full_reductions(env):
    """np.sum / np.mean over everything of an expression of same-shaped dense
    arrays is one kernel: the map is evaluated inside the reduction loop."""
    hip = env[0]
    rng = np.random.default_rng(31)
    a, b = rng.standard_normal((257, 129)), rng.standard_normal((257, 129))

    def run(func, *host, rtol=1e-12, fused=True):
        f = njit(func)
        got = f(*[hip.asarray(h) for h in host])
        want = func(*host)
        np.testing.assert_allclose(got, want, rtol=rtol)
        assert np.asarray(got).dtype == np.asarray(want).dtype, func.__name__
        marks = [s.get("fused") for s in f.last_launch["stages"]]
        assert ("map + sum" in marks) == fused, f.last_launch
        return f

    run(cases.frobenius, a, b)
    run(cases.mean_abs_difference, a, b)
    run(cases.count_greater, a, b)
    a32, b32 = a.astype(np.float32), b.astype(np.float32)
    run(cases.frobenius, a32, b32, rtol=1e-5)
    run(cases.mean_abs_difference, a32, b32, rtol=1e-5)
    ai = rng.integers(-100, 100, (64, 33)).astype(np.int32)
    run(cases.sum_of_integer_squares, ai)
    # operands of different shapes take the map and the reduction separately
    run(cases.weighted_total, a, rng.standard_normal(129), fused=False)
    # views that are not dense, too
    f = njit(cases.frobenius)
    got = f(hip.asarray(a)[::2], hip.asarray(b)[::2])
    np.testing.assert_allclose(got, cases.frobenius(a[::2], b[::2]), rtol=1e-12)


def test_concurrent_calls_from_python_threads(env):
    """Compiled functions are called from Python threads holding no lock of
    the runtime (GpuRuntime.cpp:275-300 pools events per queue): calls of one
    function on different arrays from several threads must not mix up the
    stored launch's pointer and scalar slots."""
    import threading
    hip = env[0]
    f = njit(cases.fused_map)
    g = njit(parallel=True)(cases.saxpy_loop)
    rng = np.random.default_rng(41)
    n, rounds, errors = 4096, 40, []
    f(*(hip.asarray(rng.standard_normal(n)) for _ in range(3)), 1.0)       # compile once
    g(1.0, hip.asarray(np.zeros(n)), hip.asarray(np.zeros(n)), hip.asarray(np.zeros(n)))

    def worker(seed):
        try:
            local = np.random.default_rng(seed)
            for k in range(rounds):
                a, b, c = (local.standard_normal(n) for _ in range(3))
                scale = float(seed + k)
                got = f(hip.asarray(a), hip.asarray(b), hip.asarray(c), scale).asnumpy()
                # (sin differs in the last place and t*t - t cancels)
                np.testing.assert_allclose(got, cases.fused_map(a, b, c, scale), rtol=1e-9,
                                           atol=1e-9)
                out = hip.asarray(np.zeros(n))
                g(scale, hip.asarray(a), hip.asarray(b), out)
                np.testing.assert_array_equal(out.asnumpy(), scale * a + b)
        except Exception as exc:          # noqa: BLE001 -- reported by the main thread
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(s,)) for s in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[0]


@pytest.mark.parametrize("shape", [(257, 129), (1000, 36), (64, 2048), (5, 300)])
def test_maps_run_inside_axis_reductions(env, shape):
    """np.sum / np.mean along an axis of an expression of same-shaped dense
    matrices is one generated kernel (plus the column-sum kernel over the
    partial sums for axis 0)."""
    hip = env[0]
    rng = np.random.default_rng(51)
    a, b = rng.standard_normal(shape), rng.standard_normal(shape)

    def run(func, *host, rtol=1e-11, fused=True):
        f = njit(func)
        got = f(*[hip.asarray(h) if isinstance(h, np.ndarray) else h for h in host])
        want = func(*host)
        assert got.shape == want.shape and got.dtype == want.dtype, func.__name__
        # (NumPy's own float32 sums carry an absolute error of this size)
        np.testing.assert_allclose(got.asnumpy(), want, rtol=rtol,
                                   atol=1e-12 if rtol < 1e-6 else 1e-5)
        marks = [s.get("fused") for s in f.last_launch["stages"]]
        assert ("map + axis sum" in marks) == fused, f.last_launch

    rows_fused = shape[0] >= 64
    run(cases.row_dots, a, b, fused=rows_fused)
    run(cases.row_mean_abs, a, b, 0.5, fused=rows_fused)
    columns_fused = shape[1] % 4 == 0
    run(cases.column_variance, a, b, fused=columns_fused)
    run(cases.column_counts, a, b, fused=columns_fused)
    a32, b32 = a.astype(np.float32), b.astype(np.float32)
    run(cases.row_dots, a32, b32, rtol=2e-5, fused=rows_fused)
    run(cases.column_variance, a32, b32, rtol=2e-5, fused=columns_fused)
    ai, bi = rng.integers(-9, 9, shape).astype(np.int32), rng.integers(-9, 9, shape).astype(np.int32)
    run(cases.row_dots, ai, bi, fused=rows_fused)
    # a broadcast operand: the map and the reduction run separately
    run(cases.row_dots, a, rng.standard_normal(shape[1]), fused=False)


def test_fused_map_over_tall_strided_views(env):
    """Two of three columns of ten million rows: the fused map's grid has
    more blocks of rows than a launch holds along y."""
    hip = env[0] if isinstance(env, tuple) else env
    rng = np.random.default_rng(29)
    a = rng.standard_normal((10_000_000, 3))
    b = rng.standard_normal((10_000_000, 3))
    f = njit(lambda x, y: x * 2.0 + y)
    got = f(hip.asarray(a)[:, :2], hip.asarray(b)[:, :2]).asnumpy()
    assert np.array_equal(got, a[:, :2] * 2.0 + b[:, :2])


def test_staged_reductions_of_a_lambda(env):
    """A lambda's stages get kernels too (its name is no identifier)."""
    hip = env[0]
    x = np.random.default_rng(31).uniform(0.5, 1.5, (50_000, 3)).astype(np.float32)
    got = njit(lambda a: np.sum(a * a, axis=1))(hip.asarray(x)).asnumpy()
    np.testing.assert_allclose(got, (x.astype(np.float64) ** 2).sum(axis=1), rtol=1e-5)
    got = njit(lambda a: np.mean(np.abs(a)))(hip.asarray(x))
    np.testing.assert_allclose(got, np.abs(x).astype(np.float64).mean(), rtol=1e-5)
