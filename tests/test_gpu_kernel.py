"""GPU parity: @kernel launches (hand-written twins) against the kernel
simulator, the oracle of every kernel test in the reference."""

import json
import math
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
    GOLD = json.load(f)

SHAPES = [tuple(s) for s in GOLD["kernel_shapes"]["shapes"]]
LSIZES = [tuple(s) for s in GOLD["kernel_shapes"]["local_sizes"]]


@pytest.fixture(scope="module")
def env(hip):
    from numba_mlir_amd import kernel as kapi
    from numba_mlir_amd.mlir import ops
    from oracle import oracle as orc
    from oracle.kernel_sim import kernel_sim
    return hip, kapi, ops, orc, kernel_sim


# The bodies below are the reference's (tests/test_gpu.py:580-803); the stubs
# are bound per test module so the simulator can patch them.
def get_global_id(k): raise NotImplementedError
def get_local_id(k): raise NotImplementedError
def get_group_id(k): raise NotImplementedError
def get_global_size(k): raise NotImplementedError
def get_local_size(k): raise NotImplementedError


def _id_funcs(getter):
    def func1(c):
        i = get_global_id(0)
        c[i] = getter(0)

    def func2(c):
        i = get_global_id(0)
        j = get_global_id(1)
        c[i, j] = getter(0) + getter(1) * 100

    def func3(c):
        i = get_global_id(0)
        j = get_global_id(1)
        k = get_global_id(2)
        c[i, j, k] = getter(0) + getter(1) * 100 + getter(2) * 10000

    return [func1, func2, func3]


_BUILTINS = {
    "get_global_id": lambda k: get_global_id(k),
    "get_local_id": lambda k: get_local_id(k),
    "get_group_id": lambda k: get_group_id(k),
    "get_global_size": lambda k: get_global_size(k),
    "get_local_size": lambda k: get_local_size(k),
}


@pytest.mark.parametrize("builtin", sorted(_BUILTINS))
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("lsize", [()] + LSIZES)
def test_index_builtins(env, builtin, shape, lsize):
    hip, kapi, _, _, kernel_sim = env
    if lsize == () and builtin in ("get_local_id", "get_group_id", "get_local_size"):
        pytest.skip("depends on the runtime-chosen block; covered with explicit sizes")
    func = _id_funcs(_BUILTINS[builtin])[len(shape) - 1]
    ls = tuple(lsize[:len(shape)])

    sim_res = np.zeros(shape, np.int32)
    kernel_sim(func)[shape, ls](sim_res)

    gpu_func = kapi.kernel(func, twin="nmk_twin_" + builtin + "_{rank}")
    d = hip.asarray(np.zeros(shape, np.int32))
    gpu_func[shape, ls](d)
    np.testing.assert_array_equal(d.asnumpy(), sim_res)

    launch = gpu_func[shape, ls]
    launch(d)
    block, grid = launch.last_launch["block"], launch.last_launch["grid"]
    for k, g in enumerate(shape):
        assert grid[k] == -(-g // block[k])
    if ls:
        assert block[:len(ls)] == ls


def test_default_block_matches_runtime_suggestion(env):
    hip, kapi, _, orc, _ = env
    func = _id_funcs(_BUILTINS["get_global_id"])
    for shape in SHAPES + [(4096, 4096), (300, 5, 5)]:
        k = kapi.kernel(func[len(shape) - 1],
                        twin="nmk_twin_get_global_id_{rank}")[shape, ()]
        if np.prod(shape) > 1 << 20:
            continue
        d = hip.asarray(np.zeros(shape, np.int32))
        k(d)
        assert k.last_launch["block"][:len(shape)] == \
            orc.suggest_block_size(256, shape)


@pytest.mark.parametrize("op", GOLD["unary_input"]["funcs"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_math_funcs_unary(env, op, dtype):
    """tests/test_gpu.py:524-548: b[i] = math.<op>(a[i]), rtol 1e-5."""
    hip, kapi, _, _, kernel_sim = env
    f = getattr(math, op)

    def func(a, b):
        i = get_global_id(0)
        b[i] = f(a[i])

    a = np.array(GOLD["unary_input"]["a"], dtype)
    sim_res = np.zeros(a.shape, dtype)
    kernel_sim(func)[a.shape, ()](a, sim_res)

    d_a, d_b = hip.asarray(a), hip.asarray(np.zeros(a.shape, dtype))
    kapi.kernel(func, twin="nmk_twin_unary_" + op + "_{dtype}")[a.shape, ()](d_a, d_b)
    np.testing.assert_allclose(d_b.asnumpy(), sim_res, rtol=GOLD["unary_input"]["rtol"])


def _pairwise_body(X1, X2, D):
    i = get_global_id(0)
    j = get_global_id(1)

    X1_cols = X1.shape[1]

    d = 0.0
    for k in range(X1_cols):
        tmp = X1[i, k] - X2[j, k]
        d += tmp * tmp
    D[i, j] = np.sqrt(d)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pairwise_reference_fixture(env, dtype):
    """test_pairwise1 (tests/test_gpu.py:1396-1430)."""
    hip, kapi, _, orc, kernel_sim = env
    g = GOLD["pairwise"]
    n, dims = g["npoints"], g["dims"]
    a = np.arange(n * dims, dtype=dtype).reshape(n, dims)
    b = a + 5

    sim_res = np.zeros((n, n), dtype)
    kernel_sim(_pairwise_body)[(n, n), ()](a, b, sim_res)

    d_a, d_b = hip.asarray(a), hip.asarray(b)
    d_res = hip.asarray(np.zeros((n, n), dtype))
    gpu_func = kapi.kernel(_pairwise_body, twin="nmk_twin_pairwise_{dtype}")
    gpu_func[(n, n), ()](d_a, d_b, d_res)
    got = d_res.asnumpy()
    np.testing.assert_allclose(got, sim_res, rtol=g["rtol"])
    i, j = np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
    np.testing.assert_allclose(got, math.sqrt(3.0) * np.abs(3.0 * (i - j) - 5.0),
                               rtol=g["rtol"])
    np.testing.assert_allclose(got, orc.pairwise(a, b), rtol=1e-6 if dtype == np.float32 else 1e-12)
    # explicit local size, ragged against the global size
    d_res2 = hip.asarray(np.zeros((n, n), dtype))
    gpu_func[(n, n), (24, 5)](d_a, d_b, d_res2)
    assert d_res2.asnumpy().tobytes() == got.tobytes()


@pytest.mark.parametrize("n1,n2", [(1, 2), (5, 8), (130, 514), (1024, 1026)])
def test_pairwise_remapped_twin_equals_faithful_twin(env, n1, n2):
    hip, kapi, ops, orc, _ = env
    rng = np.random.Generator(np.random.PCG64(1004))
    X, Y = rng.uniform(0, 1, (n1, 3)), rng.uniform(0, 1, (n2, 3))
    d_X, d_Y = hip.asarray(X), hip.asarray(Y)
    D1 = hip.empty((n1, n2), np.float64)
    kapi.kernel(_pairwise_body, twin="nmk_twin_pairwise_{dtype}")[(n1, n2), ()](d_X, d_Y, D1)
    D2 = hip.empty((n1, n2), np.float64)
    ops.pairwise_distance(d_X, d_Y, D2)
    assert hip.get_context().last_kernel() == "nmk_twin_pairwise_f64_rows"
    assert D1.asnumpy().tobytes() == D2.asnumpy().tobytes()
    np.testing.assert_allclose(D2.asnumpy(), orc.pairwise(X, Y), rtol=1e-12)


def test_pairwise_full_size(env):
    """Configuration 4: X, Y [8192, 3] float64 -> D [8192, 8192], rel 1e-12."""
    hip, _, ops, orc, _ = env
    from numba_mlir_amd import workloads
    X, Y = workloads.pairwise()
    D = hip.empty((8192, 8192), np.float64)
    ops.pairwise_distance(hip.asarray(X), hip.asarray(Y), D)
    got = D.asnumpy()
    np.testing.assert_allclose(got, orc.pairwise(X, Y), rtol=1e-12)
    # size-independent property: D(X, X) is symmetric with a zero diagonal
    ops.pairwise_distance(hip.asarray(X), hip.asarray(X), D)
    got = D.asnumpy()
    assert (np.diag(got) == 0).all() and np.array_equal(got, got.T)


def test_large_1d_launch_ids_do_not_wrap(env):
    """A 1-D launch of 2^31 + 1 work-items must address every id
    (tests/test_gpu.py:2269-2283)."""
    hip, kapi, _, _, _ = env

    def func(c):
        i = get_global_id(0)
        c[i] = i

    n = 2 ** 31 + 1
    k = kapi.kernel(func, twin="nmk_twin_get_global_id_1")[(n,), (256,)]
    # stride-0 view: every work-item writes c[0]; the grid must be accepted
    # and cover ceil(n / 256) blocks.
    from numba_mlir_amd.mlir.device_array import HipNdArray
    base = hip.asarray(np.zeros(1, np.int32))
    view = HipNdArray(base._buffer, (n,), np.int32, (0,), 0)
    k(view)
    assert k.last_launch["grid"][0] == (n + 255) // 256
    hip.get_context().synchronize()


def test_kernel_argument_checks(env):
    hip, kapi, _, _, _ = env
    k = kapi.kernel(lambda c: None, twin="nmk_twin_get_global_id_1")
    with pytest.raises(ValueError):
        k[(1, 2, 3, 4)]
    with pytest.raises(ValueError):
        k[4, 4, 4]
    with pytest.raises(ValueError):
        k[(4,), ()](hip.asarray(np.zeros(4, np.int32)), x=1)
    with pytest.raises(ValueError):
        k[(4,), ()](3)
    def unsupported(c):
        c[0] = [1, 2][0]

    with pytest.raises(kapi.KernelCompileError, match="line 2: Unsupported expression: List"):
        kapi.kernel(unsupported)[(4,), ()](hip.asarray(np.zeros(4, np.int32)))
    with pytest.raises(NotImplementedError):
        kapi.get_global_id(0)
