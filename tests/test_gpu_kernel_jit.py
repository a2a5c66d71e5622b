"""GPU parity: Python @kernel bodies translated and compiled for gfx950, run
through the gpux C-ABI, against the kernel simulator (the oracle of every
kernel test in the reference).  Bodies, inputs and tolerances are the
reference's own tests (numba_mlir/numba_mlir/mlir/tests/test_gpu.py, line
ranges per test) plus cases for the translator's typing rules."""

import json
import math
import os

import numpy as np
import pytest

from numba_mlir_amd import kernel as K

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_vectors.json")) as f:
    GOLD = json.load(f)

get_global_id, get_local_id = K.get_global_id, K.get_local_id
get_group_id, get_global_size = K.get_group_id, K.get_global_size
get_local_size = K.get_local_size
barrier, mem_fence = K.barrier, K.mem_fence
LOCAL_MEM_FENCE, GLOBAL_MEM_FENCE = K.LOCAL_MEM_FENCE, K.GLOBAL_MEM_FENCE
DEFAULT_LOCAL_SIZE = K.DEFAULT_LOCAL_SIZE
atomic, local, private, group = K.atomic, K.local, K.private, K.group
kernel_func = K.kernel_func

STUBS = {
    "get_global_id": K.get_global_id, "get_local_id": K.get_local_id,
    "get_group_id": K.get_group_id, "get_global_size": K.get_global_size,
    "get_local_size": K.get_local_size, "barrier": K.barrier,
    "mem_fence": K.mem_fence, "atomic_add": K.atomic.add,
    "atomic_sub": K.atomic.sub, "local_array": K.local.array,
    "private_array": K.private.array,
    "group_reduce_add": K.group.reduce_add, "group_reduce_mul": K.group.reduce_mul,
    "group_reduce_min": K.group.reduce_min, "group_reduce_max": K.group.reduce_max,
}


@pytest.fixture(scope="module")
def env(hip):
    from oracle.kernel_sim import kernel_sim
    return hip, lambda f: kernel_sim(f, STUBS)


def check(env, func, gsize, lsize, args, exact=True, rtol=1e-5, simulate=True,
          race_free=True):
    """Runs ``func`` in the simulator and on the GPU over copies of ``args``
    and compares every array argument afterwards; returns the GPU results.
    The GPU runs it twice: first the bounds-checked build (a wrong index is an
    IndexError, not a memory fault), then the plain one, which must agree."""
    hip, sim = env
    outs = []
    for boundscheck in (True, False):
        dev = [hip.asarray(a.copy()) if isinstance(a, np.ndarray) else a for a in args]
        K.kernel(func, boundscheck=boundscheck)[gsize, lsize](*dev)
        outs.append([d.asnumpy() if isinstance(a, np.ndarray) else a
                     for d, a in zip(dev, args)])
    for checked, plain in zip(*outs):
        if isinstance(checked, np.ndarray) and race_free:
            np.testing.assert_array_equal(plain, checked)
    out = outs[1]
    if simulate:
        ref = [a.copy() if isinstance(a, np.ndarray) else a for a in args]
        sim(func)[gsize, lsize](*ref)
        for got, want in zip(out, ref):
            if isinstance(want, np.ndarray):
                if exact:
                    np.testing.assert_array_equal(got, want)
                else:
                    np.testing.assert_allclose(got, want, rtol=rtol, atol=1e-30)
    return out


# ---- the reference's simple kernels ----------------------------------------

def test_simple1(env):                                       # 176-201
    def func(a, b, c):
        i = get_global_id(0)
        j = get_global_id(1)
        k = get_global_id(2)
        c[i, j, k] = a[i, j, k] + b[i, j, k]

    a = np.array([[[1, 2, 3], [4, 5, 6]]], np.float32)
    b = np.array([[[7, 8, 9], [10, 11, 12]]], np.float32)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, b, np.zeros(a.shape, a.dtype)])


def test_simple3(env):                                       # 234-259
    def func(a, b):
        i = get_global_id(0)
        b[i, 0] = a[i, 0]
        b[i, 1] = a[i, 1]

    a = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    check(env, func, a.shape[0], DEFAULT_LOCAL_SIZE, [a, np.zeros(a.shape, a.dtype)])


@pytest.mark.parametrize("val", [-3, 2, np.int32(5), 1.5, np.float32(2.5), True])
@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64])
def test_scalar_argument(env, dtype, val):                   # 289-316
    def func(a, b, c):
        i = get_global_id(0)
        c[i] = a[i] + b

    a = np.arange(-6, 6, dtype=dtype)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, val, np.zeros(a.shape, a.dtype)])


@pytest.mark.parametrize("val", [-3, 2.5, np.float32(7)])
def test_captured_constant(env, val):                        # 319-343
    def func(a, c):
        i = get_global_id(0)
        c[i] = a[i] + val

    a = np.arange(-6, 6, dtype=np.float32)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, np.zeros(a.shape, a.dtype)])


def test_empty_kernel(env):                                  # 346-362
    def func(a):
        pass

    a = np.array([[[1, 2, 3], [4, 5, 6]]], np.float32)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a])


def test_list_global_size_and_empty_local(env):              # 402-424
    def func(a, b, c):
        i = get_global_id(0)
        c[i] = a[i] + b[i]

    a = np.array([1, 2, 3, 4, 5, 6], np.float32)
    b = np.array([7, 8, 9, 10, 11, 12], np.float32)
    check(env, func, [a.shape[0]], [], [a, b, np.zeros(a.shape, a.dtype)])


def test_partial_indexing_gives_views(env):                  # 427-452
    def func(a, b):
        i = get_global_id(0)
        b1 = b[i]
        j = get_global_id(1)
        b2 = b1[j]
        k = get_global_id(2)
        b2[k] = a[i, j, k]

    a = np.arange(3 * 4 * 5).reshape((3, 4, 5))
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, np.zeros(a.shape, a.dtype)])


def test_inner_loop_with_data_dependent_bound(env):          # 455-481
    def func(a, b, c):
        i = get_global_id(0)
        res = 0.0
        for j in range(a[i]):
            res = res + b[j]
        c[i] = res

    a = np.array([1, 2, 3, 4], np.int32)
    b = np.array([5, 6, 7, 8, 9], np.float32)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, b, np.zeros(a.shape, b.dtype)])


@pytest.mark.parametrize("op", GOLD["unary_input"]["funcs"])
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_math_funcs_unary(env, op, dtype):                   # 484-548
    f = getattr(math, op)

    def func(a, b):
        i = get_global_id(0)
        b[i] = f(a[i])

    a = np.array(GOLD["unary_input"]["a"], dtype)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, np.zeros(a.shape, dtype)],
          exact=False, rtol=GOLD["unary_input"]["rtol"])


_BINARY = {
    "+": lambda a, b: a + b,
    "-": lambda a, b: a - b,
    "*": lambda a, b: a * b,
    "/": lambda a, b: a / b,
    "//": lambda a, b: a // b,
    "%": lambda a, b: a % b,
    "**": lambda a, b: a ** b,
}


@pytest.mark.parametrize("op", sorted(_BINARY))
@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64])
def test_ops_binary(env, op, dtype):                         # 551-566
    inner = kernel_func(_BINARY[op])

    def func(a, b, c):
        i = get_global_id(0)
        c[i] = inner(a[i], b[i])

    a = np.array([11, 12, 13, 14, 15], dtype)
    b = np.array([1, 2, 3, 4, 5], dtype)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, b, np.zeros(a.shape, dtype)],
          exact=False)
    if op != "**":      # signs: Python's floor and modulo conventions
        a2 = np.array([-11, 12, -13, 14, -15, 7, -7], dtype)
        b2 = np.array([3, -5, -4, 3, 7, -7, 7], dtype)
        check(env, func, a2.shape, DEFAULT_LOCAL_SIZE,
              [a2, b2, np.zeros(a2.shape, dtype)], exact=False)


# ---- index builtins (569-815) ----------------------------------------------

SHAPES = [tuple(s) for s in GOLD["kernel_shapes"]["shapes"]]
LSIZES = [tuple(s) for s in GOLD["kernel_shapes"]["local_sizes"]]
_GETTERS = {"get_global_id": get_global_id, "get_local_id": get_local_id,
            "get_group_id": get_group_id, "get_global_size": get_global_size,
            "get_local_size": get_local_size}


@pytest.mark.parametrize("builtin", sorted(_GETTERS))
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("lsize", [()] + LSIZES)
def test_index_builtins(env, builtin, shape, lsize):
    getter = _GETTERS[builtin]

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

    if len(lsize) not in (0, len(shape)):
        pytest.skip("local size of another rank")
    func = [func1, func2, func3][len(shape) - 1]
    # with a runtime-chosen block the local ids have no simulator counterpart
    simulate = len(lsize) != 0 or builtin in ("get_global_id", "get_global_size")
    out = check(env, func, shape, lsize, [np.zeros(shape, np.int32)], simulate=simulate)
    if not simulate:
        assert out[0].shape == shape


# ---- atomics (818-955) -----------------------------------------------------

@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64])
@pytest.mark.parametrize("opname", ["add", "sub"])
@pytest.mark.parametrize("mode,ret_size", [(0, 1), (1, 2)])
def test_atomics(env, dtype, opname, mode, ret_size):
    atomic_op = getattr(atomic, opname)

    if mode == 0:
        def func(a, b):
            i = get_global_id(0)
            atomic_op(b, 0, a[i])
    else:
        def func(a, b):
            i = get_global_id(0)
            atomic_op(b, i % 2, a[i])

    a = np.array([1, 2, 3, 4, 5, 6, 7, 8, 9], dtype)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, np.zeros([ret_size], dtype)])


def test_atomics_through_the_namespace(env):                 # 856-866
    def func(a, b):
        i = get_global_id(0)
        atomic.add(b, 0, a[i])

    # the simulator only patches direct calls (the reference marks this case
    # xfail for its own compiler); the translator resolves the attribute
    a = np.array([1, 2, 3, 4, 5, 6, 7, 8, 9], np.int32)
    out = check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, np.zeros([1], np.int32)],
                simulate=False)
    assert out[1][0] == a.sum()


@pytest.mark.parametrize("opname", ["add", "sub"])
@pytest.mark.parametrize("mode", [2, 3])
def test_atomics_different_types(env, opname, mode):         # 868-890
    atomic_op = getattr(atomic, opname)

    if mode == 2:
        def func(a, b):
            i = get_global_id(0)
            atomic_op(b, 0, a[i] + 1)
    else:
        def func(a, b):
            i = get_global_id(0)
            atomic_op(b, 0, 1)

    a = np.array([1, 2, 3, 4, 5, 6, 7, 8, 9], np.int32)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, np.zeros([1], np.int32)])


@pytest.mark.parametrize("funci", [1, 2])
def test_atomics_multidim(env, funci):                       # 892-925
    atomic_op = atomic.add

    def func1(a, b):
        i = get_global_id(0)
        j = get_global_id(1)
        atomic_op(b, (i % 2, 0), a[i, j])

    def func2(a, b):
        i = get_global_id(0)
        j = get_global_id(1)
        atomic_op(b, (i % 2, j % 2), a[i, j])

    func = func1 if funci == 1 else func2
    a = np.array([[1, 2, 3], [4, 5, 6], [7, 8, 9]], np.int32)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, np.zeros((2, 2), np.int32)])


def test_atomics_different_dims(env):                        # 927-955
    atomic_op = atomic.add

    def func(a, b, c):
        i = get_global_id(0)
        j = get_global_id(1)
        atomic_op(a, (i, j), c[i, j])
        atomic_op(b, (i), c[i, j])

    c = np.array([[1, 2, 3], [4, 5, 6]], np.int32)
    check(env, func, c.shape, DEFAULT_LOCAL_SIZE,
          [np.zeros(c.shape, np.int32), np.zeros(c.shape[0], np.int32), c])


@pytest.mark.parametrize("s", [slice(1, None, None), slice(None, 50, None),
                               slice(10, 90, 3), slice(None, None, -1),
                               slice(-20, -2, 2), slice(95, 5, -7)])
def test_slice_argument(env, s):                             # 958-976
    def func(s, res):
        i = get_global_id(0)
        res[s][i] = i

    res = np.zeros(100, dtype=np.int32)
    check(env, func, len(res[s]), DEFAULT_LOCAL_SIZE, [s, res])


def test_fastmath_off_keeps_two_roundings(env):              # 980-1008
    def func(a, b, c, res):
        i = get_global_id(0)
        res[i] = a[i] * b[i] + c[i]

    for a, b, c in (
        (np.array([1, 2, 3, 4], np.float32), np.array([5, 6, 7, 8], np.float32),
         np.array([9, 10, 11, 12], np.float32)),
        (np.array([1.0000001, 3.3333333, 1e-3, 7.7], np.float32),
         np.array([1.0000001, 3.0000001, 1e3, 1.3], np.float32),
         np.array([-1.0000002, -10.0, -1.0, -10.01], np.float32)),
    ):
        out = check(env, func, a.shape, DEFAULT_LOCAL_SIZE,
                    [a, b, c, np.zeros(a.shape, a.dtype)])
        assert out[3].tobytes() == (a * b + c).tobytes()


def test_fastmath_fuses_multiply_add(env):                   # 980-1008
    """kernel(fastmath=True): the reference expects exactly one fma for
    a * b + c.  A fused result is the exact product plus c rounded once."""
    hip = env[0]

    def func(a, b, c, res):
        i = get_global_id(0)
        res[i] = a[i] * b[i] + c[i]

    rng = np.random.default_rng(3)
    a = rng.uniform(1, 2, 4096).astype(np.float32)
    b = rng.uniform(1, 2, 4096).astype(np.float32)
    c = (-(a.astype(np.float64) * b)).astype(np.float32)       # cancels the leading bits
    dev = [hip.asarray(x) for x in (a, b, c)]
    fused, plain = hip.asarray(np.zeros_like(a)), hip.asarray(np.zeros_like(a))
    K.kernel(func, fastmath=True)[a.shape, ()](*dev, fused)
    K.kernel(func, fastmath=False)[a.shape, ()](*dev, plain)
    exact = (a.astype(np.float64) * b + c).astype(np.float32)  # the product is exact in double
    assert fused.asnumpy().tobytes() == exact.tobytes()
    assert plain.asnumpy().tobytes() == (a * b + c).tobytes()
    assert (fused.asnumpy() != plain.asnumpy()).any()


def test_accumulation_in_float32(env):                       # 1011-1040
    def func(a, b, res):
        i = get_global_id(0)
        d = np.float32(0)
        for j in range(10):
            d += a[i] * b[i]
        res[i] = d

    a = np.array([1, 2, 3, 4], np.float32)
    b = np.array([5, 6, 7, 8], np.float32)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, b, np.zeros(a.shape, a.dtype)])


# ---- barriers, local and private memory, group reductions (1074-1393) -------

@pytest.mark.parametrize("is_barrier", [1, 0])
@pytest.mark.parametrize("flags", [LOCAL_MEM_FENCE, GLOBAL_MEM_FENCE])
@pytest.mark.parametrize("global_size", [1, 2, 27, 67, 101])
@pytest.mark.parametrize("local_size", [1, 2, 7, 17, 33])
def test_barrier_ops(env, is_barrier, flags, global_size, local_size):
    op = barrier if is_barrier else mem_fence

    def func(a, b):
        i = get_global_id(0)
        v = a[i]
        op(flags)
        b[i] = a[i]

    a = np.arange(global_size, dtype=np.int64)
    check(env, func, global_size, local_size, [a, np.zeros(global_size, np.int64)])


@pytest.mark.parametrize("global_size", [1, 2, 4, 27, 67, 101])
@pytest.mark.parametrize("local_size", [1, 2, 7, 17, 33])
def test_barrier1(env, global_size, local_size):
    atomic_add = atomic.add

    def func(a, b):
        i = get_global_id(0)
        off = i // local_size
        atomic_add(a, off, i)
        barrier(GLOBAL_MEM_FENCE)
        b[i] = a[off]

    count = (global_size + local_size - 1) // local_size
    check(env, func, global_size, local_size,
          [np.zeros(count, np.int64), np.zeros(global_size, np.int64)])


@pytest.mark.parametrize("blocksize", [1, 10, 17, 64, 67, 101])
@pytest.mark.parametrize("two_d", [False, True])
def test_local_memory(env, blocksize, two_d):
    local_array = local.array

    if two_d:
        def func(A):
            lm = local_array(shape=(1, blocksize), dtype=np.float32)
            i = get_global_id(0)
            lm[0, i] = A[i]
            barrier(LOCAL_MEM_FENCE)
            A[i] += lm[0, blocksize - 1 - i]
    else:
        def func(A):
            lm = local_array(shape=blocksize, dtype=np.float32)
            i = get_global_id(0)
            lm[i] = A[i]
            barrier(LOCAL_MEM_FENCE)
            A[i] += lm[blocksize - 1 - i]

    check(env, func, blocksize, blocksize, [np.arange(blocksize).astype(np.float32)])


@pytest.mark.parametrize("blocksize", [1, 10, 17, 64, 67, 101])
@pytest.mark.parametrize("variant,priv_size", [(1, 1), (3, 1), (3, 11), (3, 27), (4, 100)])
def test_private_memory(env, blocksize, variant, priv_size):
    private_array = private.array

    if variant == 1:
        def func(A):
            i = get_global_id(0)
            prvt_mem = private_array(shape=1, dtype=np.float32)
            prvt_mem[0] = i
            barrier(LOCAL_MEM_FENCE)
            A[i] = prvt_mem[0] * 2
    elif variant == 3:
        def func(A):
            i = get_global_id(0)
            prvt_mem = private_array(shape=priv_size, dtype=np.float32)
            for j in range(priv_size):
                prvt_mem[j] = j + i
            res = 0
            for j in range(priv_size):
                res += prvt_mem[(j + i) % priv_size]
            A[i] = res
    else:
        def func(A):
            i = get_global_id(0)
            S = 10
            prvt_mem = private_array(shape=(S, S), dtype=np.float32)
            for j in range(S):
                for k in range(S):
                    prvt_mem[j, k] = i
            barrier(LOCAL_MEM_FENCE)
            A[i] = prvt_mem[i % S, i % S] * 2

    check(env, func, blocksize, blocksize, [np.zeros(blocksize, np.float32)],
          exact=False)


@pytest.mark.parametrize("opname", ["add", "mul", "min", "max"])
@pytest.mark.parametrize("global_size", [1, 2, 4, 27, 67, 101, 1000])
@pytest.mark.parametrize("local_size", [1, 2, 7, 17, 33, 64, 200, 256, 1024])
@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32, np.float64])
def test_group_func(env, opname, global_size, local_size, dtype):
    if global_size > 25 and opname == "mul":
        pytest.skip("products overflow (the reference skips them too)")
    group_op = getattr(group, "reduce_" + opname)

    def func(a, b):
        i = get_global_id(0)
        v = group_op(a[i])
        b[i] = v

    a = np.arange(global_size, dtype=dtype)
    # the simulator nests one greenlet per work-item: only the reference's sizes
    out = check(env, func, (global_size,), (local_size,),
                [a, np.zeros(global_size, dtype)], exact=False,
                simulate=local_size <= 33)
    fold = {"add": np.sum, "mul": np.prod, "min": np.min, "max": np.max}[opname]
    expect = np.empty(global_size, dtype)
    for start in range(0, global_size, local_size):
        stop = min(start + local_size, global_size)
        expect[start:stop] = fold(a[start:stop].astype(
            np.float64 if np.dtype(dtype).kind == "f" else dtype))
    np.testing.assert_allclose(out[1], expect, rtol=1e-5)


@pytest.mark.parametrize("shape,lsize", [((5, 7), (4, 4)), ((9, 3, 5), (4, 2, 4)),
                                         ((33, 2), (16, 2))])
def test_group_reduce_in_clipped_multidimensional_groups(env, shape, lsize):
    """The members of a clipped 2-d / 3-d group are not a prefix of its linear
    ids; every member must still see the sum over exactly the members."""
    def func2(a, b):
        i = get_global_id(0)
        j = get_global_id(1)
        b[i, j] = group.reduce_add(a[i, j])

    def func3(a, b):
        i = get_global_id(0)
        j = get_global_id(1)
        k = get_global_id(2)
        b[i, j, k] = group.reduce_add(a[i, j, k])

    a = np.arange(int(np.prod(shape)), dtype=np.int64).reshape(shape) + 1
    out = check(env, func2 if len(shape) == 2 else func3, shape, lsize,
                [a, np.zeros(shape, np.int64)], simulate=False)
    expect = np.zeros(shape, np.int64)
    ranges = [range(0, n, l) for n, l in zip(shape, lsize)]
    import itertools
    for corner in itertools.product(*ranges):
        sl = tuple(slice(c, min(c + l, n)) for c, l, n in zip(corner, lsize, shape))
        expect[sl] = a[sl].sum()
    np.testing.assert_array_equal(out[1], expect)


# ---- pairwise distance (1396-1430, 2226-2266) -------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_pairwise(env, dtype):
    def func(X1, X2, D):
        i = get_global_id(0)
        j = get_global_id(1)
        X1_cols = X1.shape[1]
        d = 0.0
        for k in range(X1_cols):
            tmp = X1[i, k] - X2[j, k]
            d += tmp * tmp
        D[i, j] = np.sqrt(d)

    g = GOLD["pairwise"]
    dims, npoints = g["dims"], g["npoints"]
    X1 = np.arange(npoints * dims, dtype=dtype).reshape(npoints, dims)
    X2 = X1 + 5
    out = check(env, func, (X1.shape[0], X2.shape[0]), DEFAULT_LOCAL_SIZE,
                [X1, X2, np.zeros((npoints, npoints), dtype)], exact=False,
                rtol=g["rtol"])
    from scipy.spatial.distance import cdist
    np.testing.assert_allclose(out[2], cdist(X1, X2), rtol=1e-6)


def test_pairwise_compiled_body_equals_handwritten_twin(env):
    """The translated body and the hand-written twins give the same bits."""
    hip, sim = env

    def func(X1, X2, D):
        i = get_global_id(0)
        j = get_global_id(1)
        X1_cols = X1.shape[1]
        d = 0.0
        for k in range(X1_cols):
            tmp = X1[i, k] - X2[j, k]
            d += tmp * tmp
        D[i, j] = np.sqrt(d)

    rng = np.random.default_rng(5)
    X1, X2 = rng.uniform(0, 1, (130, 3)), rng.uniform(0, 1, (514, 3))
    outs = []
    for kw in ({}, {"twin": "nmk_twin_pairwise_{dtype}"}):
        dev = [hip.asarray(X1), hip.asarray(X2), hip.asarray(np.zeros((130, 514)))]
        K.kernel(func, **kw)[(130, 514), DEFAULT_LOCAL_SIZE](*dev)
        outs.append(dev[2].asnumpy())
    np.testing.assert_allclose(outs[0], outs[1], rtol=1e-15)


# ---- the translator's own rules --------------------------------------------

def test_literal_typing_and_promotion(env):
    """int32 array op literal -> int64, float32 op float literal -> float64,
    int / int -> float64 (linalg_builder.py:261-291).  NumPy scalars follow
    other rules (int32 * 100000 stays int32), so the simulator is no oracle
    here; the expected values are written out."""
    def func(a, f, oi, of, od):
        i = get_global_id(0)
        x = a[i] * 100000          # int64: no 32-bit wrap
        oi[i] = x * 1000
        y = f[i] + 0.1             # float64
        of[i] = y
        od[i] = a[i] / 3           # true division in float64

    a = np.array([3, -7, 123456, 2 ** 31 - 1], np.int32)
    f = np.array([1.1, 2.2, -3.3, 1e-3], np.float32)
    out = check(env, func, a.shape, DEFAULT_LOCAL_SIZE,
                [a, f, np.zeros(4, np.int64), np.zeros(4, np.float64),
                 np.zeros(4, np.float64)], simulate=False)
    np.testing.assert_array_equal(out[2], a.astype(np.int64) * 10 ** 8)
    np.testing.assert_array_equal(out[3], f.astype(np.float64) + 0.1)
    np.testing.assert_array_equal(out[4], a.astype(np.float64) / 3)


def test_control_flow(env):
    def func(a, out):
        i = get_global_id(0)
        n = a[i]
        steps = 0
        while n != 1:                       # Collatz steps
            if n % 2 == 0:
                n = n // 2
            else:
                n = 3 * n + 1
            steps += 1
            if steps >= 1000:
                break
        total = 0
        for j in range(10, 0, -3):
            if j == 4:
                continue
            total += j
        out[i, 0] = steps
        out[i, 1] = total
        out[i, 2] = 1 if (n == 1 and not steps > 999) else 0
        out[i, 3] = max(steps, 5, i) + min(i, 3) + abs(-i)

    a = np.array([1, 2, 3, 6, 7, 27, 97, 871], np.int64)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, np.zeros((8, 4), np.int64)])


def test_negative_indices_and_slices(env):
    def func(a, out):
        i = get_global_id(0)
        n = a.shape[0]
        out[i, 0] = a[-1 - i]               # wraps from the end
        out[i, 1] = a[i - n]
        tail = a[2:]
        out[i, 2] = tail[-1] + tail.shape[0]
        rev = a[::-1]
        out[i, 3] = rev[i]
        col = out[:, 4]                     # integer index after a slice
        col[i] = len(a) + i

    a = np.arange(10, 20, dtype=np.int64)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, np.zeros((10, 5), np.int64)])


def test_device_functions_and_tuples(env):
    @kernel_func
    def hypot2(x, y):
        return x * x + y * y

    def clamp(v, lo, hi):
        if v < lo:
            return lo
        if v > hi:
            return hi
        return v

    def func(a, b, out):
        i = get_global_id(0)
        p, q = a[i], b[i]
        p, q = q, p                         # swap through a tuple
        out[i, 0] = hypot2(p, q)
        out[i, 1] = clamp(p - q, -1.5, 1.5)
        out[i, 2] = math.atan2(p, q) + math.floor(p) + float(np.float32(2) ** 3)
        idx = (i, 3)
        out[idx] = math.pi if p > q else -math.e

    a = np.array([0.5, -2.0, 3.25, 4.0], np.float64)
    b = np.array([1.5, 2.5, -3.0, 4.0], np.float64)
    check(env, func, a.shape, DEFAULT_LOCAL_SIZE, [a, b, np.zeros((4, 4))],
          exact=False, rtol=1e-12)


def test_tuple_elements_are_values(env):
    def func(out):
        i = get_global_id(0)
        pair = (i, i * 2)
        i = i + 100                         # must not show through the tuple
        if pair[1] > 6:
            pair = (pair[0], -pair[1])
        out[pair[0]] = pair[1] + i

    check(env, func, 8, DEFAULT_LOCAL_SIZE, [np.zeros(8, np.int64)])


def test_and_or_need_booleans(env):
    hip, sim = env

    def func(a, out):
        i = get_global_id(0)
        out[i] = a[i] or 7                  # Python would store a[i] or 7

    with pytest.raises(K.KernelCompileError, match="boolean values only"):
        K.kernel(func)[4, DEFAULT_LOCAL_SIZE](hip.asarray(np.arange(4)),
                                              hip.asarray(np.zeros(4, np.int64)))


def test_strided_and_transposed_arguments(env):
    hip, sim = env

    def func(a, b):
        i = get_global_id(0)
        j = get_global_id(1)
        b[j, i] = a[i, j] * 2

    base = np.arange(6 * 8, dtype=np.float32).reshape(6, 8)
    d_base = hip.asarray(base)
    d_out = hip.asarray(np.zeros((4, 3), np.float32))
    view = d_base[::2, 1:8:2]               # 3 x 4, strides (16, 2)
    K.kernel(func)[view.shape, DEFAULT_LOCAL_SIZE](view, d_out)
    np.testing.assert_array_equal(d_out.asnumpy(), (base[::2, 1:8:2] * 2).T)


def test_bounds_check_reports_instead_of_faulting(env):
    hip, sim = env

    def func(a, b):
        i = get_global_id(0)
        b[i] = a[i + 1]                     # one past the end for the last item

    a, b = hip.asarray(np.arange(8.0)), hip.asarray(np.zeros(8))
    with pytest.raises(IndexError, match="out of bounds"):
        K.kernel(func, boundscheck=True)[8, DEFAULT_LOCAL_SIZE](a, b)
    # the stray read was redirected to element 0; the flag is clear again
    np.testing.assert_array_equal(b.asnumpy(), [1, 2, 3, 4, 5, 6, 7, 0])
    K.kernel(func, boundscheck=True)[7, DEFAULT_LOCAL_SIZE](a, b)


def test_specialisation_per_signature(env):
    hip, sim = env

    def func(a, b):
        i = get_global_id(0)
        b[i] = a[i] / 2

    kern = K.kernel(func)
    names = set()
    for dtype in (np.int32, np.float32, np.float64):
        a = hip.asarray(np.arange(5, dtype=dtype))
        b = hip.asarray(np.zeros(5, np.float64))
        launch = kern[5, DEFAULT_LOCAL_SIZE]
        launch(a, b)
        names.add(launch.last_launch["kernel"])
        np.testing.assert_array_equal(b.asnumpy(), np.arange(5) / 2)
    assert len(names) == 3


def test_large_1d_launch_ids_do_not_wrap(env):               # 2268-2283
    hip, sim = env

    def func(a, b):
        i = get_global_id(0)
        if i == b:
            a[0] = b

    arr = hip.asarray(np.zeros(1, np.float32))
    b = 2 ** 31 + 10
    K.kernel(func)[2 ** 31 + 11, 1024](arr, b)
    assert arr.asnumpy()[0] == np.float32(b)
    # a dimension of a launch holds 2^32 - 1 work-items: more is an error, not a wrap
    with pytest.raises(ValueError, match="4294967295 work-items"):
        K.kernel(func)[2 ** 32 + 5, 1024](arr, b)


def test_more_rows_of_blocks_than_a_launch_has_along_y(env):
    """A 2-d launch whose second dimension needs more than 65535 blocks: the
    blocks go on along z."""
    hip, sim = env

    def func(a, out):
        i = get_global_id(0)
        j = get_global_id(1)
        out[j, i] = a[j, i] * 2.0 + i

    n = 9_000_000
    a = np.random.default_rng(1).standard_normal((n, 3)).astype(np.float32)
    d_out = hip.asarray(np.zeros((n, 3), np.float32))
    K.kernel(func)[(3, n), ()](hip.asarray(a), d_out)
    assert np.array_equal(d_out.asnumpy(), a * np.float32(2.0) + np.arange(3, dtype=np.float32))
    d_out = hip.asarray(np.zeros((n, 3), np.float32))
    K.kernel(func)[(3, n), (1, 64)](hip.asarray(a), d_out)
    assert np.array_equal(d_out.asnumpy(), a * np.float32(2.0) + np.arange(3, dtype=np.float32))


def _all_kinds_f32(rng, n):
    """float32 values of every kind: random bit patterns (all exponents, both
    signs, denormals, NaNs), a band around 1 and the special values."""
    bits = rng.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32)
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 1e-45, 1e-38,
                        1.17549435e-38, 3.4028235e38, 2.0 ** -120, 2.0 ** 120,
                        np.nextafter(np.float32(2.0 ** -120), np.float32(0)),
                        np.nextafter(np.float32(2.0 ** 120), np.float32(0))], np.float32)
    return np.concatenate([bits.view(np.float32),
                           rng.uniform(0.5, 2.0, n).astype(np.float32), special])


@pytest.mark.parametrize("op", ["log", "exp"])
def test_float32_log_and_exp_equal_the_device_library_bit_for_bit(env, op):
    """Generated kernels evaluate float32 log / exp with the library's own
    arithmetic and leave its range handling to the arguments that need it:
    the results must be the library's on every input."""
    hip = env[0]
    rng = np.random.default_rng(17)
    if op == "log":
        x = _all_kinds_f32(rng, 1 << 20)
    else:
        x = np.concatenate([rng.uniform(-110, 100, 1 << 20).astype(np.float32),
                            rng.uniform(-1, 1, 1 << 18).astype(np.float32),
                            np.array([80.0, -80.0, np.nextafter(np.float32(80), np.float32(90)),
                                      88.7, 88.8, -87.3, -87.4, -103.9, -104.0, 0.0, -0.0,
                                      np.inf, -np.inf, np.nan], np.float32)])
    f = getattr(np, op)

    def func(a, b):
        i = get_global_id(0)
        b[i] = f(a[i])

    dx = hip.asarray(x)
    got, ref = hip.asarray(np.zeros_like(x)), hip.asarray(np.zeros_like(x))
    K.kernel(func)[x.shape, ()](dx, got)
    K.kernel(func, twin="nmk_twin_unary_" + op + "_{dtype}")[x.shape, ()](dx, ref)
    g, r = got.asnumpy(), ref.asnumpy()
    same = (g.view(np.uint32) == r.view(np.uint32)) | (np.isnan(g) & np.isnan(r))
    assert same.all(), (x[~same][:5], g[~same][:5], r[~same][:5])
    # and the library agrees with NumPy to float32 accuracy where finite
    with np.errstate(all="ignore"):
        want = f(x.astype(np.float64))
    ok = np.isfinite(want) & (np.abs(want) > 1e-30) & (np.abs(want) < 1e30)
    np.testing.assert_allclose(g[ok], want[ok], rtol=3e-7)


def test_float64_erf_within_two_ulp(env):
    """erf of a double in generated kernels: piecewise Taylor polynomials from
    a table in workgroup memory.  Against mpmath the error must stay within 2
    units in the last place; signs, NaN, infinities and the saturation to
    +-1 must be right."""
    from scipy.special import erf as scipy_erf
    hip = env[0]
    rng = np.random.default_rng(18)
    x = np.concatenate([rng.uniform(-6.5, 6.5, 1 << 20), rng.uniform(-0.25, 0.25, 1 << 18),
                        10.0 ** rng.uniform(-300, 1, 1 << 12),
                        (np.arange(-97, 98) + 0.5) / 16.0, np.arange(-97, 98) / 16.0,
                        [0.0, -0.0, 3 / 32, np.nextafter(3 / 32, 0), 5e-324, 1e-310, 6.0,
                         -6.0, 7.0, 30.0, -30.0, np.inf, -np.inf, np.nan]])

    def func(a, b):
        i = get_global_id(0)
        b[i] = math.erf(a[i])

    dx = hip.asarray(x)
    got, ref = hip.asarray(np.zeros_like(x)), hip.asarray(np.zeros_like(x))
    K.kernel(func)[x.shape, (64,)](dx, got)
    K.kernel(func, twin="nmk_twin_unary_erf_{dtype}")[x.shape, ()](dx, ref)
    g, r = got.asnumpy(), ref.asnumpy()
    assert np.array_equal(np.isnan(g), np.isnan(x))
    assert np.array_equal(np.signbit(g), np.signbit(x) & ~np.isnan(x)) or \
        np.array_equal(np.signbit(g[~np.isnan(x)]), np.signbit(x[~np.isnan(x)]))
    fin = ~np.isnan(x)
    want = scipy_erf(x[fin])
    # SciPy's own routine is off by up to 2 units in the last place: a loose
    # bound on everything, the exact one on a sample with mpmath
    ulps = np.abs(g[fin] - want) / np.spacing(np.abs(want))
    assert ulps.max() <= 4, (x[fin][ulps.argmax()], ulps.max())
    import mpmath
    mpmath.mp.dps = 40
    pick = np.concatenate([rng.choice(np.flatnonzero(fin), 20000, replace=False),
                           np.argsort(-ulps)[:200]])
    worst = worst_lib = 0.0
    for xi, gi, ri in zip(x[fin][pick].tolist(), g[fin][pick].tolist(),
                          r[fin][pick].tolist()):
        exact = mpmath.erf(mpmath.mpf(xi))
        if exact == 0 or abs(xi) == np.inf:
            assert gi == float(exact)
            continue
        ulp = float(np.spacing(abs(float(exact))))
        worst = max(worst, abs(float((mpmath.mpf(gi) - exact) / ulp)))
        worst_lib = max(worst_lib, abs(float((mpmath.mpf(ri) - exact) / ulp)))
    print("erf max error in ulp: generated", worst, "device library", worst_lib)
    assert worst <= 2.0, worst
    big = np.abs(x) >= 6
    np.testing.assert_array_equal(g[big & fin], np.sign(x[big & fin]))
    # a second local size, with partial groups: the table load is per group
    K.kernel(func)[x.shape, (256,)](dx, got)
    np.testing.assert_array_equal(got.asnumpy()[fin], g[fin])
