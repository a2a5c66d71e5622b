"""GPU parity: kernel builtins (atomics, barriers, local/private arrays, group
reductions, operators) as hand-written twins against the kernel simulator;
bodies, inputs and tolerances are the reference's own tests
(numba_mlir/numba_mlir/mlir/tests/test_gpu.py, line ranges per test)."""

import numpy as np
import pytest

from numba_mlir_amd import kernel as K

pytestmark = pytest.mark.gpu

get_global_id = K.get_global_id
barrier, mem_fence = K.barrier, K.mem_fence
LOCAL_MEM_FENCE, GLOBAL_MEM_FENCE = K.LOCAL_MEM_FENCE, K.GLOBAL_MEM_FENCE
DEFAULT_LOCAL_SIZE = K.DEFAULT_LOCAL_SIZE

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
TAGS = {np.dtype(np.int32): "i32", np.dtype(np.int64): "i64",
        np.dtype(np.float32): "f32", np.dtype(np.float64): "f64"}


@pytest.fixture(scope="module")
def env(hip):
    from oracle.kernel_sim import kernel_sim
    return hip, lambda f: kernel_sim(f, STUBS)


def _run(hip, func, twin, gsize, lsize, host_args, **kw):
    """Launches the twin on device copies of the arrays; returns them as NumPy."""
    dev = [hip.asarray(a) if isinstance(a, np.ndarray) else a for a in host_args]
    K.kernel(func, twin=twin, **kw)[gsize, lsize](*dev)
    return [d.asnumpy() if isinstance(a, np.ndarray) else a
            for d, a in zip(dev, host_args)]


def test_simple1(env):                                       # 176-201
    hip, sim = env

    def func(a, b, c):
        i = get_global_id(0)
        j = get_global_id(1)
        k = get_global_id(2)
        c[i, j, k] = a[i, j, k] + b[i, j, k]

    a = np.array([[[1, 2, 3], [4, 5, 6]]], np.float32)
    b = np.array([[[7, 8, 9], [10, 11, 12]]], np.float32)
    sim_res = np.zeros(a.shape, a.dtype)
    sim(func)[a.shape, DEFAULT_LOCAL_SIZE](a, b, sim_res)
    out = _run(hip, func, "nmk_twin_add3_f32", a.shape, DEFAULT_LOCAL_SIZE,
               [a, b, np.zeros(a.shape, a.dtype)])
    np.testing.assert_array_equal(out[2], sim_res)


def test_simple3(env):                                       # 234-259
    hip, sim = env

    def func(a, b):
        i = get_global_id(0)
        b[i, 0] = a[i, 0]
        b[i, 1] = a[i, 1]

    a = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    sim_res = np.zeros(a.shape, a.dtype)
    sim(func)[a.shape[0], DEFAULT_LOCAL_SIZE](a, sim_res)
    out = _run(hip, func, "nmk_twin_copy_cols2_f32", a.shape[0],
               DEFAULT_LOCAL_SIZE, [a, np.zeros(a.shape, a.dtype)])
    np.testing.assert_array_equal(out[1], sim_res)


def test_fastmath_off_keeps_two_roundings(env):              # 980-1008
    hip, sim = env

    def func(a, b, c, res):
        i = get_global_id(0)
        res[i] = a[i] * b[i] + c[i]

    # the reference's values, plus values where fma and mul+add differ
    for a, b, c in (
        (np.array([1, 2, 3, 4], np.float32), np.array([5, 6, 7, 8], np.float32),
         np.array([9, 10, 11, 12], np.float32)),
        (np.array([1.0000001, 3.3333333, 1e-3, 7.7], np.float32),
         np.array([1.0000001, 3.0000001, 1e3, 1.3], np.float32),
         np.array([-1.0000002, -10.0, -1.0, -10.01], np.float32)),
    ):
        sim_res = np.zeros(a.shape, a.dtype)
        sim(func)[a.shape, DEFAULT_LOCAL_SIZE](a, b, c, sim_res)
        out = _run(hip, func, "nmk_twin_mul_add_f32", a.shape, DEFAULT_LOCAL_SIZE,
                   [a, b, c, np.zeros(a.shape, a.dtype)])
        assert out[3].tobytes() == sim_res.tobytes()


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32])
@pytest.mark.parametrize("opname", ["add", "sub"])
@pytest.mark.parametrize("mode,ret_size", [(0, 1), (1, 2)])
def test_atomics(env, dtype, opname, mode, ret_size):        # 820-866
    hip, sim = env
    atomic_op = getattr(K.atomic, opname)

    if mode == 0:
        def func(a, b):
            i = get_global_id(0)
            atomic_op(b, 0, a[i])
    else:
        def func(a, b):
            i = get_global_id(0)
            atomic_op(b, i % 2, a[i])

    a = np.array([1, 2, 3, 4, 5, 6, 7, 8, 9], dtype)
    sim_res = np.zeros([ret_size], dtype)
    sim(func)[a.shape, DEFAULT_LOCAL_SIZE](a, sim_res)
    twin = f"nmk_twin_atomic_{opname}_m{mode}_" + "{dtype}"
    out = _run(hip, func, twin, a.shape, DEFAULT_LOCAL_SIZE,
               [a, np.zeros([ret_size], dtype)])
    np.testing.assert_array_equal(out[1], sim_res)


@pytest.mark.parametrize("opname", ["add", "sub"])
@pytest.mark.parametrize("mode", [2, 3])
def test_atomics_different_types(env, opname, mode):         # 868-890
    hip, sim = env
    atomic_op = getattr(K.atomic, opname)

    if mode == 2:
        def func(a, b):
            i = get_global_id(0)
            atomic_op(b, 0, a[i] + 1)
    else:
        def func(a, b):
            i = get_global_id(0)
            atomic_op(b, 0, 1)

    a = np.array([1, 2, 3, 4, 5, 6, 7, 8, 9], np.int32)
    sim_res = np.zeros([1], np.int32)
    sim(func)[a.shape, DEFAULT_LOCAL_SIZE](a, sim_res)
    out = _run(hip, func, f"nmk_twin_atomic_{opname}_m{mode}_i32", a.shape,
               DEFAULT_LOCAL_SIZE, [a, np.zeros([1], np.int32)])
    np.testing.assert_array_equal(out[1], sim_res)


@pytest.mark.parametrize("funci", [1, 2])
def test_atomics_multidim(env, funci):                       # 892-925
    hip, sim = env
    atomic_op = K.atomic.add

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
    sim_res = np.zeros((2, 2), np.int32)
    sim(func)[a.shape, DEFAULT_LOCAL_SIZE](a, sim_res)
    out = _run(hip, func, f"nmk_twin_atomic_multidim{funci}_i32", a.shape,
               DEFAULT_LOCAL_SIZE, [a, np.zeros((2, 2), np.int32)])
    np.testing.assert_array_equal(out[1], sim_res)


def test_atomics_different_dims(env):                        # 927-955
    hip, sim = env
    atomic_op = K.atomic.add

    def func(a, b, c):
        i = get_global_id(0)
        j = get_global_id(1)
        atomic_op(a, (i, j), c[i, j])
        atomic_op(b, (i), c[i, j])

    c = np.array([[1, 2, 3], [4, 5, 6]], np.int32)
    a_sim, b_sim = np.zeros(c.shape, np.int32), np.zeros(c.shape[0], np.int32)
    sim(func)[c.shape, DEFAULT_LOCAL_SIZE](a_sim, b_sim, c)
    out = _run(hip, func, "nmk_twin_atomic_dims_i32", c.shape, DEFAULT_LOCAL_SIZE,
               [np.zeros(c.shape, np.int32), np.zeros(c.shape[0], np.int32), c])
    np.testing.assert_array_equal(out[0], a_sim)
    np.testing.assert_array_equal(out[1], b_sim)


@pytest.mark.parametrize("is_barrier", [1, 0])
@pytest.mark.parametrize("flags", [LOCAL_MEM_FENCE, GLOBAL_MEM_FENCE])
@pytest.mark.parametrize("global_size", [1, 2, 27, 67, 101])
@pytest.mark.parametrize("local_size", [1, 2, 7, 17, 33])
def test_barrier_ops(env, is_barrier, flags, global_size, local_size):  # 1074-1102
    hip, sim = env
    op = barrier if is_barrier else mem_fence

    def func(a, b):
        i = get_global_id(0)
        v = a[i]
        op(flags)
        b[i] = a[i]

    a = np.arange(global_size, dtype=np.int64)
    sim_res = np.zeros(global_size, a.dtype)
    sim(func)[global_size, local_size](a, sim_res)

    def twin_func(a, b, is_barrier, flags):
        pass

    dev = [hip.asarray(a), hip.asarray(np.zeros(global_size, np.int64))]
    K.kernel(twin_func, twin="nmk_twin_barrier_ops_i64")[global_size, local_size](
        dev[0], dev[1], is_barrier, flags)
    np.testing.assert_array_equal(dev[1].asnumpy(), sim_res)


@pytest.mark.parametrize("global_size", [1, 2, 4, 27, 67, 101])
@pytest.mark.parametrize("local_size", [1, 2, 7, 17, 33])
def test_barrier1(env, global_size, local_size):             # 1105-1133
    hip, sim = env
    atomic_add = K.atomic.add

    def func(a, b):
        i = get_global_id(0)
        off = i // local_size
        atomic_add(a, off, i)
        barrier(GLOBAL_MEM_FENCE)
        b[i] = a[off]

    count = (global_size + local_size - 1) // local_size
    a = np.array([0] * count, np.int64)
    sim_res = np.zeros(global_size, a.dtype)
    sim(func)[global_size, local_size](a.copy(), sim_res)

    dev = [hip.asarray(a.copy()), hip.asarray(np.zeros(global_size, np.int64))]
    K.kernel(func, twin="nmk_twin_barrier1_i64")[global_size, local_size](
        dev[0], dev[1], local_size)
    np.testing.assert_array_equal(dev[1].asnumpy(), sim_res)


@pytest.mark.parametrize("blocksize", [1, 10, 17, 64, 67, 101])
@pytest.mark.parametrize("two_d", [False, True])
def test_local_memory(env, blocksize, two_d):                # 1136-1198
    hip, sim = env
    local_array = K.local.array

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

    arr = np.arange(blocksize).astype(np.float32)
    sim_res = arr.copy()
    sim(func)[blocksize, blocksize](sim_res)

    dev = hip.asarray(arr.copy())
    K.kernel(func, twin="nmk_twin_local_memory_f32",
             local_bytes=[blocksize * 4])[blocksize, blocksize](dev, blocksize)
    np.testing.assert_allclose(dev.asnumpy(), sim_res)


@pytest.mark.parametrize("blocksize", [1, 10, 17, 64, 67, 101])
@pytest.mark.parametrize("variant,priv_size", [(1, 1), (3, 1), (3, 11), (3, 27), (4, 100)])
def test_private_memory(env, blocksize, variant, priv_size):  # 1202-1326
    hip, sim = env
    private_array = K.private.array

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

    arr = np.zeros(blocksize).astype(np.float32)
    sim_res = arr.copy()
    sim(func)[blocksize, blocksize](sim_res)
    dev = hip.asarray(arr.copy())
    K.kernel(func, twin="nmk_twin_private_memory_f32")[blocksize, blocksize](
        dev, variant, priv_size)
    np.testing.assert_allclose(dev.asnumpy(), sim_res)


@pytest.mark.parametrize("opname", ["add", "mul", "min", "max"])
@pytest.mark.parametrize("global_size", [1, 2, 4, 27, 67, 101, 1000])
@pytest.mark.parametrize("local_size", [1, 2, 7, 17, 33, 64, 200, 256])
@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.float32])
def test_group_func(env, opname, global_size, local_size, dtype):  # 1360-1393
    hip, sim = env
    if global_size > 25 and opname == "mul":
        pytest.skip("products overflow (the reference skips them too)")
    group_op = getattr(K.group, "reduce_" + opname)

    def func(a, b):
        i = get_global_id(0)
        v = group_op(a[i])
        b[i] = v

    a = np.arange(global_size, dtype=dtype)
    out = _run(hip, func, f"nmk_twin_group_reduce_{opname}_" + "{dtype}",
               (global_size,), (local_size,), [a, np.zeros(global_size, dtype)])
    if local_size <= 33:         # the reference's own sizes: against the simulator
        sim_res = np.zeros(global_size, a.dtype)
        sim(func)[(global_size,), (local_size,)](a, sim_res)
        np.testing.assert_allclose(out[1], sim_res, rtol=1e-5)
    # every size: closed form per work-group (the simulator nests one
    # greenlet per work-item and runs out of stack beyond ~100 items)
    fold = {"add": np.sum, "mul": np.prod, "min": np.min, "max": np.max}[opname]
    expect = np.empty(global_size, dtype)
    for start in range(0, global_size, local_size):
        stop = min(start + local_size, global_size)
        expect[start:stop] = fold(a[start:stop].astype(np.float64 if dtype == np.float32 else dtype))
    np.testing.assert_allclose(out[1], expect, rtol=1e-5)


_OPS = {"+": "add", "-": "sub", "*": "mul", "/": "truediv", "//": "floordiv",
        "%": "mod", "**": "pow"}


@pytest.mark.parametrize("op", sorted(_OPS))
@pytest.mark.parametrize("dtype", [np.int32, np.float32, np.float64])
def test_gpu_ops_binary(env, op, dtype):                     # 551-566, 503-521
    hip, sim = env
    f = eval(f"lambda a, b: a {op} b")

    def func(a, b, c):
        i = get_global_id(0)
        c[i] = f(a[i], b[i])

    a = np.array([11, 12, 13, 14, 15], dtype)
    b = np.array([1, 2, 3, 4, 5], dtype)
    sim_res = np.zeros(a.shape, dtype)
    sim(func)[a.shape, DEFAULT_LOCAL_SIZE](a, b, sim_res)
    out = _run(hip, func, f"nmk_twin_binary_{_OPS[op]}_" + "{dtype}", a.shape,
               DEFAULT_LOCAL_SIZE, [a, b, np.zeros(a.shape, dtype)])
    np.testing.assert_allclose(out[2], sim_res, rtol=1e-5)
    # signs: Python's floor/mod conventions
    a2 = np.array([-11, 12, -13, 14, -15], dtype)
    b2 = np.array([3, -5, -4, 3, 7], dtype)
    if op in ("//", "%", "-", "*"):
        sim_res = np.zeros(a.shape, dtype)
        sim(func)[a.shape, DEFAULT_LOCAL_SIZE](a2, b2, sim_res)
        out = _run(hip, func, f"nmk_twin_binary_{_OPS[op]}_" + "{dtype}", a.shape,
                   DEFAULT_LOCAL_SIZE, [a2, b2, np.zeros(a.shape, dtype)])
        np.testing.assert_allclose(out[2], sim_res, rtol=1e-5)
