"""GPU tests of the HIP device array (the analogue of the reference's dpctl
USM arrays) and of njit-level bodies that mix allocation kinds."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env(hip):
    from numba_mlir_amd.mlir import ops
    return hip, ops


@pytest.mark.parametrize("usm_type", ["device", "shared", "host"])
@pytest.mark.parametrize("order", ["C", "F"])
def test_round_trip_and_interface(env, usm_type, order):
    hip, _ = env
    a = np.asarray(np.arange(24, dtype=np.float64).reshape(4, 6), order=order)
    d = hip.asarray(a, usm_type=usm_type)
    assert d.shape == a.shape and d.dtype == a.dtype and d.strides == a.strides
    assert d.usm_type == usm_type
    np.testing.assert_array_equal(d.asnumpy(), a)
    iface = d.__hip_array_interface__
    assert iface["data"] == (d.ptr, False) and iface["shape"] == a.shape
    assert iface["strides"] == (None if order == "C" else (1, 4))     # in elements
    assert iface["typestr"] == a.dtype.str
    from numba_mlir_amd.mlir import python_rt
    rec = python_rt.unbox(d)               # what compiled code would receive
    assert rec.data == d.ptr and rec.nitems == 24 and rec.itemsize == 8
    assert tuple(rec.shape) == a.shape and tuple(rec.strides) == a.strides
    assert iface["queue"] == hip.get_context().queue
    np.testing.assert_array_equal(d.T.asnumpy(), a.T)
    if usm_type != "device":
        view = d.as_host_view()            # host-dereferenceable, no copy
        np.testing.assert_array_equal(view, a)
        view[0, 0] = -5
        assert d.asnumpy()[0, 0] == -5
    else:
        with pytest.raises(ValueError):
            d.as_host_view()


def test_default_device_caps(env):
    hip, _ = env
    caps = hip.get_default_device()
    assert caps.has_fp64 and caps.arch == "gfx950" and caps.subgroup_size == 64
    assert caps.filter_string == hip.DEFAULT_DEVICE


def test_buffers_are_released(env):
    hip, _ = env
    import gc
    for _ in range(1500):                # 1500 x 256 MiB = 375 GiB > HBM: only fits if freed
        x = hip.empty((1 << 28,), np.uint8)   # released through gpuxDeAlloc
        del x
    gc.collect()


@pytest.mark.parametrize("size", [1, 13, 127, 1024])
def test_mixed_allocation_kinds(env, size):
    """c = a + b with a in device memory, b in shared memory, c in device
    memory (test_dpctl_simple1 / test_cfd_simple2, tests/test_gpu.py:1490-1520,
    1644-1670)."""
    hip, ops = env
    a = np.arange(size, dtype=np.float32)
    b = np.arange(size, dtype=np.float32) * 3
    d_a = hip.asarray(a, usm_type="device")
    d_b = hip.asarray(b, usm_type="shared")
    d_c = hip.asarray(np.zeros(size, np.float32), usm_type="device")
    ops.add(d_a, d_b, out=d_c)
    np.testing.assert_array_equal(d_c.asnumpy(), a + b)


def test_scalar_broadcast(env):
    """b[:] = a * 2 (test_cfd_simple1, tests/test_gpu.py:1616-1641)."""
    hip, ops = env
    a = np.arange(1024, dtype=np.float32)
    two = hip.asarray(np.array([2], np.float32))
    out = hip.asarray(np.zeros(1024, np.float32))
    ops.multiply(hip.asarray(a), two, out=out)
    np.testing.assert_array_equal(out.asnumpy(), a * 2)


def test_l2_norm(env):
    """test_l2_norm (tests/test_gpu.py:2198-2223): rtol 1e-5."""
    hip, ops = env
    src = np.arange(10 * 10, dtype=np.float32).reshape(10, 10)
    res = np.sqrt(np.square(src).sum(axis=1))
    got = ops.l2_norm_rows(hip.asarray(src)).asnumpy()
    np.testing.assert_allclose(got, res, rtol=1e-5)
    rng = np.random.default_rng(3)
    for shape in ((333, 1000), (64, 8192), (5, 3)):
        x = rng.standard_normal(shape, dtype=np.float32)
        got = ops.l2_norm_rows(hip.asarray(x)).asnumpy()
        truth = np.sqrt((x.astype(np.float64) ** 2).sum(axis=1))
        np.testing.assert_allclose(got, truth, rtol=1e-5)


@pytest.mark.parametrize("first", [1, 3, 5, 8, 13, 16])
def test_transfers_of_views_that_start_inside_a_word(env, first):
    """A contiguous view whose first byte is not on a 16-byte boundary (and
    whose last is not either) goes to the host and back in 128-bit words with
    single bytes only at its two ends; what lies around it is untouched."""
    hip = env[0]
    n = (36 << 20) + 11                  # three staging chunks
    rng = np.random.default_rng(first)
    host = rng.integers(0, 255, n, dtype=np.uint8)
    d = hip.asarray(host)
    view = d[first:n - 7]
    assert view.ptr % 16 == first % 16
    np.testing.assert_array_equal(view.asnumpy(), host[first:n - 7])
    fresh = rng.integers(0, 255, n - 7 - first, dtype=np.uint8)
    view.copy_from_host(fresh)
    expect = host.copy()
    expect[first:n - 7] = fresh
    np.testing.assert_array_equal(d.asnumpy(), expect)
    small = d[first:first + 5]           # shorter than the distance to a boundary
    np.testing.assert_array_equal(small.asnumpy(), expect[first:first + 5])
