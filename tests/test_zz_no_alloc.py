"""GPU parity of mkl_gemm_float32_device_noalloc, the gemm entry point that
allocates no device memory, against mkl_gemm_float32_device through the raw
C-ABI: two calls in a row on one GPU, the second on a smaller problem, so the
fixed workspace still holds the first call's partial products."""

import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


class Memref2F32(ctypes.Structure):
    """Memref<2, float> (numba_mlir/numba_mlir/math_runtime/include/Common.hpp:17-28)."""
    _fields_ = [("userData", ctypes.c_void_p), ("data", ctypes.c_void_p),
                ("offset", ctypes.c_size_t), ("dims", ctypes.c_size_t * 2),
                ("strides", ctypes.c_size_t * 2)]


def _memref(arr):
    ref = Memref2F32()
    ref.userData = None
    ref.data = arr.ptr
    ref.offset = 0
    ref.dims[0], ref.dims[1] = arr.shape
    ref.strides[0], ref.strides[1] = arr.elem_strides
    return ref


@pytest.fixture(scope="module")
def gemm_entry_points(hip):
    from numba_mlir_amd.mlir import math_runtime

    lib = math_runtime.runtime_hip_lib
    sig = [ctypes.c_void_p, ctypes.POINTER(Memref2F32), ctypes.POINTER(Memref2F32),
           ctypes.c_float, ctypes.c_float, ctypes.POINTER(Memref2F32)]
    lib.mkl_gemm_float32_device.argtypes = sig
    lib.mkl_gemm_float32_device.restype = None
    lib.mkl_gemm_float32_device_noalloc.argtypes = sig
    lib.mkl_gemm_float32_device_noalloc.restype = ctypes.c_int
    return hip, lib, math_runtime


def _both(hip, lib, mrt, m, n, k, alpha, beta, seed):
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((m, k), dtype=np.float32)
    b = rng.standard_normal((k, n), dtype=np.float32)
    c0 = rng.standard_normal((m, n), dtype=np.float32)
    d_a, d_b = hip.asarray(a), hip.asarray(b)
    queue = d_a.ctx.queue
    ra, rb = _memref(d_a), _memref(d_b)

    d_ref = hip.asarray(c0)
    rc = _memref(d_ref)
    lib.mkl_gemm_float32_device(queue, ra, rb, alpha, beta, rc)
    ref_kernel = mrt.last_kernel()

    d_got = hip.asarray(c0)
    rc = _memref(d_got)
    status = lib.mkl_gemm_float32_device_noalloc(queue, ra, rb, alpha, beta, rc)
    return status, d_got.asnumpy(), d_ref.asnumpy(), ref_kernel, mrt.last_kernel(), (a, b, c0)


def test_two_calls_in_a_row_match_the_allocating_entry_point(gemm_entry_points):
    hip, lib, mrt = gemm_entry_points
    # 1024^3 cuts K into four slices (16 MiB of workspace), 640 x 516 x 1028
    # is ragged and cuts it into eight (10 MiB), 4096 x 3072 x 64 does not split
    for m, n, k, alpha, beta in ((1024, 1024, 1024, 1.0, 0.0),
                                 (640, 516, 1028, 1.5, -0.5),
                                 (256, 384, 2048, 0.5, 2.0),
                                 (4096, 3072, 64, 1.0, 0.0)):
        status, got, ref, k_ref, k_got, (a, b, c0) = _both(
            hip, lib, mrt, m, n, k, alpha, beta, seed=m + n + k)
        assert status == 0
        assert ("_splitk" in k_got) == (k > 64)
        # The allocating entry point may share K out differently (even shares
        # of the slabs need a larger workspace than the fixed one): the same
        # kernel gives the same bits, another one the same product to
        # float32's accuracy.
        assert k_got == k_ref or "_even" in k_ref, (k_got, k_ref)
        if k_got == k_ref:
            assert np.array_equal(got, ref), (m, n, k)
        truth = beta * c0.astype(np.float64) + alpha * (
            a.astype(np.float64) @ b.astype(np.float64))
        scale = abs(beta) * np.abs(c0) + abs(alpha) * (
            np.abs(a).astype(np.float64) @ np.abs(b))
        assert (np.abs(got - truth) <= 1e-4 * scale + 1e-30).all()
        assert (np.abs(got - ref) <= 1e-4 * scale + 1e-30).all()


def test_operands_off_the_word_grid_stay_on_tiles_and_edges(gemm_entry_points):
    """The allocating entry point repacks an operand whose rows do not end on
    a 128-bit word into its workspace; this one cannot, and runs the whole
    tiles on the matrix cores and the rest on the strided kernel."""
    hip, lib, mrt = gemm_entry_points
    m, n, k = 1540, 2052, 1001
    rng = np.random.default_rng(5)
    a_wide = rng.standard_normal((m, k + 3), dtype=np.float32)
    b = rng.standard_normal((k, n), dtype=np.float32)
    d_a, d_b = hip.asarray(a_wide)[:, :k], hip.asarray(b)
    outs = []
    for entry in (lib.mkl_gemm_float32_device, lib.mkl_gemm_float32_device_noalloc):
        d_c = hip.asarray(np.zeros((m, n), np.float32))
        status = entry(d_a.ctx.queue, _memref(d_a), _memref(d_b), 1.0, 0.0, _memref(d_c))
        assert not status
        outs.append((mrt.last_kernel(), d_c.asnumpy()))
    assert outs[0][0].endswith("+packed") and outs[1][0] == "sgemm_mfma_128x128+edges"
    a = a_wide[:, :k]
    truth = a.astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(a).astype(np.float64) @ np.abs(b)
    for _, got in outs:
        assert (np.abs(got - truth) <= 1e-4 * scale + 1e-30).all()


def test_a_thin_product_keeps_its_partial_sums_in_the_fixed_array(gemm_entry_points):
    """A few rows times a long matrix cuts K into slices whose partial sums
    go through the workspace: both entry points cut alike and give the same
    bits, the second call on a smaller problem."""
    hip, lib, mrt = gemm_entry_points
    for m, n, k in ((4, 4096, 4096), (2, 1100, 2048)):
        status, got, ref, k_ref, k_got, (a, b, c0) = _both(
            hip, lib, mrt, m, n, k, 1.5, -0.5, seed=m + n + k)
        assert status == 0
        assert k_got == k_ref == "sgemm_thin_cols"
        assert np.array_equal(got, ref), (m, n, k)
        truth = -0.5 * c0.astype(np.float64) + 1.5 * (
            a.astype(np.float64) @ b.astype(np.float64))
        scale = 0.5 * np.abs(c0) + 1.5 * (np.abs(a).astype(np.float64) @ np.abs(b))
        assert (np.abs(got - truth) <= 1e-5 * scale + 1e-30).all()


def test_the_entry_point_allocates_no_device_memory(gemm_entry_points):
    """Free device memory, read with hipMemGetInfo, is the same before and
    after calls on split-K shapes this process has not run before (a route
    through the heap workspace would take at least 8 MiB for the first of
    them and more for the second)."""
    hip, lib, mrt = gemm_entry_points
    hiprt = ctypes.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hiprt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    rng = np.random.default_rng(3)
    cases = []
    for m, n, k in ((896, 1152, 1536), (1280, 768, 4096), (8, 2048, 8192)):
        a = hip.asarray(rng.standard_normal((m, k), dtype=np.float32))
        b = hip.asarray(rng.standard_normal((k, n), dtype=np.float32))
        c = hip.asarray(np.zeros((m, n), np.float32))
        cases.append((a, b, c))
    mrt.runtime_hip_lib.nmrtMathRuntimeFinalize()    # the heap workspace, if any, goes
    before = free_bytes()
    for a, b, c in cases:
        status = lib.mkl_gemm_float32_device_noalloc(
            a.ctx.queue, _memref(a), _memref(b), 1.0, 0.0, _memref(c))
        assert status == 0
        assert "_splitk" in mrt.last_kernel() or mrt.last_kernel() == "sgemm_thin_cols"
        assert free_bytes() == before, mrt.last_kernel()
    # (and the allocating entry point does take its workspace from the heap)
    a, b, c = cases[1]
    lib.mkl_gemm_float32_device(a.ctx.queue, _memref(a), _memref(b), 1.0, 0.0, _memref(c))
    assert free_bytes() < before
