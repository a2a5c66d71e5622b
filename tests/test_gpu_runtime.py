"""GPU tests of the raw gpux* C-ABI, driven the way compiled host code drives
it (reference call order: mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:228-857)."""

import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt(native_libs):
    from numba_mlir_amd.mlir import gpu_runtime
    return gpu_runtime.runtime_lib, gpu_runtime, native_libs


NO_DEPS = (ctypes.c_void_p * 1)(None)


def _alloc(lib, g, q, nbytes, kind):
    res = g.GPUAllocResult()
    lib.gpuxAlloc(q, nbytes, 64, kind, NO_DEPS, ctypes.byref(res))
    lib.gpuxWait(q, res.event)
    lib.gpuxDestroyEvent(q, res.event)
    return res.ptr


def _params(g, entries):
    descs = (g.GPUParamDesc * (len(entries) + 1))()
    keep = []
    for i, (val, ptype) in enumerate(entries):
        if val is None:
            descs[i].data, descs[i].size = None, ptype[1]
            descs[i].type = 8
            continue
        keep.append(val)
        descs[i].data = ctypes.cast(ctypes.pointer(val), ctypes.c_void_p)
        descs[i].size = ctypes.sizeof(val)
        descs[i].type = ptype
    descs[len(entries)].data = None
    descs[len(entries)].size = 0
    descs[len(entries)].type = 0
    return descs, keep


def _host_view(ptr, n, dtype):
    buf = (ctypes.c_uint8 * (n * np.dtype(dtype).itemsize)).from_address(ptr)
    return np.frombuffer(buf, dtype=dtype)


def test_full_call_sequence_on_shared_memory(rt):
    """queue -> module -> kernel -> suggest -> alloc(shared) -> launch -> wait
    -> destroy event; the result is read directly on the host, as compiled
    host code reads a reduction result from shared USM."""
    lib, g, low = rt
    q = lib.gpuxQueueCreate(b"level_zero:gpu:0")
    blob = low.kernel_blob("twins")
    mod = lib.gpuxModuleLoad(q, blob, len(blob))
    kern = lib.gpuxKernelGet(mod, b"nmk_twin_get_global_id_2")

    shape = (7, 13)
    gs = (ctypes.c_uint32 * 2)(*shape)
    bs = (ctypes.c_uint32 * 2)()
    lib.gpuxSuggestBlockSize(q, kern, gs, bs, 2)
    assert tuple(bs) == (7, 13)

    n = shape[0] * shape[1]
    ptr = _alloc(lib, g, q, n * 4, 1)              # Shared
    host = _host_view(ptr, n, np.int32)
    host[:] = -1
    descs, keep = _params(g, [
        (ctypes.c_void_p(ptr), 8), (ctypes.c_int64(7), 5), (ctypes.c_int64(13), 5),
        (ctypes.c_int64(13), 5), (ctypes.c_int64(1), 5),
        (ctypes.c_int64(7), 5), (ctypes.c_int64(13), 5), (ctypes.c_int64(1), 5)])
    ev = lib.gpuxLaunchKernel(q, kern, 1, 1, 1, bs[0], bs[1], 1, NO_DEPS, descs)
    lib.gpuxWait(q, ev)
    lib.gpuxDestroyEvent(q, ev)
    i, j = np.meshgrid(np.arange(7), np.arange(13), indexing="ij")
    assert np.array_equal(host.reshape(shape), i + 100 * j)

    lib.gpuxDeAlloc(q, ptr)
    lib.gpuxKernelDestroy(kern)
    lib.gpuxModuleDestroy(mod)
    lib.gpuxQueueDestroy(q)


def test_host_and_device_allocations(rt):
    lib, g, low = rt
    q = lib.gpuxQueueCreate(None)
    blob = low.kernel_blob("maps")
    mod = lib.gpuxModuleLoad(q, blob, len(blob))
    fill = lib.gpuxKernelGet(mod, b"nmk_fill_u32")
    n = 100003
    for kind in (3, 1):                            # Host, Shared
        ptr = _alloc(lib, g, q, n * 4, kind)
        assert ptr % 64 == 0
        descs, keep = _params(g, [(ctypes.c_void_p(ptr), 8),
                                  (ctypes.c_uint32(0xC0FFEE), 4),
                                  (ctypes.c_int64(n), 5)])
        ev = lib.gpuxLaunchKernel(q, fill, 64, 1, 1, 256, 1, 1, NO_DEPS, descs)
        lib.gpuxWait(q, ev)
        lib.gpuxDestroyEvent(q, ev)
        assert (_host_view(ptr, n, np.uint32) == 0xC0FFEE).all()
        lib.gpuxDeAlloc(q, ptr)
    # Local: no pointer, DeAlloc(NULL) balances
    res = g.GPUAllocResult()
    lib.gpuxAlloc(q, 1024, 64, 2, NO_DEPS, ctypes.byref(res))
    assert res.ptr is None
    lib.gpuxDestroyEvent(q, res.event)
    lib.gpuxDeAlloc(q, None)
    dev = _alloc(lib, g, q, 1 << 20, 0)
    assert dev and dev % 256 == 0
    # the queue stays usable for the buffer after the creator let go of it
    lib.gpuxKernelDestroy(fill)
    lib.gpuxModuleDestroy(mod)
    lib.gpuxQueueDestroy(q)
    lib.gpuxDeAlloc(q, dev)


def test_dependent_launches_and_event_chain(rt):
    """An event returned by one launch orders the next (deps array)."""
    lib, g, low = rt
    q = lib.gpuxQueueCreate(b"gpu")
    blob = low.kernel_blob("maps")
    mod = lib.gpuxModuleLoad(q, blob, len(blob))
    fill = lib.gpuxKernelGet(mod, b"nmk_fill_u32")
    n = 1 << 22
    ptr = _alloc(lib, g, q, n * 4, 1)
    ev = None
    for value in range(1, 6):
        deps = (ctypes.c_void_p * 2)(ev, None) if ev else NO_DEPS
        descs, keep = _params(g, [(ctypes.c_void_p(ptr), 8),
                                  (ctypes.c_uint32(value), 4),
                                  (ctypes.c_int64(n), 5)])
        new_ev = lib.gpuxLaunchKernel(q, fill, 256, 1, 1, 256, 1, 1, deps, descs)
        if ev:
            lib.gpuxDestroyEvent(q, ev)
        ev = new_ev
    lib.gpuxWait(q, ev)
    lib.gpuxDestroyEvent(q, ev)
    assert (_host_view(ptr, n, np.uint32) == 5).all()
    lib.gpuxDeAlloc(q, ptr)
    lib.gpuxKernelDestroy(fill)
    lib.gpuxModuleDestroy(mod)
    lib.gpuxQueueDestroy(q)


@pytest.mark.parametrize("local", [1, 8, 64, 100, 256])
def test_workgroup_memory_param(rt, local):
    """A ptr param with data == NULL becomes `size` bytes of LDS."""
    lib, g, low = rt
    q = lib.gpuxQueueCreate(None)
    blob = low.kernel_blob("twins")
    mod = lib.gpuxModuleLoad(q, blob, len(blob))
    kern = lib.gpuxKernelGet(mod, b"nmk_twin_group_reverse_i32")
    groups = 37
    n = local * groups
    a_ptr = _alloc(lib, g, q, n * 4, 1)
    b_ptr = _alloc(lib, g, q, n * 4, 1)
    a = _host_view(a_ptr, n, np.int32)
    a[:] = np.arange(n, dtype=np.int32) * 3 + 1
    i64 = ctypes.c_int64
    descs, keep = _params(g, [
        (ctypes.c_void_p(a_ptr), 8), (i64(n), 5), (i64(1), 5),
        (ctypes.c_void_p(b_ptr), 8), (i64(n), 5), (i64(1), 5),
        (None, (8, local * 4)),
        (i64(n), 5), (i64(1), 5), (i64(1), 5)])
    ev = lib.gpuxLaunchKernel(q, kern, groups, 1, 1, local, 1, 1, NO_DEPS, descs)
    lib.gpuxWait(q, ev)
    lib.gpuxDestroyEvent(q, ev)
    expect = a.reshape(groups, local)[:, ::-1].ravel()
    assert np.array_equal(_host_view(b_ptr, n, np.int32), expect)
    for p in (a_ptr, b_ptr):
        lib.gpuxDeAlloc(q, p)
    lib.gpuxKernelDestroy(kern)
    lib.gpuxModuleDestroy(mod)
    lib.gpuxQueueDestroy(q)


@pytest.mark.parametrize("shape", [(1,), (7,), (1, 1), (7, 13), (1, 1, 1),
                                   (7, 13, 23), (4096, 4096), (2 ** 24,)])
def test_suggest_block_size_on_device(rt, shape):
    from oracle import oracle as orc
    lib, g, low = rt
    q = lib.gpuxQueueCreate(None)
    blob = low.kernel_blob("twins")
    mod = lib.gpuxModuleLoad(q, blob, len(blob))
    kern = lib.gpuxKernelGet(mod, f"nmk_twin_get_global_id_{len(shape)}".encode())
    gs = (ctypes.c_uint32 * len(shape))(*shape)
    bs = (ctypes.c_uint32 * len(shape))()
    lib.gpuxSuggestBlockSize(q, kern, gs, bs, len(shape))
    assert tuple(bs) == orc.suggest_block_size(256, shape)
    lib.gpuxKernelDestroy(kern)
    lib.gpuxModuleDestroy(mod)
    lib.gpuxQueueDestroy(q)


def test_queue_interface_is_visible_to_companion_libraries(rt, hip):
    """The math runtime casts the queue to GPUQueueInterface* and uses the HIP
    extension; an end-to-end gemm on a queue created here proves the layout."""
    from numba_mlir_amd.mlir import math_runtime, ops
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    b = np.arange(8, dtype=np.float32).reshape(4, 2)
    got = ops.dot(hip.asarray(a), hip.asarray(b)).asnumpy()
    assert np.array_equal(got, a @ b)
    assert math_runtime.last_kernel() == "sgemm_generic"


def test_async_mode_keeps_order(hip):
    """Launches enqueued without a wait still execute in order."""
    from numba_mlir_amd.mlir import ops
    ctx = hip.get_context()
    rng = np.random.default_rng(0)
    a = rng.standard_normal((512, 1024))
    b = rng.standard_normal((1, 1024))
    d_a, d_b = hip.asarray(a), hip.asarray(b)
    out = hip.empty(a.shape, a.dtype)
    ctx.set_async(True)
    ops.add(d_a, d_b, out=out)
    for _ in range(10):
        ops.add(out, d_b, out=out)
    ctx.synchronize()
    ctx.set_async(False)
    expect = a + b
    for _ in range(10):
        expect = expect + b
    assert out.asnumpy().tobytes() == expect.tobytes()


@pytest.mark.parametrize("shared_queue", [False, True])
def test_call_sequence_from_six_threads(rt, shared_queue):
    """Compiled functions run on whatever Python thread calls them: six
    threads repeat alloc -> launch -> wait -> read -> dealloc, each on a queue
    of its own or all on one (ctypes drops the GIL during the calls)."""
    import threading
    lib, g, low = rt
    blob = low.kernel_blob("twins")
    one = lib.gpuxQueueCreate(None) if shared_queue else None
    errors = []

    def work(seed):
        try:
            q = one if shared_queue else lib.gpuxQueueCreate(None)
            mod = lib.gpuxModuleLoad(q, blob, len(blob))
            kern = lib.gpuxKernelGet(mod, b"nmk_twin_get_global_id_2")
            for it in range(60):
                r, c = 3 + (seed + it) % 5, 5 + (seed * 7 + it) % 11
                ptr = _alloc(lib, g, q, r * c * 4, 1)
                host = _host_view(ptr, r * c, np.int32)
                host[:] = -1
                descs, keep = _params(g, [
                    (ctypes.c_void_p(ptr), 8), (ctypes.c_int64(r), 5), (ctypes.c_int64(c), 5),
                    (ctypes.c_int64(c), 5), (ctypes.c_int64(1), 5),
                    (ctypes.c_int64(r), 5), (ctypes.c_int64(c), 5), (ctypes.c_int64(1), 5)])
                ev = lib.gpuxLaunchKernel(q, kern, 1, 1, 1, r, c, 1, NO_DEPS, descs)
                lib.gpuxWait(q, ev)
                lib.gpuxDestroyEvent(q, ev)
                i, j = np.meshgrid(np.arange(r), np.arange(c), indexing="ij")
                if not np.array_equal(host.reshape(r, c), i + 100 * j):
                    errors.append((seed, it, host.copy()))
                lib.gpuxDeAlloc(q, ptr)
            lib.gpuxKernelDestroy(kern)
            lib.gpuxModuleDestroy(mod)
            if not shared_queue:
                lib.gpuxQueueDestroy(q)
        except Exception as exc:      # noqa: BLE001
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(s,)) for s in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if shared_queue:
        lib.gpuxQueueDestroy(one)
    assert not errors, errors[:2]
