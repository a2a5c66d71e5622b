"""Host-only unit tests of the gpux runtime's own logic: the runtime sources
linked against a recording HIP table (tests/host/HipApiMock.cpp).  Covers
argument marshalling, terminators, reference counting, the event pool, device
strings and fatal paths; no GPU involved."""

import ctypes
import os
import subprocess
import sys
import threading

import pytest

from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "host"))
import build_mock  # noqa: E402

ELF = b"\x7fELF" + bytes(124)


class Desc(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("size", ctypes.c_int32),
                ("type", ctypes.c_int32)]


class AllocResult(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("event", ctypes.c_void_p)]


def _load():
    lib = ctypes.CDLL(build_mock.build())
    vp, sz = ctypes.c_void_p, ctypes.c_size_t
    lib.gpuxQueueCreate.restype = vp
    lib.gpuxQueueCreate.argtypes = [ctypes.c_char_p]
    lib.gpuxQueueDestroy.argtypes = [vp]
    lib.gpuxModuleLoad.restype = vp
    lib.gpuxModuleLoad.argtypes = [vp, ctypes.c_char_p, sz]
    lib.gpuxModuleDestroy.argtypes = [vp]
    lib.gpuxKernelGet.restype = vp
    lib.gpuxKernelGet.argtypes = [vp, ctypes.c_char_p]
    lib.gpuxKernelDestroy.argtypes = [vp]
    lib.gpuxLaunchKernel.restype = vp
    lib.gpuxLaunchKernel.argtypes = [vp, vp, sz, sz, sz, sz, sz, sz, vp, vp]
    lib.gpuxWait.argtypes = [vp, vp]
    lib.gpuxDestroyEvent.argtypes = [vp, vp]
    lib.gpuxAlloc.argtypes = [vp, sz, sz, ctypes.c_int, vp,
                              ctypes.POINTER(AllocResult)]
    lib.gpuxDeAlloc.argtypes = [vp, vp]
    lib.gpuxSuggestBlockSize.argtypes = [vp, vp, ctypes.POINTER(ctypes.c_uint32),
                                         ctypes.POINTER(ctypes.c_uint32), sz]
    lib.gpuxDuplicateQueue.restype = vp
    lib.gpuxDuplicateQueue.argtypes = [vp]
    lib.mockCounter.restype = ctypes.c_long
    lib.mockCounter.argtypes = [ctypes.c_char_p]
    return lib


@pytest.fixture(scope="module")
def rt():
    return _load()


def counter(rt, name):
    return rt.mockCounter(name.encode())


NO_DEPS = (ctypes.c_void_p * 1)(None)


def make_params(entries):
    """entries: list of (ctypes value or None, size, type)."""
    descs = (Desc * (len(entries) + 1))()
    keep = []
    for i, (val, size, ptype) in enumerate(entries):
        if val is not None:
            keep.append(val)
            descs[i].data = ctypes.cast(ctypes.pointer(val), ctypes.c_void_p)
        else:
            descs[i].data = None
        descs[i].size = size
        descs[i].type = ptype
    descs[len(entries)] = Desc(None, 0, 0)
    return descs, keep


def last_launch(rt, nparams):
    grid = (ctypes.c_uint * 3)()
    block = (ctypes.c_uint * 3)()
    shared = ctypes.c_uint()
    params = (ctypes.c_uint64 * 32)()
    ptrs = (ctypes.c_void_p * 32)()
    stream = ctypes.c_void_p()
    rt.mockLastLaunch(grid, block, ctypes.byref(shared), params, ptrs,
                      ctypes.byref(stream))
    return list(grid), list(block), shared.value, list(params)[:nparams], \
        list(ptrs)[:nparams], stream.value


@pytest.fixture()
def qk(rt):
    q = rt.gpuxQueueCreate(None)
    m = rt.gpuxModuleLoad(q, ELF, len(ELF))
    k = rt.gpuxKernelGet(m, b"kern_wg256")
    yield q, m, k
    rt.gpuxKernelDestroy(k)
    rt.gpuxModuleDestroy(m)
    rt.gpuxQueueDestroy(q)


def test_every_param_type_is_passed_by_slot(rt, qk):
    q, _, k = qk
    entries = [
        (ctypes.c_uint64(1), 1, 1),                      # bool_
        (ctypes.c_int64(-7 & 0xFF), 1, 2),               # int8
        (ctypes.c_int64(300), 2, 3),                     # int16
        (ctypes.c_int64(123456), 4, 4),                  # int32
        (ctypes.c_int64(-5), 8, 5),                      # int64
        (ctypes.c_uint64(0x3fc00000), 4, 6),             # float32 1.5 bits
        (ctypes.c_double(2.25), 8, 7),                   # float64
        (ctypes.c_uint64(0xdeadbeef000), 8, 8),          # ptr (device pointer)
    ]
    descs, keep = make_params(entries)
    rt.mockExpectParams(len(entries))
    ev = rt.gpuxLaunchKernel(q, k, 3, 2, 1, 64, 2, 1, NO_DEPS, descs)
    grid, block, shared, params, ptrs, _ = last_launch(rt, len(entries))
    assert (grid, block, shared) == ([3, 2, 1], [64, 2, 1], 0)
    # kernelParams[i] is the caller's own value slot
    for i in range(len(entries)):
        assert ptrs[i] == descs[i].data
    assert params[3] == 123456 and params[7] == 0xdeadbeef000
    assert ctypes.c_int64(params[4]).value == -5
    rt.gpuxWait(q, ev)
    rt.gpuxDestroyEvent(q, ev)


def test_workgroup_memory_params_become_offsets(rt, qk):
    q, _, k = qk
    entries = [
        (ctypes.c_uint64(0x1000), 8, 8),
        (None, 100, 8),           # LDS buffer A: offset 0
        (ctypes.c_int64(9), 8, 5),
        (None, 40, 8),            # LDS buffer B: offset 112 (16-byte aligned)
        (None, 8, 8),             # LDS buffer C: offset 160
    ]
    descs, keep = make_params(entries)
    rt.mockExpectParams(len(entries))
    ev = rt.gpuxLaunchKernel(q, k, 1, 1, 1, 64, 1, 1, NO_DEPS, descs)
    _, _, shared, params, _, _ = last_launch(rt, len(entries))
    assert params[1] == 0 and params[3] == 112 and params[4] == 160
    assert shared == 168
    rt.gpuxDestroyEvent(q, ev)


@pytest.mark.parametrize("ndeps", [0, 1, 5])
def test_dependency_arrays_are_null_terminated(rt, qk, ndeps):
    """Dependencies from another queue become stream waits on recorded events;
    the array is scanned up to its NULL terminator."""
    q, _, k = qk
    q2 = rt.gpuxQueueCreate(b"gpu:1")
    m2 = rt.gpuxModuleLoad(q2, ELF, len(ELF))
    k2 = rt.gpuxKernelGet(m2, b"kern")
    descs, _ = make_params([])
    rt.mockExpectParams(0)
    evs = [rt.gpuxLaunchKernel(q2, k2, 1, 1, 1, 1, 1, 1, NO_DEPS, descs)
           for _ in range(ndeps)]
    deps = (ctypes.c_void_p * (ndeps + 1))(*evs, None)
    before = counter(rt, "stream_waits"), counter(rt, "event_records")
    ev = rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, deps, descs)
    assert counter(rt, "stream_waits") - before[0] == ndeps
    assert counter(rt, "event_records") - before[1] == ndeps
    # using the same dependencies again re-uses their records
    ev2 = rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, deps, descs)
    assert counter(rt, "event_records") - before[1] == ndeps
    # allocation waits for its dependencies on the host: one drain of the
    # other queue's stream covers them all
    before = counter(rt, "stream_syncs")
    res = AllocResult()
    rt.gpuxAlloc(q, 64, 64, 0, deps, ctypes.byref(res))
    assert counter(rt, "stream_syncs") - before == (1 if ndeps else 0)
    rt.gpuxDeAlloc(q, res.ptr)
    for e in [ev, ev2, res.event]:
        rt.gpuxDestroyEvent(q, e)
    for e in evs:
        rt.gpuxDestroyEvent(q2, e)
    rt.gpuxKernelDestroy(k2)
    rt.gpuxModuleDestroy(m2)
    rt.gpuxQueueDestroy(q2)


def test_same_queue_events_are_stream_positions(rt, qk):
    """A queue is one in-order stream: its own events need no device marker,
    no stream wait, and one drain completes every earlier position."""
    q, _, k = qk
    descs, _ = make_params([])
    rt.mockExpectParams(0)
    base = {n: counter(rt, n) for n in ("event_records", "stream_waits",
                                        "stream_syncs", "events_created")}
    evs = []
    for _ in range(4):
        deps = (ctypes.c_void_p * 2)(evs[-1], None) if evs else NO_DEPS
        evs.append(rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, deps, descs))
    assert counter(rt, "event_records") == base["event_records"]
    assert counter(rt, "stream_waits") == base["stream_waits"]
    assert counter(rt, "events_created") == base["events_created"]
    rt.gpuxWait(q, evs[-1])                       # drains the stream once
    assert counter(rt, "stream_syncs") == base["stream_syncs"] + 1
    for e in evs[:-1]:                            # earlier positions: known done
        rt.gpuxWait(q, e)
    assert counter(rt, "stream_syncs") == base["stream_syncs"] + 1
    ev = rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, NO_DEPS, descs)
    rt.gpuxWait(q, ev)                            # a new position: drains again
    assert counter(rt, "stream_syncs") == base["stream_syncs"] + 2
    for e in evs + [ev]:
        rt.gpuxDestroyEvent(q, e)


def test_empty_launch_returns_a_waitable_event_but_launches_nothing(rt, qk):
    q, _, k = qk
    descs, _ = make_params([])
    before = counter(rt, "launches")
    ev = rt.gpuxLaunchKernel(q, k, 0, 1, 1, 64, 1, 1, NO_DEPS, descs)
    assert counter(rt, "launches") == before and ev
    rt.gpuxWait(q, ev)
    rt.gpuxDestroyEvent(q, ev)


def test_allocation_event_is_already_complete(rt, qk):
    q, _, k = qk
    descs, _ = make_params([])
    rt.mockExpectParams(0)
    pending = rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, NO_DEPS, descs)
    res = AllocResult()
    rt.gpuxAlloc(q, 64, 64, 0, NO_DEPS, ctypes.byref(res))
    before = counter(rt, "stream_syncs")
    rt.gpuxWait(q, res.event)                     # no drain needed
    assert counter(rt, "stream_syncs") == before
    rt.gpuxDestroyEvent(q, res.event)
    rt.gpuxDestroyEvent(q, pending)
    rt.gpuxDeAlloc(q, res.ptr)


def test_queue_lives_until_last_event_and_allocation(rt):
    base = counter(rt, "streams_live")
    q = rt.gpuxQueueCreate(b"level_zero:gpu:1")
    assert counter(rt, "current_device") == 1
    assert counter(rt, "streams_live") == base + 1
    m = rt.gpuxModuleLoad(q, ELF, len(ELF))
    k = rt.gpuxKernelGet(m, b"kern")
    descs, _ = make_params([])
    rt.mockExpectParams(0)
    ev = rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, NO_DEPS, descs)
    res = AllocResult()
    rt.gpuxAlloc(q, 1024, 64, 0, NO_DEPS, ctypes.byref(res))
    rt.gpuxDestroyEvent(q, res.event)
    rt.gpuxKernelDestroy(k)
    rt.gpuxModuleDestroy(m)
    rt.gpuxQueueDestroy(q)                       # creator's reference only
    assert counter(rt, "streams_live") == base + 1
    rt.gpuxDestroyEvent(q, ev)
    assert counter(rt, "streams_live") == base + 1   # allocation still holds it
    rt.gpuxDeAlloc(q, res.ptr)                   # e.g. from a MemInfo destructor
    assert counter(rt, "streams_live") == base
    assert counter(rt, "events_live") == 0       # the pool died with the queue


def test_allocation_kinds(rt, qk):
    q, _, _ = qk
    live = counter(rt, "allocs_live")
    ptrs = {}
    for kind in (0, 1, 3):
        res = AllocResult()
        rt.gpuxAlloc(q, 4096, 64, kind, NO_DEPS, ctypes.byref(res))
        assert res.ptr and res.ptr % 64 == 0 and res.event
        rt.gpuxWait(q, res.event)
        rt.gpuxDestroyEvent(q, res.event)
        ptrs[kind] = res.ptr
    assert counter(rt, "allocs_live") == live + 3
    res = AllocResult()
    rt.gpuxAlloc(q, 4096, 64, 2, NO_DEPS, ctypes.byref(res))   # Local: no pointer
    assert res.ptr is None and res.event
    rt.gpuxDestroyEvent(q, res.event)
    fd, fh = counter(rt, "frees_device"), counter(rt, "frees_host")
    rt.gpuxDeAlloc(q, None)                       # balances the Local alloc
    rt.gpuxDeAlloc(q, ptrs[0])
    rt.gpuxDeAlloc(q, ptrs[1])
    rt.gpuxDeAlloc(q, ptrs[3])
    assert counter(rt, "frees_device") == fd + 2 and counter(rt, "frees_host") == fh + 1
    assert counter(rt, "allocs_live") == live
    # zero-byte requests still return a distinct pointer
    rt.gpuxAlloc(q, 0, 64, 0, NO_DEPS, ctypes.byref(res))
    assert res.ptr
    rt.gpuxDestroyEvent(q, res.event)
    rt.gpuxDeAlloc(q, res.ptr)


def test_large_device_blocks_are_kept_for_reuse(rt, qk):
    """gpuxDeAlloc keeps device blocks of 64 KiB and more; the next gpuxAlloc
    of the same (256-byte rounded) size takes one without calling hipMalloc."""
    q, _, _ = qk
    res = AllocResult()

    def alloc(nbytes, kind=0):
        rt.gpuxAlloc(q, nbytes, 64, kind, NO_DEPS, ctypes.byref(res))
        rt.gpuxDestroyEvent(q, res.event)
        return res.ptr

    mallocs, frees = counter(rt, "mallocs_device"), counter(rt, "frees_device")
    a = alloc(1 << 20)
    b = alloc(1 << 20)
    assert a != b and counter(rt, "mallocs_device") == mallocs + 2
    rt.gpuxDeAlloc(q, a)
    rt.gpuxDeAlloc(q, b)
    assert counter(rt, "frees_device") == frees            # kept, not freed
    c = alloc((1 << 20) - 100)                               # rounds to the same size
    d = alloc(1 << 20)
    assert {c, d} == {a, b} and counter(rt, "mallocs_device") == mallocs + 2
    e = alloc(2 << 20)                                       # another size: a new block
    assert e not in (a, b) and counter(rt, "mallocs_device") == mallocs + 3
    small = alloc(4096)                                      # below the threshold
    rt.gpuxDeAlloc(q, small)
    assert counter(rt, "frees_device") == frees + 1
    shared = alloc(1 << 20, kind=1)                          # only device memory is kept
    rt.gpuxDeAlloc(q, shared)
    assert counter(rt, "frees_device") == frees + 2
    for p in (c, d, e):
        rt.gpuxDeAlloc(q, p)


def test_kept_blocks_go_back_to_the_queue_that_released_them(rt, qk):
    """A released block may still be in use by work of the releasing queue's
    stream: only that queue (same in-order stream) gets it back at once;
    another queue on the device gets it once the first one's stream has been
    drained and destroyed."""
    q, _, _ = qk
    res = AllocResult()

    def alloc(queue, nbytes):
        rt.gpuxAlloc(queue, nbytes, 64, 0, NO_DEPS, ctypes.byref(res))
        rt.gpuxDestroyEvent(queue, res.event)
        return res.ptr

    size = 3 << 20                                           # a size no other test keeps
    q2 = rt.gpuxQueueCreate(None)                            # same device, its own stream
    a = alloc(q2, size)
    rt.gpuxDeAlloc(q2, a)
    mallocs = counter(rt, "mallocs_device")
    b = alloc(q, size)                                       # q must not see q2's block
    assert b != a and counter(rt, "mallocs_device") == mallocs + 1
    c = alloc(q2, size)                                      # q2 itself does
    assert c == a and counter(rt, "mallocs_device") == mallocs + 1
    rt.gpuxDeAlloc(q2, c)
    syncs = counter(rt, "stream_syncs")
    rt.gpuxQueueDestroy(q2)                                  # last reference: drained, destroyed
    assert counter(rt, "stream_syncs") == syncs + 1
    d = alloc(q, size)                                       # now anybody's
    assert d == a and counter(rt, "mallocs_device") == mallocs + 1
    rt.gpuxDeAlloc(q, b)
    rt.gpuxDeAlloc(q, d)


def test_an_event_returns_to_the_queue_that_handed_it_out(rt, qk):
    """gpuxDestroyEvent names a queue, but the event belongs to its owner's
    pool and holds a reference to the owner: both go back there."""
    q, _, k = qk
    q2 = rt.gpuxQueueCreate(None)
    descs, _ = make_params([])
    rt.mockExpectParams(0)
    streams = counter(rt, "streams_live")
    ev = rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, NO_DEPS, descs)
    rt.gpuxWait(q, ev)
    rt.gpuxDestroyEvent(q2, ev)                              # the wrong queue is named
    rt.gpuxQueueDestroy(q2)                                  # q2 held no event: it goes
    assert counter(rt, "streams_live") == streams - 1
    ev2 = rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, NO_DEPS, descs)
    assert ev2 == ev                                         # reused from q's own pool
    rt.gpuxWait(q, ev2)
    rt.gpuxDestroyEvent(q, ev2)


def test_event_pool_reuses_events(rt, qk):
    """Cross-queue use creates a device event once per pooled slot."""
    q, _, k = qk
    q2 = rt.gpuxQueueCreate(None)
    m2 = rt.gpuxModuleLoad(q2, ELF, len(ELF))
    k2 = rt.gpuxKernelGet(m2, b"kern")
    descs, _ = make_params([])
    rt.mockExpectParams(0)
    created = counter(rt, "events_created")
    for _ in range(200):
        ev = rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, NO_DEPS, descs)
        deps = (ctypes.c_void_p * 2)(ev, None)
        ev2 = rt.gpuxLaunchKernel(q2, k2, 1, 1, 1, 1, 1, 1, deps, descs)
        rt.gpuxWait(q2, ev2)
        rt.gpuxDestroyEvent(q2, ev2)
        rt.gpuxDestroyEvent(q, ev)
    assert counter(rt, "events_created") - created <= 1
    rt.gpuxKernelDestroy(k2)
    rt.gpuxModuleDestroy(m2)
    rt.gpuxQueueDestroy(q2)


def test_event_pool_is_thread_safe(rt, qk):
    q, _, k = qk
    descs, _ = make_params([])
    rt.mockExpectParams(0)
    launches = counter(rt, "launches")
    errors = []

    def worker():
        try:
            for _ in range(300):
                evs = [rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, NO_DEPS, descs)
                       for _ in range(3)]
                for e in evs:
                    rt.gpuxDestroyEvent(q, e)
        except Exception as exc:   # pragma: no cover
            errors.append(exc)

    threads = [threading.Thread(target=worker) for _ in range(8)]
    [t.start() for t in threads]
    [t.join() for t in threads]
    assert not errors
    assert counter(rt, "launches") - launches == 8 * 300 * 3
    assert counter(rt, "events_live") <= 8 * 3 + 1


SHAPES = [(1,), (7,), (1, 1), (7, 13), (1, 1, 1), (7, 13, 23), (4096, 4096),
          (8192, 8192), (2 ** 24,), (16384, 8192), (100, 3), (300, 5, 5)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("bound", [64, 256, 1024])
def test_suggest_block_size_follows_the_reference_rule(rt, qk, shape, bound):
    q, m, _ = qk
    k = rt.gpuxKernelGet(m, f"kern_wg{bound}".encode())
    g = (ctypes.c_uint32 * len(shape))(*shape)
    b = (ctypes.c_uint32 * len(shape))()
    rt.gpuxSuggestBlockSize(q, k, g, b, len(shape))
    # preferred workgroup = min(launch bound, 256), then the closed form
    assert tuple(b) == orc.suggest_block_size(min(bound, 256), shape)
    total = 1
    for x in b:
        total *= x
    assert total <= 256
    rt.gpuxKernelDestroy(k)


@pytest.mark.parametrize("name,ordinal", [
    (None, 0), (b"", 0), (b"gpu", 0), (b"hip", 0), (b"hip:gpu", 0),
    (b"hip:gpu:1", 1), (b"level_zero:gpu:0", 0), (b"opencl:gpu:1", 1),
    (b"gpu:1", 1), (b"1", 1), (b"*:*:0", 0),
])
def test_device_strings(rt, name, ordinal):
    q = rt.gpuxQueueCreate(name)
    assert counter(rt, "current_device") == ordinal
    rt.gpuxQueueDestroy(q)


def test_duplicate_queue_copies_the_native_handle(rt):
    native = ctypes.c_void_p(0x1234)
    dup = rt.gpuxDuplicateQueue(ctypes.cast(ctypes.pointer(native), ctypes.c_void_p))
    assert dup and ctypes.cast(dup, ctypes.POINTER(ctypes.c_void_p))[0] == 0x1234
    ctypes.CDLL(None).free(ctypes.c_void_p(dup))


FATAL = {
    "device ordinal out of range":
        ("q = rt.gpuxQueueCreate(b'hip:gpu:7')", "2 HIP device(s) present"),
    "cpu device":
        ("q = rt.gpuxQueueCreate(b'opencl:cpu:0')", "only drives GPU devices"),
    "bad blob":
        ("q = rt.gpuxQueueCreate(None); rt.gpuxModuleLoad(q, b'x' * 128, 128)",
         "Invalid module"),
    "missing kernel":
        ("q = rt.gpuxQueueCreate(None); m = rt.gpuxModuleLoad(q, ELF, len(ELF));"
         "rt.gpuxKernelGet(m, b'missing')", "Kernel 'missing' not found"),
    "unknown alloc type":
        ("q = rt.gpuxQueueCreate(None); r = AllocResult();"
         "rt.gpuxAlloc(q, 8, 64, 9, NO_DEPS, ctypes.byref(r))",
         "Invalid allocation type"),
    "unknown param type":
        ("q = rt.gpuxQueueCreate(None); m = rt.gpuxModuleLoad(q, ELF, len(ELF));"
         "k = rt.gpuxKernelGet(m, b'k'); d, keep = make_params([(ctypes.c_int64(1), 8, 42)]);"
         "rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, NO_DEPS, d)",
         "Unhandled param type: 42"),
    "wrong param size":
        ("q = rt.gpuxQueueCreate(None); m = rt.gpuxModuleLoad(q, ELF, len(ELF));"
         "k = rt.gpuxKernelGet(m, b'k'); d, keep = make_params([(ctypes.c_int64(1), 4, 5)]);"
         "rt.gpuxLaunchKernel(q, k, 1, 1, 1, 1, 1, 1, NO_DEPS, d)",
         "needs a 8-byte value, got 4"),
    "grid.y too large":
        ("q = rt.gpuxQueueCreate(None); m = rt.gpuxModuleLoad(q, ELF, len(ELF));"
         "k = rt.gpuxKernelGet(m, b'k'); d, keep = make_params([]);"
         "rt.gpuxLaunchKernel(q, k, 1, 70000, 1, 1, 1, 1, NO_DEPS, d)",
         "exceeds the HIP limits"),
    "more work-items along x than a launch counts":
        ("q = rt.gpuxQueueCreate(None); m = rt.gpuxModuleLoad(q, ELF, len(ELF));"
         "k = rt.gpuxKernelGet(m, b'k'); d, keep = make_params([]);"
         "rt.gpuxLaunchKernel(q, k, 67108865, 1, 1, 256, 1, 1, NO_DEPS, d)",
         "exceeds 4294967295 work-items along a dimension"),
    "foreign pointer":
        ("q = rt.gpuxQueueCreate(None); rt.gpuxDeAlloc(q, 0x40)",
         "was not allocated by gpuxAlloc"),
}


@pytest.mark.parametrize("case", sorted(FATAL))
def test_fatal_paths(case):
    body, message = FATAL[case]
    code = (
        "import sys, ctypes\n"
        f"sys.path.insert(0, {os.path.join(ROOT, 'tests')!r})\n"
        f"sys.path.insert(0, {ROOT!r})\n"
        "from test_runtime_host import _load, make_params, AllocResult, NO_DEPS, ELF\n"
        "rt = _load()\n" + body + "\n")
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True,
                          text=True)
    assert proc.returncode == -6, (proc.returncode, proc.stdout, proc.stderr)
    assert message in proc.stdout, proc.stdout


def test_blob_dump_env(tmp_path):
    code = (
        "import sys\n"
        f"sys.path.insert(0, {os.path.join(ROOT, 'tests')!r})\n"
        f"sys.path.insert(0, {ROOT!r})\n"
        "from test_runtime_host import _load, ELF\n"
        "rt = _load(); q = rt.gpuxQueueCreate(None)\n"
        "rt.gpuxModuleLoad(q, ELF, len(ELF))\n")
    env = dict(os.environ, NUMBA_MLIR_DUMP_KERNEL_BLOB="1",
               NUMBA_MLIR_LOG_GPU_RUNTIME_CALLS="1")
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True,
                          text=True, cwd=tmp_path, env=env)
    assert proc.returncode == 0, proc.stderr
    dumps = [f for f in os.listdir(tmp_path) if f.startswith("kernel_dump_")]
    assert len(dumps) == 1
    assert open(os.path.join(tmp_path, dumps[0]), "rb").read() == ELF
    lines = proc.stdout.split("\n")
    assert lines[0] == "gpuxQueueCreate enter" and "gpuxModuleLoad exit" in lines
