"""``@kernel`` launches on the HIP runtime.

In the reference ``Kernel.__call__`` hands the Python body to the compiler,
which wraps it in one ``_gpu_range`` loop per dimension and emits a GPU kernel
(reference: numba_mlir/numba_mlir/mlir/kernel_impl.py:97-206).  Here the body is translated to HIP by ``kernel_compiler`` (types inferred from
the launch arguments, one specialisation per signature), compiled to a gfx950
code object and launched through ``gpuxModuleLoad`` / ``gpuxKernelGet`` /
``gpuxLaunchKernel``.  A kernel may instead be bound to a hand-written twin of
its body (``twin=`` names a symbol of the built-in "twins" code object;
``{dtype}`` and ``{rank}`` are filled from the first array argument): the
benchmark's pairwise kernel uses one whose work-items are remapped for
coalesced stores.  Everything around the body is the reference's behaviour:

* launch geometry: ``grid_k = ceil(global_k / local_k)``, tail guarded
  in-kernel, dimension 0 <-> x (reference: LowerToGpu.cpp:1113-1137);
* an empty local size asks ``gpuxSuggestBlockSize`` (LowerToGpu.cpp:373-471);
* all array arguments must live on one device (dpctl_interop.py:270-275).

The index builtins exist as Python stubs only; calling them outside a kernel
is an error, as in the reference.
"""

import ctypes
import threading
import weakref

import numpy as np

from . import kernel_compiler, lowered
from .gpu_runtime import runtime_lib
from .utils import readenv
from .device_array import HipNdArray, disjoint, streams
from .kernel_base import KernelBase
from .lowered import GPUParamDesc, lib

DEFAULT_LOCAL_SIZE = ()
LOCAL_MEM_FENCE = 1
GLOBAL_MEM_FENCE = 2

_DTYPE_TAGS = {
    np.dtype(np.int32): "i32",
    np.dtype(np.int64): "i64",
    np.dtype(np.float32): "f32",
    np.dtype(np.float64): "f64",
}


def _stub_error():
    raise NotImplementedError("This is a stub")


def get_global_id(axis):
    _stub_error()


def get_local_id(axis):
    _stub_error()


def get_group_id(axis):
    _stub_error()


def get_global_size(axis):
    _stub_error()


def get_local_size(axis):
    _stub_error()


class Stub(object):
    """Namespace of kernel-only functions; not instantiable (reference:
    numba_mlir/numba_mlir/mlir/kernel_impl.py:252-260)."""

    __slots__ = ()

    def __new__(cls):
        raise NotImplementedError("%s is not instantiable" % cls)


def _stub(name, params):
    exec(f"def {name}({params}): _stub_error()", globals())
    return globals()[name]


class atomic(Stub):
    """``atomic.add(arr, idx, val)`` / ``atomic.sub`` (kernel_impl.py:263-322)."""

    add = staticmethod(_stub("atomic_add", "arr, idx, val"))
    sub = staticmethod(_stub("atomic_sub", "arr, idx, val"))


def barrier(flags=None):
    """Work-group barrier with LOCAL_MEM_FENCE / GLOBAL_MEM_FENCE
    (kernel_impl.py:330-345)."""
    _stub_error()


def mem_fence(flags=None):
    _stub_error()


class local(Stub):
    """``local.array(shape, dtype)``: work-group memory (kernel_impl.py:366-400)."""

    array = staticmethod(_stub("local_array", "shape, dtype"))


class private(Stub):
    """``private.array(shape, dtype)``: per-work-item memory."""

    array = staticmethod(_stub("private_array", "shape, dtype"))


class group(Stub):
    """Work-group reductions (kernel_impl.py:440-482)."""

    reduce_add = staticmethod(_stub("group_reduce_add", "value"))
    reduce_mul = staticmethod(_stub("group_reduce_mul", "value"))
    reduce_min = staticmethod(_stub("group_reduce_min", "value"))
    reduce_max = staticmethod(_stub("group_reduce_max", "value"))


def kernel_func(func):
    """Device function callable from kernels (``mlir_njit(mlir_force_inline=
    True)`` in the reference, kernel_impl.py:209); a plain function here: the
    kernel compiler translates whatever Python function a kernel calls."""
    return func


def check_device_args(args):
    """All device arrays of a launch must share a queue."""
    ctx = None
    for a in args:
        if isinstance(a, HipNdArray):
            if ctx is None:
                ctx = a.ctx
            elif a.ctx is not ctx:
                raise ValueError(
                    f"Device arrays must share a device: {ctx.device} and "
                    f"{a.ctx.device}")
    if ctx is None:
        raise ValueError("A kernel launch needs at least one device array")
    return ctx


class _ParamList:
    """Builds the GPUParamDesc array the compiled host code would build
    (reference: mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:444-628)."""

    def __init__(self):
        self._slots = []

    def _add(self, cvalue, ptype):
        self._slots.append((cvalue, ptype))
        return cvalue

    def add_array(self, arr):
        """Returns the pointer slot (a launch plan rewrites it per call)."""
        slot = self._add(ctypes.c_void_p(arr.ptr), lowered.PARAM_PTR)
        for n in arr.shape:
            self._add(ctypes.c_int64(n), lowered.PARAM_INT64)
        for s in arr.elem_strides:
            self._add(ctypes.c_int64(s), lowered.PARAM_INT64)
        return slot

    def add_local(self, nbytes):
        self._slots.append((None, nbytes))

    _SCALAR_PARAMS = {
        np.dtype(np.bool_): (ctypes.c_bool, lowered.PARAM_BOOL),
        np.dtype(np.int8): (ctypes.c_int8, lowered.PARAM_INT8),
        np.dtype(np.uint8): (ctypes.c_uint8, lowered.PARAM_INT8),
        np.dtype(np.int16): (ctypes.c_int16, lowered.PARAM_INT16),
        np.dtype(np.uint16): (ctypes.c_uint16, lowered.PARAM_INT16),
        np.dtype(np.int32): (ctypes.c_int32, lowered.PARAM_INT32),
        np.dtype(np.uint32): (ctypes.c_uint32, lowered.PARAM_INT32),
        np.dtype(np.int64): (ctypes.c_int64, lowered.PARAM_INT64),
        np.dtype(np.uint64): (ctypes.c_uint64, lowered.PARAM_INT64),
        np.dtype(np.float32): (ctypes.c_float, lowered.PARAM_FLOAT32),
        np.dtype(np.float64): (ctypes.c_double, lowered.PARAM_FLOAT64),
    }

    def add_scalar(self, value):
        """Returns the value slot."""
        if isinstance(value, (bool, np.bool_)):
            return self._add(ctypes.c_bool(bool(value)), lowered.PARAM_BOOL)
        if isinstance(value, np.generic) and value.dtype in self._SCALAR_PARAMS:
            ctype, ptype = self._SCALAR_PARAMS[value.dtype]
            return self._add(ctype(value.item()), ptype)
        if isinstance(value, int):
            return self._add(ctypes.c_int64(value), lowered.PARAM_INT64)
        if isinstance(value, float):
            return self._add(ctypes.c_double(value), lowered.PARAM_FLOAT64)
        raise TypeError(f"Unsupported kernel argument type: {type(value)}")

    SLICE_NONE = -2 ** 63         # an omitted bound

    def add_slice(self, value):
        """Returns the three slots (start, stop, step)."""
        return [self._add(ctypes.c_int64(self.SLICE_NONE if part is None else int(part)),
                          lowered.PARAM_INT64)
                for part in (value.start, value.stop, value.step)]

    def build(self):
        descs = (GPUParamDesc * (len(self._slots) + 1))()
        for i, (cvalue, ptype) in enumerate(self._slots):
            if cvalue is None:     # workgroup memory: data == NULL, size = bytes
                descs[i].data = None
                descs[i].size = ptype
                descs[i].type = lowered.PARAM_PTR
                continue
            descs[i].data = ctypes.cast(ctypes.pointer(cvalue), ctypes.c_void_p)
            descs[i].size = ctypes.sizeof(cvalue)
            descs[i].type = ptype
        descs[len(self._slots)].data = None
        descs[len(self._slots)].size = 0
        descs[len(self._slots)].type = lowered.PARAM_NULL
        return descs


NO_DEPS = (ctypes.c_void_p * 1)(None)
MAX_SPECIALISATIONS = 16   # per kernel, before new shapes get the general form
MAX_PLANS = 64             # stored launches per kernel
TICKET_COUNTERS = 17 * 64  # of a generated reduction (jit_support.h: kTicketGroups + 1 counters, kTicketStride apart)
REDUCTION_BLOCKS = 2048    # of a generated 1-d reduction: eight per compute unit


def _release_handles(handles):
    for kern, module in handles:
        runtime_lib.gpuxKernelDestroy(kern)
        runtime_lib.gpuxModuleDestroy(module)


def _loaded_kernel(ctx, compiled):
    """gpuxModuleLoad + gpuxKernelGet once per context and code object; the
    handles are released before the context's queue (finalizers run last in,
    first out)."""
    table = getattr(ctx, "_jit_kernels", None)
    if table is None:
        table = ctx._jit_kernels = {}
        ctx._jit_handles = []
        weakref.finalize(ctx, _release_handles, ctx._jit_handles)
    key = (compiled.name, getattr(compiled, "fastmath", False))
    kern = table.get(key)
    if kern is None:
        blob = kernel_compiler.build_code_object(compiled)
        module = runtime_lib.gpuxModuleLoad(ctx.queue, blob, len(blob))
        kern = runtime_lib.gpuxKernelGet(module, compiled.name.encode())
        table[key] = kern
        ctx._jit_handles.append((kern, module))
    return kern


def _bounds_flag(ctx):
    """One zeroed int32 per context for bounds-checked launches."""
    flag = getattr(ctx, "_jit_bounds_flag", None)
    if flag is None:
        flag = ctx._jit_bounds_flag = HipNdArray.from_numpy(np.zeros(1, np.int32),
                                                               device=ctx.device)
    return flag


def captured_constants(func):
    """Hash of what a function's closure holds: constants a body captures are
    compiled in, so they belong to the key of its specialisations."""
    cells = []
    for cell in func.__closure__ or ():
        try:
            v = cell.cell_contents
        except ValueError:
            continue
        cells.append(v if isinstance(v, (bool, int, float, np.generic, tuple)) else id(v))
    try:
        return hash(tuple(cells))
    except TypeError:
        return id(func)


class Kernel(KernelBase):
    def __init__(self, func, kwargs):
        super().__init__(func)
        self.twin = kwargs.get("twin")
        # local.array sizes of a twin's body in bytes: a list, or a callable
        # (global_size, local_size) -> list.  Each becomes a workgroup-memory
        # parameter after the user arguments (GpuRuntimeToLlvm.cpp:507-536).
        # Compiled kernels know their own.
        self.local_bytes = kwargs.get("local_bytes", ())
        # boundscheck=True (or NUMBA_MLIR_KERNEL_BOUNDSCHECK=1, cf. Numba's
        # NUMBA_BOUNDSCHECK): an out-of-range index raises IndexError after the
        # launch instead of reading or writing foreign memory.
        self.boundscheck = bool(kwargs.get(
            "boundscheck", readenv("NUMBA_MLIR_KERNEL_BOUNDSCHECK", int, 0)))
        # fastmath=True lets a * b + c contract into one fused multiply-add
        # (the reference's kernel(fastmath=True), test_gpu.py:980-1008)
        self.fastmath = bool(kwargs.get("fastmath", False))
        self.last_launch = None
        self.last_plan = None  # the LaunchPlan of the most recent compiled launch
        self._compiled = {}
        self._plans = {}       # stored launches (shared by configured copies)

    def _twin_name(self, args):
        first = next((a for a in args if isinstance(a, HipNdArray)), None)
        tag = _DTYPE_TAGS.get(first.dtype) if first is not None else None
        return self.twin.format(dtype=tag, rank=len(self.global_size))

    def compile(self, args, ndim, remap=False, noalias=False, stream=True):
        """The specialisation of the body for these arguments (translated on
        first use; constants captured by the body are part of the key).
        ``noalias``: the caller found no two array arguments overlapping;
        ``stream``: they are too large to stay cached between launches."""
        import sys
        # Specialised on dense layouts and short trailing extents; a kernel
        # that keeps meeting new ones gets the general form for the rest.
        captured = captured_constants(self.py_func)
        for specialize in (True, False):
            types = [kernel_compiler.type_of_argument(a, specialize) for a in args]
            key = (ndim, tuple(kernel_compiler.type_key(t) for t in types),
                   captured, self.boundscheck, remap, noalias, stream)
            compiled = self._compiled.get(key)
            if compiled is not None or len(self._compiled) < MAX_SPECIALISATIONS:
                break
        if compiled is None:
            compiled = kernel_compiler.translate(self.py_func, types, ndim,
                                                 sys.modules[__name__],
                                                 self.boundscheck, remap,
                                                 noalias=noalias, stream=stream)
            compiled.fastmath = self.fastmath
            self._compiled[key] = compiled
        return compiled

    def __call__(self, *args, **kwargs):
        self.check_call_args(args, kwargs)
        ctx = check_device_args(args)

        ndim = len(self.global_size)
        assert 1 <= ndim <= 3, f"Invalid dim count: {ndim}"
        gsize3 = [int(g) for g in self.global_size] + [1] * (3 - ndim)

        if self.twin is not None:
            name = self._twin_name(args)
            compiled = kern = None
            if len(self.local_size) != 0:
                block = [int(n) for n in self.local_size]
            else:
                gsize = (ctypes.c_uint32 * ndim)(*[min(g, 0xFFFFFFFF) for g in gsize3[:ndim]])
                bsize = (ctypes.c_uint32 * ndim)()
                lib.nmhipSuggestBlockSize(ctx.handle, name.encode(), gsize, bsize, ndim)
                block = list(bsize)
            block += [1] * (3 - ndim)
            grid = [(g + b - 1) // b for g, b in zip(gsize3, block)]
        else:
            # Types, shapes and strides seen before replay a stored launch.
            noalias = disjoint([a for a in args if isinstance(a, HipNdArray)])
            key = (ctx, plan_key(args), captured_constants(self.py_func),
                   tuple(gsize3[:ndim]), tuple(self.local_size), noalias)
            plan = self._plans.get(key)
            if plan is not None:
                plan.run(args)
                self.last_launch, self.last_plan = plan.info, plan
                return
            # With a runtime-chosen block a body that cannot observe its
            # grouping is laid out for coalescing (last dimension on x), unless
            # that pushes a long dimension past the y / z grid limit.
            remap = len(self.local_size) == 0 and remap_mode(gsize3[:ndim])
            stream = streams([a for a in args if isinstance(a, HipNdArray)])
            compiled = self.compile(args, ndim, remap, noalias, stream)
            kern = _loaded_kernel(ctx, compiled)
            block, grid = _geometry(ctx, compiled, kern, gsize3[:ndim], self.local_size)
            if compiled.reversed_dims and max(grid[1:]) > 65535:
                compiled = self.compile(args, ndim, False, noalias, stream)
                kern = _loaded_kernel(ctx, compiled)
                block, grid = _geometry(ctx, compiled, kern, gsize3[:ndim],
                                        self.local_size)
            name = compiled.name

        if compiled is not None:
            plan = LaunchPlan(ctx, compiled, kern, self.py_func.__name__, grid, block,
                              gsize3, args)
            plan.run()
            if len(self._plans) >= MAX_PLANS:
                self._plans.clear()
            self._plans[key] = plan
            self.last_launch, self.last_plan = plan.info, plan
            return

        params = _ParamList()
        for a in args:
            if isinstance(a, HipNdArray):
                params.add_array(a)
            else:
                params.add_scalar(a)
        local_bytes = self.local_bytes
        if callable(local_bytes):
            local_bytes = local_bytes(tuple(gsize3[:ndim]), tuple(block[:ndim]))
        for nbytes in local_bytes:
            params.add_local(int(nbytes))
        for g in gsize3:
            params.add_scalar(int(g))
        descs = params.build()
        self.last_launch = {"kernel": name, "grid": tuple(grid), "block": tuple(block)}
        if 0 in gsize3:
            return
        lib.nmhipLaunch(ctx.handle, name.encode(), (ctypes.c_size_t * 3)(*grid),
                        (ctypes.c_size_t * 3)(*block), descs)


def remap_mode(global_size):
    """How a grid of these extents is laid out on the lanes when the body
    cannot observe its grouping: not at all (one dimension), last dimension
    on x with flat blocks (True), or -- when that dimension is shorter than a
    wave and the next one is not -- with lanes along the next dimension too
    ("tall")."""
    if len(global_size) < 2:
        return False
    if int(global_size[-1]) < 64 and int(global_size[-2]) >= 64:
        return "tall"
    return True


def _geometry(ctx, compiled, kern, global_size, local_size):
    """Block and grid of a compiled kernel in hardware order (x, y, z)."""
    ndim = len(global_size)
    order = list(range(ndim))
    if compiled.reversed_dims:
        order.reverse()
    sizes = [int(global_size[k]) for k in order]
    rows = getattr(compiled, "rows_per_lane", 1)
    if compiled.reversed_dims:
        # flat blocks, several work-items per lane along y (see translate_kernel)
        gsize = (ctypes.c_uint32 * 1)(min(sizes[0], 0xFFFFFFFF))
        bsize = (ctypes.c_uint32 * 1)()
        runtime_lib.gpuxSuggestBlockSize(ctx.queue, kern, gsize, bsize, 1)
        block = [int(bsize[0])] + [1] * (ndim - 1)
        if getattr(compiled, "lanes_along_y", False):
            # a grid of a few columns: whole rows side by side in a wave, as
            # many as bring the block to 256 lanes
            block[1] = max(1, min(256 // max(block[0], 1), sizes[1]))
    elif len(local_size) != 0:
        block = [int(local_size[k]) for k in order]
    else:
        gsize = (ctypes.c_uint32 * ndim)(*[min(g, 0xFFFFFFFF) for g in sizes])
        bsize = (ctypes.c_uint32 * ndim)()
        runtime_lib.gpuxSuggestBlockSize(ctx.queue, kern, gsize, bsize, ndim)
        block = list(bsize)
    sizes += [1] * (3 - ndim)
    block += [1] * (3 - ndim)
    grid = [(g + b - 1) // b for g, b in zip(sizes, block)]
    if rows > 1:
        grid[1] = (grid[1] + rows - 1) // rows     # blocks of block[1] * rows rows
    if ndim <= 2 and grid[1] > 65535:
        # (the generated kernels count their blocks along y, then z)
        grid[2] = (grid[1] + 65534) // 65535
        grid[1] = 65535
    return block, grid


class LaunchPlan:
    """One kernel launch with everything that depends only on the arguments'
    types, shapes and strides already done: the kernel handle, the geometry
    and the GPUParamDesc array.  ``run`` rewrites the pointer and scalar slots
    and replays the compiled host code's sequence for one kernel: launch,
    wait, destroy event (GpuRuntimeToLlvm.cpp:444-628)."""

    def __init__(self, ctx, compiled, kern, func_name, grid, block, gsize3, args,
                 ret=None, partials=()):
        self.ctx, self.compiled, self.kern, self.func_name = ctx, compiled, kern, func_name
        self.grid, self.block = tuple(grid), tuple(block)
        for g, b in zip(self.grid, self.block):
            if g * b > 2 ** 32 - 1:
                # (the runtime would abort the process: say it here instead)
                raise ValueError(
                    f"kernel '{func_name}': {g} blocks of {b} work-items are more than the "
                    "4294967295 work-items a launch holds along one dimension")
        self.info = {"kernel": compiled.name, "grid": self.grid, "block": self.block}
        self.empty = 0 in gsize3
        params = _ParamList()
        self._arg_slots = []
        for a in args:
            if isinstance(a, HipNdArray):
                self._arg_slots.append(params.add_array(a))
            elif isinstance(a, slice):
                self._arg_slots.append(params.add_slice(a))
            else:
                self._arg_slots.append(params.add_scalar(a))
        self._ret_slot = params.add_array(ret) if ret is not None else None
        # one pointer per reduction variable (the arrays stay with the plan)
        self.partials = list(partials)
        self.partials_free = threading.Lock()   # held from a launch into them to their read-back
        self._partial_slots = [params._add(ctypes.c_void_p(part.ptr), lowered.PARAM_PTR)
                               for part in partials]
        # the counters by which the launch's last block knows itself (zero
        # between launches: the kernel puts them back)
        self._ticket = None
        if self.partials:
            self._ticket = HipNdArray.from_numpy(np.zeros(TICKET_COUNTERS, np.uint32),
                                                 device=ctx.device)
            params._add(ctypes.c_void_p(self._ticket.ptr), lowered.PARAM_PTR)
        for nbytes in compiled.local_bytes:
            params.add_local(int(nbytes))
        for g in gsize3:
            params.add_scalar(int(g))
        self._flag = None
        if compiled.boundscheck:
            self._flag = _bounds_flag(ctx)
            params._add(ctypes.c_void_p(self._flag.ptr), lowered.PARAM_PTR)
        self._params = params             # owns the slots the descriptors point at
        self._descs = params.build()
        self._lock = threading.Lock()     # slots are rewritten per call
        self._launch = (ctx.queue, kern, *self.grid, *self.block, NO_DEPS, self._descs)
        # what later arguments must look like (the kernel and its geometry
        # were chosen for these types, shapes and strides)
        self._key = plan_key(args)
        self._ret_key = None if ret is None else (ret.dtype, ret.shape, ret.strides)

    def _refresh(self, args, ret, partials):
        """Rewrites the pointer and scalar slots (the lock is held)."""
        for slot, a in zip(self._arg_slots, args):
            if isinstance(a, HipNdArray):
                slot.value = a.ptr
            elif isinstance(a, slice):
                for part_slot, part in zip(slot, (a.start, a.stop, a.step)):
                    part_slot.value = (_ParamList.SLICE_NONE if part is None
                                       else int(part))
            else:
                slot.value = a.item() if isinstance(a, np.generic) else a
        if ret is not None:
            self._ret_slot.value = ret.ptr
        for slot, part in zip(self._partial_slots, partials):
            slot.value = part.ptr

    def enqueue(self, args=None, ret=None):
        """Launches without waiting and returns the event (the caller passes
        it to ``retire``): back-to-back launches for timing."""
        if args is not None:
            # (run() is called with arguments its caller has already matched
            # to this plan; here they come from anywhere)
            if len(args) != len(self._key) or not all(
                    _fits(k, a) for k, a in zip(self._key, plan_key(args))):
                raise ValueError(
                    f"{self.func_name}: arguments differ in type, shape or strides from "
                    "those this launch was prepared for")
            if (ret is None) != (self._ret_key is None) or (
                    ret is not None and
                    not _fits(self._ret_key, (ret.dtype, ret.shape, ret.strides))):
                raise ValueError(
                    f"{self.func_name}: the result array must have dtype "
                    f"{self._ret_key[0] if self._ret_key else None} and the shape and strides "
                    "this launch was prepared for")
            arrays = [a for a in args if isinstance(a, HipNdArray)]
            if ret is not None:
                arrays.append(ret)
            if getattr(self.compiled, "noalias", False) and not disjoint(arrays):
                raise ValueError(
                    f"{self.func_name}: this launch was translated for arrays that do not "
                    "overlap; the arguments given do")
        with self._lock:                  # the launch call copies the values out
            if args is not None:
                self._refresh(args, ret, ())
            event = runtime_lib.gpuxLaunchKernel(*self._launch)
            self.ctx.pending.append(event)    # the context's synchronize() waits for it
            return event

    def retire(self, event):
        queue = self.ctx.queue
        runtime_lib.gpuxWait(queue, event)
        with self._lock:
            try:
                self.ctx.pending.remove(event)
            except ValueError:
                pass
        runtime_lib.gpuxDestroyEvent(queue, event)

    def run(self, args=None, ret=None, partials=()):
        """Launches; ``args`` (same types, shapes and strides as the plan was
        built for) refresh the pointer and scalar slots first."""
        if self.empty:
            return
        queue = self.ctx.queue
        with self._lock:                  # the launch call copies the values out
            if args is not None:
                self._refresh(args, ret, partials)
            event = runtime_lib.gpuxLaunchKernel(*self._launch)
        runtime_lib.gpuxWait(queue, event)
        runtime_lib.gpuxDestroyEvent(queue, event)
        flag = self._flag
        if flag is not None and flag.asnumpy()[0] != 0:
            flag.copy_from_host(np.zeros(1, np.int32))
            raise IndexError(
                f"kernel '{self.func_name}' indexed an array out of bounds (the access "
                "was redirected to element 0)")


def _dense_size(shape, strides, itemsize):
    """Element count of a C-contiguous array, None for any other layout."""
    expect = itemsize
    for n, st in zip(reversed(shape), reversed(strides)):
        if n != 1 and st != expect:
            return None
        expect *= n
    return expect // itemsize


def _fits(planned, given):
    """Whether an argument (its ``plan_key`` entry) can stand in for the one
    a launch was prepared with: the same entry, or -- the dispatchers prepare
    launches on arrays with their dimensions merged -- a dense array of the
    same type and size as a dense planned one."""
    if planned == given:
        return True
    if not (isinstance(planned, tuple) and isinstance(given, tuple)):
        return False
    (pd, ps, pst), (gd, gs, gst) = planned, given
    if pd != gd:
        return False
    size = _dense_size(ps, pst, pd.itemsize)
    return size is not None and size == _dense_size(gs, gst, gd.itemsize)


def plan_key(args):
    """What a launch plan depends on besides the kernel: per argument its
    type, and for arrays dtype, shape and strides (not the address)."""
    return tuple((a.dtype, a.shape, a.strides) if isinstance(a, HipNdArray)
                 else (a.dtype if isinstance(a, np.generic) else type(a))
                 for a in args)


def plan_compiled(ctx, compiled, func_name, global_size, args, ret=None,
                  make_partials=None):
    """Loads a translated function (once) and prepares its launch over
    ``global_size`` with a runtime-chosen block.  ``make_partials(blocks)``
    supplies the per-block result arrays of a function with reductions once
    the grid is known."""
    kern = _loaded_kernel(ctx, compiled)
    per_lane = getattr(compiled, "elements_per_thread", 1)
    lanes = [-(-int(global_size[0]) // per_lane)] + [int(g) for g in global_size[1:]]
    block, grid = _geometry(ctx, compiled, kern, lanes, ())
    if getattr(compiled, "grid_stride", False):
        # (a launch counts the work-items of a dimension in 32 bits; the
        # kernel strides over the rest)
        grid[0] = min(grid[0], (2 ** 32 - 1) // max(block[0], 1))
    if getattr(compiled, "grid_stride", False) and getattr(compiled, "stages_table", False) \
            and not make_partials and grid[0] >= 4096:
        # Every block stages its table before its first element: half the
        # blocks, two trips a lane (the Black-Scholes body over 2^24 options:
        # 8192 blocks against 16384), in whole groups of 128 blocks (the
        # kernel then takes its two trips 128 pieces apart).
        grid[0] = -(-grid[0] // 256) * 128
    if make_partials and getattr(compiled, "grid_stride", False):
        # a reduction: few, long-running blocks (one partial result each); the
        # more arrays they stream at once, the fewer (two arrays of 512 MiB:
        # 239 us on 1024 blocks, 264 on 2048; one array: 136 and 125)
        n_arrays = max(1, sum(isinstance(a, HipNdArray) for a in args))
        grid[0] = min(grid[0], max(REDUCTION_BLOCKS // n_arrays, 512))
    gsize3 = [int(g) for g in global_size] + [1] * (3 - len(global_size))
    partials = make_partials(grid[0] * grid[1] * grid[2]) if make_partials else ()
    return LaunchPlan(ctx, compiled, kern, func_name, grid, block, gsize3, args, ret,
                      partials)


def kernel(func=None, **kwargs):
    if func is None:

        def wrapper(f):
            return Kernel(f, kwargs)

        return wrapper
    return Kernel(func, kwargs)
