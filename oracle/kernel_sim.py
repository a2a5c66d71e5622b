"""TEST INFRASTRUCTURE -- not part of the product.

Work-item by work-item executor for ``@kernel`` bodies: the oracle the
reference itself uses for every GPU kernel test (its ``kernel_sim``).

Restates the launch semantics of the reference's simulator
(reference: numba_mlir/numba_mlir/mlir/kernel_sim_impl.py:37-234,
numba_mlir/numba_mlir/mlir/kernel_sim.py):

* a missing local size means all-ones (kernel_sim_impl.py:196-197);
* work-groups are visited in row-major order of their ids, work-items of a
  group in row-major order of their global ids (203-229);
* groups on the upper edge are clipped to the global size (206-208);
* ``get_local_id = global_id % local_size``, ``get_group_id = global_id //
  local_size`` (175-182);
* ``barrier``: every work-item of a group is a greenlet; a barrier switches to
  the next one round-robin (62-73, 214-225); ``mem_fence`` is a no-op;
* ``local.array``: allocated (zeroed) by the first work-item of the group to
  reach the call site, shared by the others in call order (155-164);
  ``private.array``: a fresh zeroed array per call (167-168);
* ``group.reduce_*``: item 0 stores its value, later items fold theirs in
  item order, then a barrier; everyone reads the total (76-82);
* ``atomic.add/sub``: plain ``arr[idx] += val`` / ``-= val`` (items run one at a
  time).

The kernel-only names are patched into the body's globals and closure cells
for the duration of a launch (108-136, 199-233): any global or cell whose
value is one of the stub objects passed as ``stubs`` is replaced by the
simulator's implementation.
"""

from functools import reduce as _reduce
from itertools import product

import numpy as np

try:
    from greenlet import greenlet
    _HAVE_GREENLET = True
except ImportError:      # pragma: no cover
    _HAVE_GREENLET = False


class _State:
    def __init__(self, global_size, local_size):
        self.global_size = tuple(global_size)
        self.local_size = tuple(local_size)
        self.indices = [0] * len(global_size)
        self.wg_size = 1
        self.tasks = []
        self.current_task = 0
        self.local_arrays = []
        self.current_local_array = 0
        self.reduce_val = None


class KernelSim:
    NAMES = ("get_global_id", "get_local_id", "get_group_id", "get_global_size",
             "get_local_size", "barrier", "mem_fence", "atomic_add",
             "atomic_sub", "local_array", "private_array", "group_reduce_add",
             "group_reduce_mul", "group_reduce_min", "group_reduce_max")

    def __init__(self, func, stubs=None):
        self.py_func = func
        self.stubs = stubs
        self.global_size = ()
        self.local_size = ()

    def __getitem__(self, args):
        if not isinstance(args, tuple):
            args = (args,)
        gs = args[0]
        gs = (gs,) if isinstance(gs, (int, np.integer)) else tuple(gs)
        ls = args[1] if len(args) > 1 else ()
        ls = (ls,) if isinstance(ls, (int, np.integer)) else tuple(ls)
        if len(ls) != 0 and len(ls) < len(gs):
            ls = ls + (1,) * (len(gs) - len(ls))
        sim = KernelSim(self.py_func, self.stubs)
        sim.global_size, sim.local_size = gs, ls
        return sim

    # -- implementations ------------------------------------------------------
    def _impl(self, state):
        def barrier_impl(flags=None):
            if state.wg_size > 1:
                saved = (list(state.indices), state.current_local_array)
                state.current_local_array = 0
                nxt = state.current_task + 1
                if nxt >= state.wg_size:
                    nxt = 0
                state.current_task = nxt
                state.tasks[nxt].switch()
                state.indices[:] = saved[0]
                state.current_local_array = saved[1]

        def group_reduce(op):
            def impl(value):
                if state.current_task == 0:
                    state.reduce_val = value
                else:
                    state.reduce_val = op(state.reduce_val, value)
                barrier_impl()
                return state.reduce_val
            return impl

        def local_array(shape, dtype):
            cur = state.current_local_array
            if state.current_task == 0:
                arr = np.zeros(shape, dtype)
                state.local_arrays.append(arr)
            else:
                arr = state.local_arrays[cur]
            state.current_local_array = cur + 1
            return arr

        def atomic_add(arr, idx, val):
            arr[idx] += val

        def atomic_sub(arr, idx, val):
            arr[idx] -= val

        return {
            "get_global_id": lambda k: state.indices[k],
            "get_local_id": lambda k: state.indices[k] % state.local_size[k],
            "get_group_id": lambda k: state.indices[k] // state.local_size[k],
            "get_global_size": lambda k: state.global_size[k],
            "get_local_size": lambda k: state.local_size[k],
            "barrier": barrier_impl,
            "mem_fence": lambda flags=None: None,
            "atomic_add": atomic_add,
            "atomic_sub": atomic_sub,
            "local_array": local_array,
            "private_array": lambda shape, dtype: np.zeros(shape, dtype),
            "group_reduce_add": group_reduce(lambda a, b: a + b),
            "group_reduce_mul": group_reduce(lambda a, b: a * b),
            "group_reduce_min": group_reduce(lambda a, b: min(a, b)),
            "group_reduce_max": group_reduce(lambda a, b: max(a, b)),
        }

    def _replacements(self, impl):
        """Maps stub objects (by identity) and stub names to implementations."""
        by_obj = {}
        if self.stubs is not None:
            for name in self.NAMES:
                obj = self.stubs.get(name)
                if obj is not None:
                    by_obj[id(obj)] = impl[name]
        return by_obj

    def __call__(self, *args, need_barrier=True):
        global_size = self.global_size
        local_size = self.local_size
        if len(local_size) == 0:
            local_size = (1,) * len(global_size)
        state = _State(global_size, local_size)
        impl = self._impl(state)
        by_obj = self._replacements(impl)

        func = self.py_func
        g = func.__globals__
        saved_globals = {}
        for name, val in list(g.items()):
            if id(val) in by_obj:
                saved_globals[name] = val
                g[name] = by_obj[id(val)]
            elif self.stubs is None and name in impl and callable(val):
                saved_globals[name] = val
                g[name] = impl[name]
        saved_cells = []
        for cell in (func.__closure__ or ()):
            try:
                val = cell.cell_contents
            except ValueError:
                continue
            if id(val) in by_obj:
                saved_cells.append((cell, val))
                cell.cell_contents = by_obj[id(val)]
        try:
            groups = tuple((gs + ls - 1) // ls
                           for gs, ls in zip(global_size, local_size))
            for gid in product(*(range(n) for n in groups)):
                offset = tuple(i * l for i, l in zip(gid, local_size))
                size = tuple(min(gs - o, l)
                             for o, gs, l in zip(offset, global_size, local_size))
                count = _reduce(lambda a, b: a * b, size)
                state.wg_size = count
                state.current_task = 0
                state.local_arrays = []
                state.current_local_array = 0
                items = list(product(*(range(o, o + s)
                                       for o, s in zip(offset, size))))
                if need_barrier and _HAVE_GREENLET:
                    def make(indices):
                        def run():
                            state.indices[:] = indices
                            func(*args)
                        return run
                    state.tasks = [greenlet(make(idx)) for idx in items]
                    for t in state.tasks:
                        t.switch()
                    state.tasks = []
                else:
                    for indices in items:
                        state.indices[:] = indices
                        func(*args)
        finally:
            for cell, val in saved_cells:
                cell.cell_contents = val
            g.update(saved_globals)


def kernel_sim(func, stubs=None):
    """``stubs``: dict name -> stub object to replace (by identity) wherever
    the body refers to it (module globals or closure cells); without it, module
    globals named like the index builtins are replaced by name."""
    return KernelSim(func, stubs)
