"""TEST INFRASTRUCTURE -- not part of the product.

Work-item by work-item executor for ``@kernel`` bodies: the oracle the
reference itself uses for every GPU kernel test (its ``kernel_sim``).

Restates the launch semantics of the reference's simulator
(reference: numba_mlir/numba_mlir/mlir/kernel_sim_impl.py:171-234):

* a missing local size means all-ones (196-197);
* work-groups are visited in row-major order of their ids, work-items of a
  group in row-major order of their global ids (203-229);
* groups on the upper edge are clipped to the global size (206-208);
* ``get_local_id = global_id % local_size``, ``get_group_id = global_id //
  local_size`` (175-182).

Barriers, local arrays and group reductions are not simulated (the hot path
uses none).  The index builtins are looked up through ``builtins`` passed to
the body's globals for the duration of the call.
"""

from itertools import product


class _State:
    def __init__(self, global_size, local_size):
        self.global_size = tuple(global_size)
        self.local_size = tuple(local_size)
        self.indices = [0] * len(global_size)


class KernelSim:
    BUILTINS = ("get_global_id", "get_local_id", "get_group_id",
                "get_global_size", "get_local_size")

    def __init__(self, func):
        self.py_func = func
        self.global_size = ()
        self.local_size = ()

    def __getitem__(self, args):
        if not isinstance(args, tuple):
            args = (args,)
        gs = args[0]
        gs = (gs,) if isinstance(gs, int) else tuple(gs)
        ls = args[1] if len(args) > 1 else ()
        ls = (ls,) if isinstance(ls, int) else tuple(ls)
        if len(ls) != 0 and len(ls) < len(gs):
            ls = ls + (1,) * (len(gs) - len(ls))
        sim = KernelSim(self.py_func)
        sim.global_size, sim.local_size = gs, ls
        return sim

    def __call__(self, *args):
        global_size = self.global_size
        local_size = self.local_size
        if len(local_size) == 0:
            local_size = (1,) * len(global_size)
        state = _State(global_size, local_size)

        impl = {
            "get_global_id": lambda k: state.indices[k],
            "get_local_id": lambda k: state.indices[k] % state.local_size[k],
            "get_group_id": lambda k: state.indices[k] // state.local_size[k],
            "get_global_size": lambda k: state.global_size[k],
            "get_local_size": lambda k: state.local_size[k],
        }
        g = self.py_func.__globals__
        saved = {name: g[name] for name in self.BUILTINS if name in g}
        g.update(impl)
        try:
            groups = tuple((gs + ls - 1) // ls
                           for gs, ls in zip(global_size, local_size))
            for gid in product(*(range(n) for n in groups)):
                offset = tuple(i * l for i, l in zip(gid, local_size))
                size = tuple(min(gs - o, l)
                             for o, gs, l in zip(offset, global_size, local_size))
                for indices in product(*(range(o, o + s)
                                         for o, s in zip(offset, size))):
                    state.indices[:] = indices
                    self.py_func(*args)
        finally:
            for name in self.BUILTINS:
                if name in saved:
                    g[name] = saved[name]
                else:
                    g.pop(name, None)


def kernel_sim(func):
    return KernelSim(func)
