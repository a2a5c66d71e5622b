"""Launch-geometry front of a ``@kernel`` object: ``kern[global, local](*args)``.

Behaviour kept from the reference's launch wrapper
(reference: numba_mlir/numba_mlir/mlir/kernel_base.py:33-58):

* the subscript takes one or two items, ``kern[global]`` or
  ``kern[global, local]``;
* each item is an int (a 1-d launch) or a list/tuple of one to three ints;
* the global size is the iteration space, not a number of blocks;
* a local size with fewer entries than the global size is filled up with
  ones, an empty local size leaves the block shape to the runtime;
* subscripting returns a configured copy, the decorated object itself is
  never modified, so ``kern[a]`` and ``kern[b]`` can be kept side by side;
* keyword arguments in the call are refused.

Every misuse is a ``ValueError``.
"""

MAX_LAUNCH_RANK = 3


class LaunchGeometryError(ValueError):
    """Wrong subscript or call form of a kernel object."""


def as_extent_tuple(item, what):
    """An int or a sequence of up to three ints, as a tuple."""
    if isinstance(item, bool):
        raise LaunchGeometryError(f"{what} size must be an int or a tuple of ints, "
                                  f"got a bool")
    if isinstance(item, int):
        return (item,)
    if not isinstance(item, (tuple, list)):
        raise LaunchGeometryError(
            f"{what} size must be an int or a tuple of ints, got "
            f"{type(item).__name__}")
    if len(item) > MAX_LAUNCH_RANK:
        raise LaunchGeometryError(
            f"{what} size has {len(item)} entries, a launch has at most "
            f"{MAX_LAUNCH_RANK} dimensions")
    return tuple(item)


class KernelBase:
    """Holds the Python function and one launch geometry."""

    def __init__(self, func):
        self.py_func = func
        self.global_size = ()
        self.local_size = ()

    def copy(self):
        twin = object.__new__(type(self))
        twin.__dict__.update(self.__dict__)
        return twin

    def configure(self, global_size, local_size):
        """A copy of this kernel bound to ``global_size`` / ``local_size``."""
        global_size = tuple(global_size)
        local_size = tuple(local_size)
        missing = len(global_size) - len(local_size)
        if missing < 0:
            raise LaunchGeometryError(
                f"local size {local_size} has more dimensions than global size "
                f"{global_size}")
        if local_size:
            local_size += (1,) * missing
        bound = self.copy()
        bound.global_size = global_size
        bound.local_size = local_size
        return bound

    def check_call_args(self, args, kwargs):
        if kwargs:
            names = ", ".join(sorted(kwargs))
            raise LaunchGeometryError(
                f"a kernel takes positional arguments only (got {names})")

    def __getitem__(self, geometry):
        items = geometry if isinstance(geometry, tuple) else (geometry,)
        if len(items) == 1:
            return self.configure(as_extent_tuple(items[0], "global"), ())
        if len(items) == 2:
            return self.configure(as_extent_tuple(items[0], "global"),
                                  as_extent_tuple(items[1], "local"))
        raise LaunchGeometryError(
            f"expected kern[global_size] or kern[global_size, local_size], got "
            f"{len(items)} items")
