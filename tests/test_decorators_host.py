"""Host-side logic of ``njit`` that needs no GPU: which functions are taken as
one parallel loop."""

import numpy as np

from numba_mlir_amd import decorators
from numba_mlir_amd.decorators import njit, prange


def _by_name(x):
    s = 0.0
    for i in prange(x.shape[0]):
        s += x[i]
    return s


def _by_attribute(x):
    s = 0.0
    for i in decorators.prange(x.shape[0]):
        s += x[i]
    return s


def _nested_by_attribute(a):
    for h in decorators.prange(a.shape[0]):
        for w in decorators.prange(a.shape[1]):
            a[h, w] = h + w


def _sequential(x):
    s = 0.0
    for i in range(x.shape[0]):
        s += x[i]
    return s


def _unknown_callee(x):
    for i in np.nothing_of_that_name(3):
        pass


def test_prange_is_found_by_name_and_through_a_module():
    """``for i in prange(n)`` and ``for i in module.prange(n)`` are the same
    loop (the reference's users write ``numba.prange``)."""
    assert njit(parallel=True)(_by_name)._has_parallel_loop()
    assert njit(parallel=True)(_by_attribute)._has_parallel_loop()
    nested = njit(parallel=True)(_nested_by_attribute)
    assert nested._has_parallel_loop() and nested._grid_rank() == 2
    assert not njit(parallel=True)(_sequential)._has_parallel_loop()
    assert not njit(parallel=True)(_unknown_callee)._has_parallel_loop()


def _n_first(x):
    n = len(x)
    s = 0.0
    for i in range(1, n):
        s += x[i]
    return s


def _small_inner_loop(x, y):
    acc = x * 0.0
    for k in range(3):
        acc = acc * y + x
    return acc


def test_sequential_loops_over_an_array_are_refused_not_run_per_element():
    """Without prange such a loop is host code in the reference; as the loop
    of every work-item of a fused map it would be quadratic."""
    import pytest
    from numba_mlir_amd.mlir import kernel_compiler
    from numba_mlir_amd.mlir.device_array import HipNdArray
    x = HipNdArray.__new__(HipNdArray)          # (only its type is looked at)
    for func in (_sequential, _n_first):
        with pytest.raises(kernel_compiler.KernelCompileError, match="write it with prange"):
            njit(func)._refuse_sequential_array_loops([x])
    njit(_small_inner_loop)._refuse_sequential_array_loops([x, x])
    njit(_by_name)._refuse_sequential_array_loops([x])      # (prange is not range)


def test_stage_kernels_of_a_lambda_get_identifier_names():
    f = njit(lambda a: np.sum(a * a, axis=1))
    assert f._stage_stem == "lambda" and njit(_by_name)._stage_stem == "_by_name"


def test_arrays_built_and_sliced_become_stages_of_their_own():
    """np.concatenate / tril / outer / arange and basic indexing of a local
    array split a straight-line body: array arguments become operands
    (expressions materialised by a map first), the rest stays host
    expressions."""
    import ast

    from numba_mlir_amd.mlir import staging

    src = ("def f(a, b):\n"
           "    c = np.concatenate((a, b + 1), axis=0)\n"
           "    d = np.tril(c[1:5], -1)\n"
           "    e = c[2] + d[0, 0]\n"
           "    return np.outer(a, b).copy() + np.arange(3) + a.shape[0]\n")
    plan = staging.plan_of(ast.parse(src).body[0], lambda name: name == "np")
    kinds = [(st.kind, st.op) for st in plan.stages if st.kind in ("make", "view")]
    assert kinds == [("make", "concatenate"), ("view", "getitem"), ("make", "tril"),
                     ("view", "getitem"), ("view", "getitem"), ("make", "outer"),
                     ("view", "copy"), ("make", "arange"), ("view", "shape"),
                     ("view", "getitem")]
    concatenate = next(st for st in plan.stages if st.op == "concatenate")
    assert concatenate.operands[0] == "a" and concatenate.operands[1].startswith("_nmk_t")
    assert [key for key, _ in concatenate.args[2]] == ["axis"]
    tril = next(st for st in plan.stages if st.op == "tril")
    assert tril.args[1] == [0, None]          # the array, then k on the host
    # a.shape[0] is read from the array on the host, not inside the map (where
    # the array is a view with its dimensions merged)
    assert "shape" not in ast.unparse(plan.stages[-1].expr)


def test_stores_into_slices_are_stores_into_views():
    import ast

    from numba_mlir_amd.mlir import staging

    src = ("def f(a, b):\n"
           "    a[1:-1, 2:5] = b[:-2, :3] * 2.0\n"
           "    a[0, :] -= len(b)\n")
    plan = staging.plan_of(ast.parse(src).body[0], lambda name: name == "np")
    kinds = [(st.kind, st.op) for st in plan.stages]
    assert kinds == [("view", "getitem"), ("view", "getitem"), ("store", None),
                     ("view", "getitem"), ("view", "len"), ("view", "getitem"),
                     ("store", None)]
    # each store goes into the view made just before it
    assert plan.stages[2].target == plan.stages[1].target
    assert plan.stages[6].target == plan.stages[5].target
