"""``njit`` / ``vectorize`` / ``prange`` for functions over device arrays.

In the reference ``@njit`` hands the function to Numba and the MLIR pipeline,
which fuses whole-array expressions into parallel loops and offloads them
(reference: numba_mlir/numba_mlir/decorators.py:24-120; the fused
Black-Scholes test, numba_mlir/numba_mlir/mlir/tests/test_numpy.py:2796-2866).
Here a call is served in one of three ways, tried in this order:

1. *library lowering*: a function whose body is one ``return`` of a map,
   reduction or contraction the hand-written kernels cover -- ``a + b``
   (also ``-``, ``*``) with broadcasting, ``np.sum/prod/min/max(x[, axis])``,
   ``np.sqrt(np.sum(x * x))``, ``np.dot(a, b)`` / ``a @ b`` -- goes to that
   kernel, which is what the linalg lowering does with these patterns;
2. *one parallel loop*: assignments followed by a single top-level
   ``for i in prange(...)`` become one kernel, one work-item per iteration;
   scalars the loop only updates with ``+=`` / ``*=`` are reductions (lanes,
   blocks, then the host fold their shares) and may be returned;
3. *elementwise fusion*: any other function built from whole-array
   arithmetic, ``math``/``numpy`` scalar functions, ``vectorize``d functions and
   ``out[:] = ...`` stores becomes one fused kernel over the broadcast shape.

Anything else (scalar indexing outside a loop, reductions mixed with maps,
several loops) is reported as unsupported rather than run on the host.
NumPy arguments are copied to the device for the call and back afterwards.
"""

import ast
import functools
import inspect
import math
import re

import numpy as np

from .mlir import device_array as hip
from .mlir import kernel_compiler, kernel_impl, ops, staging
from .mlir.device_array import HipNdArray
from .mlir.utils import readenv


def prange(*args):
    """``range`` on the host; the grid of the offloaded loop under ``njit``."""
    return range(*args)


prange._nmk_prange = True


class _Vectorized:
    """A scalar function applied elementwise (reference:
    numba_mlir/numba_mlir/mlir/vectorize.py:16-20).  Inside ``njit`` functions
    it is inlined as a device function; called directly it maps over NumPy
    arrays on the host."""

    def __init__(self, func):
        self.py_func = self._nmk_vectorized = func
        functools.update_wrapper(self, func)

    def __call__(self, *args):
        return np.vectorize(self.py_func)(*args)


def vectorize(arg_or_function=(), **kws):
    if inspect.isfunction(arg_or_function):
        return _Vectorized(arg_or_function)
    return _Vectorized


ELEMENTS_PER_THREAD = 4     # of a fused 1-d map or prange loop
MAX_PLANS = kernel_impl.MAX_PLANS   # stored launches per compiled function


_BINARY = {ast.Add: ops.add, ast.Sub: ops.subtract, ast.Mult: ops.multiply,
           ast.Div: ops.divide}
_REDUCE = {"sum": ops.sum, "prod": ops.prod, "min": ops.amin, "max": ops.amax,
           "amin": ops.amin, "amax": ops.amax}


def _collapse(shape, views):
    """Merges adjacent dimensions of an iteration space that every array
    walks with one stride (a dimension's stride equals the next one's stride
    times its extent; broadcast dimensions, stride 0, merge with each other)
    and drops dimensions of extent 1.  Returns the new shape and the views."""
    arrays = [v for v in views if isinstance(v, HipNdArray)]
    if 0 in shape or not shape:
        return tuple(shape), views
    dims = [(n, [a.strides[d] for a in arrays]) for d, n in enumerate(shape) if n != 1]
    if not dims:
        dims = [(1, [0] * len(arrays))]
    merged = [dims[0]]
    for n, strides in dims[1:]:
        before_n, before = merged[-1]
        if all(b == s * n for b, s in zip(before, strides)):
            merged[-1] = (before_n * n, strides)
        else:
            merged.append((n, strides))
    new_shape = tuple(n for n, _ in merged)
    out, k = [], 0
    for v in views:
        if isinstance(v, HipNdArray):
            strides = tuple(st[k] for _, st in merged)
            out.append(HipNdArray(v._buffer, new_shape, v.dtype, strides, v._offset))
            k += 1
        else:
            out.append(v)
    return new_shape, out


def _reduce_nd(op, x, axis):
    """A reduction kernel applied to a dense array of any rank along its first
    or last axis (or all of it), through a 2-d view.  Booleans are counted as
    integers, as NumPy does."""
    if x.dtype == np.bool_:
        x = _CAST_TO[np.int64](x)
    if x.dtype in _NARROW_INTEGERS:
        return _reduce_narrow(op, x, axis)
    if axis is None and not (x.is_c_contiguous() or x.is_f_contiguous()):
        x = _copy(x)                      # a strided view: its elements, densely
    if x.ndim <= 2 or not x.is_c_contiguous():
        return op(x, axis=axis)
    if axis is None:
        return op(x.reshape((x.size,)), axis=None)
    axis = axis + x.ndim if axis < 0 else axis
    if axis == 0:
        return op(x.reshape((x.shape[0], x.size // max(x.shape[0], 1))),
                  axis=0).reshape(x.shape[1:])
    if axis == x.ndim - 1:
        return op(x.reshape((x.size // max(x.shape[-1], 1), x.shape[-1])),
                  axis=1).reshape(x.shape[:-1])
    raise NotImplementedError("reductions of arrays of rank > 2 run along the first or "
                              "the last axis")


# Integer types the reduction kernels do not take as they are: widened to
# int64 (every value fits) and reduced there.
_NARROW_INTEGERS = tuple(np.dtype(t) for t in (np.int8, np.int16, np.uint8, np.uint16, np.uint32))


def _reduce_narrow(op, x, axis):
    """Sums and products come back in the type NumPy gives them along an axis
    (int64, uint64 for unsigned input) and, like the other integer types
    here, in the input's own type over everything (the reference casts a full
    reduction back, numpy/funcs.py:163-229); minima and maxima in the input's
    type."""
    result = _reduce_nd(op, _astype(x, np.dtype(np.int64)), axis)
    if op in (ops.amin, ops.amax) or axis is None:
        back = x.dtype
    else:
        back = np.dtype(np.uint64 if x.dtype.kind == "u" else np.int64)
    if isinstance(result, HipNdArray):
        return result if result.dtype == back else _astype(result, back)
    return np.asarray(result).astype(back)[()]


_DIVIDE = []
_FILL = []


def _to_float32(x):
    return np.float32(x)


def _to_float64(x):
    return np.float64(x)


def _to_int64(x):
    return np.int64(x)


def _mean_float32(total, count):
    return np.float32(total / count)


def _mean_float64(total, count):
    return np.float64(total / count)


class _Lazy(dict):
    """type -> Dispatcher of the helper above, made on first use."""

    def __init__(self, helpers):
        super().__init__()
        self._helpers = helpers

    def __missing__(self, key):
        if key not in self._helpers:
            raise kernel_compiler.KernelCompileError(f"No conversion to {key.__name__}")
        self[key] = Dispatcher(self._helpers[key])
        return self[key]


_CAST_TO = _Lazy({np.float32: _to_float32, np.float64: _to_float64, np.int64: _to_int64})
_DIVIDE_TO = _Lazy({np.float32: _mean_float32, np.float64: _mean_float64})


def _fill_body(a, value):
    a[:] = value


def _fill(array, value):
    if not _FILL:
        _FILL.append(Dispatcher(_fill_body))
    _FILL[0]._run([array, value])



def _span(x):
    lo = hi = x._offset
    for n, st in zip(x.shape, x.strides):
        if n > 1:
            lo += min(0, (n - 1) * st)
            hi += max(0, (n - 1) * st)
    return lo, hi


def _overlaps(x, target):
    """Whether x may share elements with target without being the same view
    (the same view is read and written element by element, which is safe)."""
    if x._buffer is not target._buffer or not x.size or not target.size:
        return False
    if x._offset == target._offset and x.shape == target.shape and x.strides == target.strides:
        return False
    (lo, hi), (tlo, thi) = _span(x), _span(target)
    return lo <= thi and tlo <= hi


def _copy(x):
    """A dense C-ordered copy on x's device (numpy/funcs.py:255-262)."""
    out = HipNdArray.empty(x.shape, x.dtype, device=x.ctx.device)
    if out.size:
        _fill(out, x)
    return out


_CASTS = {}


def _astype(x, dtype):
    """x converted element by element into a new dense array."""
    if dtype == x.dtype:
        return _copy(x)
    name = dtype.name
    if dtype.kind not in "iuf" or not hasattr(np, name):
        raise NotImplementedError(f"conversion to {name} is not implemented")
    if name not in _CASTS:
        source = f"def _to_{name}(x):\n    return np.{name}(x)\n"
        scope = {"np": np}
        exec(source, scope)                                   # noqa: S102
        func = scope[f"_to_{name}"]
        func.__nmk_ast__ = ast.parse(source).body[0]
        _CASTS[name] = func
    return _CAST_TO_ANY[_CASTS[name]]._run([x])


def _arange_body(out, start, step):
    i = kernel_impl.get_global_id(0)
    out[i] = start + i * step


def _eye_body(out, k):
    i = kernel_impl.get_global_id(0)
    j = kernel_impl.get_global_id(1)
    out[i, j] = 1 if j - i == k else 0


def _tril_body(a, out, k):
    i = kernel_impl.get_global_id(0)
    j = kernel_impl.get_global_id(1)
    out[i, j] = a[i, j] if j - i <= k else 0


def _triu_body(a, out, k):
    i = kernel_impl.get_global_id(0)
    j = kernel_impl.get_global_id(1)
    out[i, j] = a[i, j] if j - i >= k else 0


def _outer_body(a, b):
    return a * b


def _center_body(x, mean):
    return x - mean


def _scale_body(x, factor):
    return x * factor


class _LazyKernels(dict):
    def __missing__(self, body):
        self[body] = kernel_impl.kernel(body)
        return self[body]


class _LazyFunctions(dict):
    def __missing__(self, body):
        self[body] = Dispatcher(body)
        return self[body]


_KERNELS = _LazyKernels()
_FUNCTIONS = _LazyFunctions()
_CAST_TO_ANY = _LazyFunctions()


def _arange(ctx, *args, dtype=None):
    """numpy.arange on the device (numpy/funcs.py:642-668): the same length
    and type as NumPy gives, element i = start + i step."""
    if not 1 <= len(args) <= 3:
        raise TypeError("arange takes start, stop and step")
    if len(args) == 1:
        start, stop, step = 0, args[0], 1
    else:
        start, stop, step = args[0], args[1], args[2] if len(args) == 3 else 1
    if step == 0:
        raise ValueError("Maximum allowed size exceeded")
    if dtype is None:
        whole = all(isinstance(v, (int, np.integer)) for v in (start, stop, step))
        dtype = np.int64 if whole else np.float64
    dtype = np.dtype(dtype)
    count = max(0, int(math.ceil((stop - start) / step)))
    out = HipNdArray.empty((count,), dtype, device=ctx.device)
    if count:
        _KERNELS[_arange_body][(count,), ()](out, dtype.type(start), dtype.type(step))
    return out


def _eye(ctx, n, m=None, k=0, dtype=np.float64):
    """numpy.eye (numpy/funcs.py:670-700)."""
    m = n if m is None else m
    out = HipNdArray.empty((int(n), int(m)), dtype, device=ctx.device)
    if out.size:
        _KERNELS[_eye_body][(int(n), int(m)), ()](out, int(k))
    return out


def _tri(x, k, lower):
    """numpy.tril / triu of a matrix."""
    if x.ndim != 2:
        raise NotImplementedError("tril and triu are implemented for matrices")
    out = HipNdArray.empty(x.shape, x.dtype, device=x.ctx.device)
    if out.size:
        _KERNELS[_tril_body if lower else _triu_body][x.shape, ()](x, out, int(k))
    return out


def _outer(a, b):
    """numpy.outer: the operands flattened, one fused map over the product's shape."""
    a = a if a.ndim == 1 else _copy(a).reshape((a.size,))
    b = b if b.ndim == 1 else _copy(b).reshape((b.size,))
    return _FUNCTIONS[_outer_body]._run([a.reshape((a.size, 1)), b.reshape((1, b.size))])


def _concatenate(arrays, axis=0):
    """numpy.concatenate: one strided store per piece into the new array."""
    if not arrays:
        raise ValueError("need at least one array to concatenate")
    first = arrays[0]
    if not -first.ndim <= axis < first.ndim:
        raise ValueError(f"axis {axis} is out of bounds for array of dimension {first.ndim}")
    axis %= first.ndim
    for a in arrays[1:]:
        if a.ndim != first.ndim or \
                any(p != q for d, (p, q) in enumerate(zip(a.shape, first.shape)) if d != axis):
            raise ValueError("all the input array dimensions except for the concatenation "
                             "axis must match exactly")
    shape = list(first.shape)
    shape[axis] = sum(a.shape[axis] for a in arrays)
    out = HipNdArray.empty(tuple(shape), np.result_type(*[a.dtype for a in arrays]),
                           device=first.ctx.device)
    at = 0
    for a in arrays:
        if a.size:
            where = tuple(slice(at, at + a.shape[axis]) if d == axis else slice(None)
                          for d in range(first.ndim))
            _fill(out[where], a)
        at += a.shape[axis]
    return out


def _cov(m, y=None, rowvar=True, bias=False, ddof=None):
    """numpy.cov as the reference builds it (numpy/funcs.py:1455-1549): rows
    are variables; the result keeps a floating input's type (integers become
    float64); a single 1-d input gives a scalar."""
    scalar = m.ndim == 1 and y is None
    rows = []
    for x in (m, y):
        if x is None:
            continue
        if x.ndim > 2:
            raise ValueError("m has more than 2 dimensions")
        x = x.reshape((1, x.size)) if x.ndim < 2 else x
        if not rowvar and (y is None or x.shape[0] != 1):
            x = x.T
        rows.append(x)
    dtype = np.result_type(*[x.dtype for x in rows])
    if dtype.kind != "f":
        dtype = np.dtype(np.float64)
    rows = [x if x.dtype == dtype else _CAST_TO[dtype.type]._run([x]) for x in rows]
    X = rows[0] if len(rows) == 1 else _concatenate(rows, 0)
    if ddof is None:
        ddof = 0 if bias else 1
    fact = max(X.shape[1] - ddof, 0.0)
    mean = _mean(X, 1)
    centered = _FUNCTIONS[_center_body]._run([X, mean.reshape((X.shape[0], 1))])
    c = _dot(centered, centered.T)
    with np.errstate(divide="ignore"):
        c = _FUNCTIONS[_scale_body]._run([c, dtype.type(np.true_divide(1, fact))])
    return c.asnumpy()[0, 0] if scalar else c


def _mean(x, axis):
    if x.dtype in _NARROW_INTEGERS:
        x = _astype(x, np.dtype(np.int64))        # (no wrap-round of the total)
    total = _reduce_nd(ops.sum, x, axis)
    float_t = x.dtype.type if x.dtype.kind == "f" else np.float64
    if axis is None:
        if isinstance(total, HipNdArray):
            total = total.asnumpy().reshape(-1)[0]
        return float_t(float_t(total) / float_t(x.size))
    if not _DIVIDE:
        _DIVIDE.append(Dispatcher(lambda s, n: s / n))
    return _DIVIDE[0](total, float_t(x.shape[axis]))


def _matmul_body(a, b, out):
    i = kernel_impl.get_global_id(0)
    j = kernel_impl.get_global_id(1)
    acc = out[i, j] * 0
    for k in range(a.shape[1]):
        acc += a[i, k] * b[k, j]
    out[i, j] = acc


def _matmul(a, b, out=None):
    """The product of two matrices: the gemm kernels for float32 and float64
    (operands of two types are converted to their common type first), a plain
    generated kernel, one work-item per element, for integers (the reference
    lowers those to linalg.matmul, numpy/funcs.py:889-906)."""
    dtype = np.result_type(a.dtype, b.dtype)
    if dtype == np.bool_:
        dtype = np.dtype(np.int64)
    if dtype.kind == "f" and dtype.itemsize < 4:
        dtype = np.dtype(np.float32)
    if dtype.kind not in "iuf":
        raise TypeError(f"no matrix product of {a.dtype} and {b.dtype}")
    if out is not None and out.dtype != dtype:
        raise TypeError(f"out must be of type {dtype}")
    a = a if a.dtype == dtype else _astype(a, dtype)
    b = b if b.dtype == dtype else _astype(b, dtype)
    if dtype in (np.float32, np.float64):
        return ops.dot(a, b, out=out)
    if dtype.kind == "u" and dtype.itemsize == 8:
        raise TypeError("no matrix product of uint64")
    if a.shape[1] != b.shape[0]:
        raise ValueError(f"shapes {a.shape} and {b.shape} not aligned")
    if out is None:
        out = HipNdArray.empty((a.shape[0], b.shape[1]), dtype, device=a.ctx.device)
    if out.size:
        _fill(out, dtype.type(0))
        if a.shape[1]:
            _KERNELS[_matmul_body][out.shape, ()](a, b, out)
    return out


def _dot(a, b, out=None):
    """numpy.dot of device arrays of rank 1 or 2 through the matrix kernels."""
    if not (isinstance(a, HipNdArray) and isinstance(b, HipNdArray)):
        raise TypeError("both operands must be device arrays")
    if a.ndim == 2 and b.ndim == 2:
        if out is not None and (not isinstance(out, HipNdArray) or
                                out.shape != (a.shape[0], b.shape[1])):
            raise ValueError("out must be a device array of the product's shape")
        return _matmul(a, b, out=out)
    if out is not None:
        raise NotImplementedError("out= is implemented for 2-d operands")
    if a.ndim == 1 and b.ndim == 1:
        if a.shape != b.shape:
            raise ValueError(f"shapes {a.shape} and {b.shape} do not match")
        total = ops.sum(ops.multiply(a, b))
        return total.asnumpy().reshape(-1)[0] if isinstance(total, HipNdArray) else total
    if a.ndim == 2 and b.ndim == 1:
        return _matmul(a, b.reshape((b.shape[0], 1))).reshape((a.shape[0],))
    if a.ndim == 1 and b.ndim == 2:
        return _matmul(a.reshape((1, a.shape[0])), b).reshape((b.shape[1],))
    raise NotImplementedError("np.dot is implemented for rank 1 and 2")


class Dispatcher:
    def __init__(self, py_func, parallel=False, boundscheck=None, **options):
        self.py_func = py_func
        # inside another compiled function or kernel a call of this one is
        # inlined as a device function of its scalar arguments
        self._nmk_vectorized = py_func
        self.parallel = parallel
        if boundscheck is None:
            boundscheck = readenv("NUMBA_MLIR_KERNEL_BOUNDSCHECK", int, 0)
        self.boundscheck = bool(boundscheck)
        self.options = options
        self.last_launch = None          # what served the most recent call
        self.last_plan = None            # its LaunchPlan, for a generated kernel
        self._compiled = {}
        self._plans = {}
        self._loop_plans = {}
        self._stage_plan = None        # (staging.Plan or None,) once analysed
        self._stage_funcs = {}         # (stage index, captured constants) -> Dispatcher
        try:
            node = kernel_compiler._function_ast(py_func)
        except kernel_compiler.KernelCompileError:
            node = None
        self._node = node
        self._names = None             # what the body's free names are bound to
        self._parallel_loop = None     # whether the body has a top-level prange loop
        self._library_form = None      # the one-expression pattern, parsed once
        self._rank = None              # grid dimensions of the prange nest
        self._asked = None             # parameters whose shape or elements the body reads
        functools.update_wrapper(self, py_func)

    # -- entry ---------------------------------------------------------------
    def __call__(self, *args, **kwargs):
        if kwargs:
            raise ValueError("kwargs not supported")
        host = [isinstance(a, np.ndarray) for a in args]
        if any(host):
            dev = [hip.asarray(a) if h else a for a, h in zip(args, host)]
            result = self._run(dev)
            for a, d, h in zip(args, dev, host):
                if h and a.flags.writeable:
                    a[...] = d.asnumpy()
            return result.asnumpy() if isinstance(result, HipNdArray) else result
        return self._run(list(args))

    def _run(self, args):
        if self._node is None:
            raise kernel_compiler.KernelCompileError(
                f"No source available for {self.py_func!r}")
        served = self._library(args)
        if served is not NotImplemented:
            return served
        if self._has_parallel_loop():
            return self._parallel(args)
        plan = self._plan()
        if plan is not None:
            return self._staged(plan, args)
        return self._elementwise(args)

    # -- 1. library lowering -------------------------------------------------
    def _params(self):
        return [a.arg for a in self._node.args.args]

    def _single_expression(self):
        """The expression of a body that is one ``return``, else None."""
        if self._library_form is None:
            body = self._node.body
            expr = body if isinstance(self._node, ast.Lambda) else None
            if expr is None:
                stmts = [s for s in body if not (isinstance(s, ast.Expr) and
                                                 isinstance(s.value, ast.Constant))]
                if len(stmts) == 1 and isinstance(stmts[0], ast.Return) and \
                        stmts[0].value is not None:
                    expr = stmts[0].value
            shapes = (ast.BinOp, ast.Call)
            self._library_form = (expr if isinstance(expr, shapes) else False,)
        return self._library_form[0]

    def _library(self, args):
        expr = self._single_expression()
        if expr is False or expr is None:
            return NotImplemented
        by_name = dict(zip(self._params(), args))

        def array(node):
            if isinstance(node, ast.Name) and isinstance(by_name.get(node.id), HipNdArray):
                return by_name[node.id]
            return None

        def np_call(node, names):
            """np.<name>(...) or <array>.<name>(...): (name, positional, keywords)."""
            if not isinstance(node, ast.Call) or not isinstance(node.func, ast.Attribute):
                return None
            if node.func.attr not in names:
                return None
            base = node.func.value
            if isinstance(base, ast.Name) and self._resolve(base.id) is np:
                return node.func.attr, list(node.args), node.keywords
            if array(base) is not None:
                return node.func.attr, [base] + list(node.args), node.keywords
            return None

        try:
            # a (+|-|*) b
            if isinstance(expr, ast.BinOp) and type(expr.op) in _BINARY:
                a, b = array(expr.left), array(expr.right)
                if a is not None and b is not None and a.dtype == b.dtype and \
                        a.ndim <= 2 and b.ndim <= 2:
                    return self._served("library", _BINARY[type(expr.op)](a, b), a.ctx)
            # a @ b, np.dot(a, b)
            if isinstance(expr, ast.BinOp) and isinstance(expr.op, ast.MatMult):
                a, b = array(expr.left), array(expr.right)
                if a is not None and b is not None and a.ndim <= 2 and b.ndim <= 2:
                    return self._served("library", _dot(a, b), a.ctx)
            call = np_call(expr, ("dot",))
            if call and len(call[1]) == 2 and not call[2]:
                a, b = array(call[1][0]), array(call[1][1])
                if a is not None and b is not None and a.ndim <= 2 and b.ndim <= 2:
                    return self._served("library", _dot(a, b), a.ctx)
            # np.dot(a, b, c), np.dot(a, b, out=c) (test_gpu.py:2101-2138)
            if call and len(call[1]) + len(call[2]) == 3 and \
                    all(k.arg == "out" for k in call[2]):
                nodes = call[1] + [k.value for k in call[2]]
                a, b, c = (array(n) for n in nodes)
                if a is not None and b is not None and c is not None and \
                        a.ndim == b.ndim == 2:
                    return self._served("library", _dot(a, b, out=c), a.ctx)
            # np.sum(x, axis=k) and friends
            call = np_call(expr, tuple(_REDUCE))
            if call:
                name, pos, kws = call
                x = array(pos[0]) if pos else None
                axis = None
                ok = x is not None and len(pos) <= 2 and all(k.arg == "axis" for k in kws)
                for node in pos[1:] + [k.value for k in kws]:
                    if isinstance(node, ast.Constant) and (node.value is None or
                                                           isinstance(node.value, int)):
                        axis = node.value
                    else:
                        ok = False
                if ok:
                    result = _reduce_nd(_REDUCE[name], x, axis)
                    if axis is None and isinstance(result, HipNdArray):
                        result = result.asnumpy().reshape(-1)[0]   # a scalar, as NumPy's
                    return self._served("library", result, x.ctx)
            # np.mean(x[, axis]): the sum over the count, in the array's float
            # type (float64 for integers; reference numpy/funcs.py:306-328)
            call = np_call(expr, ("mean",))
            if call:
                name, pos, kws = call
                x = array(pos[0]) if pos else None
                axis = None
                ok = x is not None and len(pos) <= 2 and all(k.arg == "axis" for k in kws)
                for node in pos[1:] + [k.value for k in kws]:
                    if isinstance(node, ast.Constant) and (node.value is None or
                                                           isinstance(node.value, int)):
                        axis = node.value
                    else:
                        ok = False
                if ok:
                    return self._served("library", _mean(x, axis), x.ctx)
            # np.sqrt(np.square(a).sum(axis=1)), np.sqrt(np.sum(a * a, axis=1)): the
            # fused row-norm kernel (test_l2_norm, test_gpu.py:2198-2223)
            call = np_call(expr, ("sqrt",))
            if call and len(call[1]) == 1 and not call[2]:
                inner = call[1][0]
                x = None
                if isinstance(inner, ast.Call) and isinstance(inner.func, ast.Attribute) and \
                        inner.func.attr == "sum":
                    base = inner.func.value
                    if isinstance(base, ast.Name) and self._resolve(base.id) is np:
                        operand, rest = (inner.args[0] if inner.args else None), inner.args[1:]
                    else:
                        operand, rest = base, inner.args
                    axis = [a for a in rest] + [k.value for k in inner.keywords
                                                if k.arg == "axis"]
                    if operand is not None and len(axis) == 1 and \
                            len(rest) + len(inner.keywords) == 1 and \
                            isinstance(axis[0], ast.Constant) and axis[0].value in (1, -1):
                        sq = np_call(operand, ("square",))
                        if sq and len(sq[1]) == 1 and not sq[2]:
                            x = array(sq[1][0])
                        elif isinstance(operand, ast.BinOp) and \
                                isinstance(operand.op, ast.Mult) and \
                                isinstance(operand.left, ast.Name) and \
                                isinstance(operand.right, ast.Name) and \
                                operand.left.id == operand.right.id:
                            x = array(operand.left)
                if x is not None and x.dtype == np.float32 and x.ndim == 2:
                    return self._served("library", ops.l2_norm_rows(x), x.ctx)
            # np.sqrt(np.sum(x * x))
            if call and len(call[1]) == 1 and not call[2]:
                inner = np_call(call[1][0], ("sum",))
                if inner and len(inner[1]) == 1 and not inner[2]:
                    prod = inner[1][0]
                    if isinstance(prod, ast.BinOp) and isinstance(prod.op, ast.Mult) and \
                            isinstance(prod.left, ast.Name) and \
                            isinstance(prod.right, ast.Name) and \
                            prod.left.id == prod.right.id:
                        x = array(prod.left)
                        if x is not None and x.dtype == np.float32:
                            return self._served(
                                "library", ops.sqrt_sum_squares(x).asnumpy().reshape(-1)[0],
                                x.ctx)
        except (TypeError, ValueError, NotImplementedError):
            return NotImplemented       # outside what the kernel covers: fuse instead
        return NotImplemented

    def _resolve(self, name):
        if self._names is None:
            cv = inspect.getclosurevars(self.py_func)
            self._names = dict(getattr(self.py_func, "__globals__", {}))
            for table in (cv.builtins, cv.globals, cv.nonlocals):
                self._names.update(table)
        return self._names.get(name)

    @property
    def _stage_stem(self):
        """The function's name as an identifier (a lambda's is not one): the
        stem of the names of the kernels generated for its stages."""
        name = self.py_func.__name__
        if name.isidentifier():
            return name
        name = re.sub(r"\W", "_", name).strip("_") or "function"
        return name if not name[0].isdigit() else "f" + name

    def _callee(self, node):
        """The Python object a call's function expression names: a name, or
        attributes of one (``numba_mlir.prange``), else None."""
        if isinstance(node, ast.Name):
            return self._resolve(node.id)
        if isinstance(node, ast.Attribute):
            base = self._callee(node.value)
            return getattr(base, node.attr, None) if base is not None else None
        return None

    def _served(self, how, result, ctx):
        self.last_launch = {"path": how, "kernel": ctx.last_kernel()}
        return result

    # -- 2. one parallel loop ------------------------------------------------
    def _has_parallel_loop(self):
        if self._parallel_loop is None:
            self._parallel_loop = False
            if not isinstance(self._node, ast.Lambda):
                for stmt in self._node.body:
                    if isinstance(stmt, ast.For) and isinstance(stmt.iter, ast.Call):
                        target = self._callee(stmt.iter.func)
                        if getattr(target, "_nmk_prange", False):
                            self._parallel_loop = True
        return self._parallel_loop

    def _compile(self, mode, args, ndim, remap):
        captured = kernel_impl.captured_constants(self.py_func)
        arrays = [a for a in args if isinstance(a, HipNdArray)]
        noalias = hip.disjoint(arrays)
        stream = hip.streams(arrays)
        for specialize in (True, False):
            types = [kernel_compiler.type_of_argument(a, specialize) for a in args]
            key = (mode, ndim, tuple(kernel_compiler.type_key(t) for t in types),
                   captured, remap, noalias, stream)
            compiled = self._compiled.get(key)
            if compiled is not None or len(self._compiled) < kernel_impl.MAX_SPECIALISATIONS:
                break
        if compiled is None:
            compiled = kernel_compiler.translate(
                self.py_func, types, ndim, kernel_impl, self.boundscheck, remap, mode,
                noalias=noalias, elements_per_thread=ELEMENTS_PER_THREAD, stream=stream)
            # njit(fastmath=True): multiply-adds may fuse
            compiled.fastmath = bool(self.options.get("fastmath", False))
            self._compiled[key] = compiled
        return compiled

    def _grid_rank(self):
        """Depth of the perfect nest of prange loops at the top level (up to
        three; inner bounds must not depend on outer loop variables)."""
        if self._rank is None:
            loop = next(s for s in self._node.body if isinstance(s, ast.For))
            rank, seen = 1, {loop.target.id} if isinstance(loop.target, ast.Name) else set()
            while rank < 3 and len(loop.body) == 1 and isinstance(loop.body[0], ast.For):
                inner = loop.body[0]
                it = inner.iter
                if not (isinstance(it, ast.Call) and
                        getattr(self._callee(it.func), "_nmk_prange", False)):
                    break
                used = {n.id for a in it.args for n in ast.walk(a) if isinstance(n, ast.Name)}
                if used & seen or not isinstance(inner.target, ast.Name):
                    break
                seen.add(inner.target.id)
                loop, rank = inner, rank + 1
            self._rank = rank
        return self._rank

    def _host_scope(self, args):
        """The names the body's host-side statements see."""
        func = self.py_func
        scope = dict(getattr(func, "__globals__", {}))
        for name, cell in zip(func.__code__.co_freevars, func.__closure__ or ()):
            try:
                scope[name] = cell.cell_contents
            except ValueError:            # not yet bound
                pass
        scope.update(zip(self._params(), args))
        return scope

    @staticmethod
    def _host_code(compiled):
        """A translated loop's host-side sources as code objects (once)."""
        code = getattr(compiled, "_host_code", None)
        if code is None:
            code = compiled._host_code = (
                [compile(src, "<loop preamble>", "exec") for src in compiled.preamble_source],
                [[compile(src, "<loop bound>", "eval") for src in sources]
                 for sources in compiled.grid_sources],
                None if compiled.return_source is None else
                compile(compiled.return_source, "<loop result>", "eval"))
        return code

    def _parallel(self, args):
        ctx = kernel_impl.check_device_args(args)
        arrays = [a for a in args if isinstance(a, HipNdArray)]
        # what the choice of kernel depends on: types, shapes, strides, aliasing
        key = (ctx, kernel_impl.plan_key(args),
               kernel_impl.captured_constants(self.py_func), hip.disjoint(arrays))
        entry = self._loop_plans.get(key)
        if entry is None:
            if len(self._loop_plans) >= MAX_PLANS:
                self._loop_plans.clear()
            rank = self._grid_rank()
            entry = self._loop_plans[key] = {
                "nest": self._compile("parallel", args, rank, rank > 1),
                "flat": None, "plans": {}}
        scope = self._host_scope(args)

        def trip_counts(kernel):
            preamble, bounds, _ = self._host_code(kernel)
            for code in preamble:
                try:                      # scalars the loop bounds may be built from
                    exec(code, scope)     # noqa: S102
                except Exception:         # noqa: BLE001 -- device-only values
                    pass
            return tuple(len(range(*[int(eval(code, scope)) for code in codes]))  # noqa: S307
                         for codes in bounds)

        compiled = entry["nest"]
        counts = trip_counts(compiled)
        if len(counts) > 1 and max(counts[:-1]) > 65535:
            # the outer loops land on grid y / z, which are 16-bit: keep only
            # the outermost loop as the grid
            if entry["flat"] is None:
                entry["flat"] = self._compile("parallel", args, 1, False)
            compiled = entry["flat"]
            scope = self._host_scope(args)
            counts = trip_counts(compiled)
        count = math.prod(counts)
        partials = []
        read_back = None

        def make_partials(blocks):
            # (a slot per block and one for the total, which the launch's last
            # block leaves there)
            for _, dtype, _ in compiled.reductions:
                partials.append(HipNdArray.empty((max(blocks, 1) + 1,), dtype,
                                                 device=ctx.device))
            return partials

        def totals(arrays):
            return [part[part.shape[0] - 1:].asnumpy()[0] for part in arrays]

        if count == 0 and compiled.reductions:
            info = {"kernel": compiled.name, "grid": (0, 0, 0), "block": (0, 0, 0)}
        else:
            plan = entry["plans"].get((compiled.name, counts))
            if plan is None:
                plan = kernel_impl.plan_compiled(
                    ctx, compiled, self.py_func.__name__, counts, args,
                    make_partials=make_partials if compiled.reductions else None)
                plan.run()
                read_back = totals(partials)         # (before others see the plan)
                if len(entry["plans"]) >= MAX_PLANS:
                    entry["plans"].clear()
                entry["plans"][(compiled.name, counts)] = plan
            elif compiled.reductions and plan.partials_free.acquire(blocking=False):
                # the launch's own arrays of partial results, read back before
                # another call of this thread or any other may write them
                try:
                    partials = plan.partials
                    plan.run(args, partials=partials)
                    read_back = totals(partials)
                finally:
                    plan.partials_free.release()
            else:
                if compiled.reductions:
                    make_partials(math.prod(plan.grid))
                plan.run(args, partials=partials)
            info = plan.info
            self.last_plan = plan
        self.last_launch = dict(info, path="parallel loop")
        # the totals of the reduction variables (added up by the launch's last
        # block) onto the values the variables had before the loop
        if read_back is None:
            read_back = totals(partials)
        for (name, dtype, op), fold in zip(compiled.reductions, read_back):
            start = np.dtype(dtype).type(scope[name])
            with np.errstate(over="ignore"):
                fold = np.dtype(dtype).type(fold)
                scope[name] = start + fold if op == "add" else start * fold
        return_code = self._host_code(compiled)[2]
        if return_code is not None:
            return eval(return_code, scope)                              # noqa: S307
        return None

    # -- 3. straight-line bodies split at reductions and contractions -------
    def _plan(self):
        if self._stage_plan is None:
            plan = None
            if isinstance(self._node, (ast.FunctionDef, ast.Lambda)):
                plan = staging.plan_of(
                    self._node, lambda name: self._resolve(name) is np,
                    lambda name: isinstance(self._resolve(name), Dispatcher))
            self._stage_plan = (plan,)
        return self._stage_plan[0]

    def _staged(self, plan, args):
        if len(args) != len(plan.params):
            raise TypeError(f"{self.py_func.__name__}() takes {len(plan.params)} arguments")
        env = dict(zip(plan.params, args))
        scope = None
        launches = []
        for k, stage in enumerate(plan.stages):
            if stage.kind == "map" and stage.deferred:
                continue                  # evaluated inside the reduction that follows
            if stage.kind == "lib" and stage.fused_map is not None:
                if scope is None:
                    scope = self._host_scope(())
                value = self._stage_fused_reduction(k, stage, env, scope, launches)
                if value is not NotImplemented:
                    env[stage.target] = value
                    continue
                env[stage.fused_map.target] = self._stage_map(
                    k - 1, stage.fused_map, env, scope, launches)
            if stage.kind == "lib":
                env[stage.target] = self._stage_library(
                    stage, [env[n] for n in stage.operands], launches, env)
                continue
            if stage.kind == "view":
                if scope is None:
                    scope = self._host_scope(())
                env[stage.target] = self._stage_view(stage, env, scope)
                continue
            if stage.kind == "alloc":
                if scope is None:
                    scope = self._host_scope(())
                env[stage.target] = self._stage_alloc(stage, env, scope, args)
                continue
            if stage.kind == "make":
                if scope is None:
                    scope = self._host_scope(())
                env[stage.target] = self._stage_make(stage, env, scope, args)
                launches.append({"path": "library", "op": stage.op})
                continue
            if stage.kind == "call":
                callee = self._resolve(stage.op)
                value = callee._run([env[n] for n in stage.args])
                launches.append(callee.last_launch)
                if stage.target is not None:
                    env[stage.target] = value
                continue
            if stage.kind != "store" and isinstance(stage.expr, ast.Name) and \
                    stage.expr.id in env:
                value = env[stage.expr.id]            # another name for a value
            else:
                if scope is None:
                    scope = self._host_scope(())
                value = self._stage_map(k, stage, env, scope, launches)
            if stage.kind == "return":
                self.last_launch = {"path": "staged", "stages": launches}
                if isinstance(value, HipNdArray) and value.ndim == 0:
                    value = value.asnumpy()[()]          # one indexed element
                return value
            if stage.kind == "map":
                env[stage.target] = value
        self.last_launch = {"path": "staged", "stages": launches}
        return None

    def _stage_dispatcher(self, k, stage, scope):
        """The compiled function of map / store stage ``k`` and its parameters."""
        key = (k, kernel_impl.captured_constants(self.py_func))
        entry = self._stage_funcs.get(key)
        if entry is None:
            func, params = staging.stage_function(
                stage, f"{self._stage_stem}_stage{k}", scope)
            entry = self._stage_funcs[key] = (
                Dispatcher(func, boundscheck=self.boundscheck, **self.options), params)
        return entry

    def _stage_map(self, k, stage, env, scope, launches):
        missing = [n for n in stage.inputs if n not in env]
        if missing:
            raise kernel_compiler.KernelCompileError(
                f"{self.py_func.__name__}, line {stage.node.lineno}: '{missing[0]}' is "
                "used before it is assigned")
        if not any(isinstance(env[n], HipNdArray) for n in stage.inputs) and \
                not (stage.kind == "store" and isinstance(env.get(stage.target), HipNdArray)):
            # scalars only (the result of a full reduction, say): on the host
            expr = ast.fix_missing_locations(ast.Expression(body=stage.expr))
            value = eval(compile(expr, "<scalar stage>", "eval"), scope, dict(env))  # noqa: S307
            launches.append({"path": "host scalar"})
            return value
        sub, params = self._stage_dispatcher(k, stage, scope)
        values = [env[p] for p in params]
        if stage.kind == "store" and isinstance(env.get(stage.target), HipNdArray):
            # x[1:] += x[:-1]: an operand that shares memory with the target
            # under another view is read in full first, as NumPy does
            target = env[stage.target]
            values = [_copy(v) if isinstance(v, HipNdArray) and _overlaps(v, target) else v
                      for v in values]
        value = sub._run(values)
        launches.append(sub.last_launch)
        return value

    def _stage_fused_reduction(self, k, stage, env, scope, launches):
        """np.sum / np.mean of a map over operands of one dense shape: the map
        runs inside a parallel-loop reduction.  NotImplemented when the
        operands do not fit (the caller then runs the two stages)."""
        source = stage.fused_map
        if any(n not in env for n in source.inputs):
            return NotImplemented
        values = [env[n] for n in source.inputs]
        arrays = [n for n, v in zip(source.inputs, values) if isinstance(v, HipNdArray)]
        if not arrays:
            return NotImplemented
        first = env[arrays[0]]
        if first.size == 0 or not all(
                env[n].shape == first.shape and env[n].is_c_contiguous() for n in arrays):
            return NotImplemented
        # the type the map stage itself would give its result (it follows from
        # the operands' types: looked up once per combination)
        type_key = ("map dtype", k, kernel_impl.captured_constants(self.py_func), tuple(
            (v.dtype, v.ndim) if isinstance(v, HipNdArray) else type(v) for v in values))
        dtype = self._stage_funcs.get(type_key)
        if dtype is None:
            try:
                sub, params = self._stage_dispatcher(k - 1, source, scope)
                flat = [env[p].reshape((first.size,)) if p in arrays else env[p]
                        for p in params]
                dtype = sub._compile("elementwise", flat, 1, False).ret_dtype
            except kernel_compiler.KernelCompileError:
                return NotImplemented
            self._stage_funcs[type_key] = dtype if dtype is not None else False
        if dtype is None or dtype is False:
            return NotImplemented
        dtype = np.dtype(dtype)
        if dtype.kind not in "fiub":
            return NotImplemented
        integer = dtype.kind != "f"
        axis = stage.kwargs.get("axis")
        if axis is not None:
            return self._stage_fused_axis_reduction(k, stage, env, scope, launches, arrays,
                                                    dtype, axis)
        key = ("sum", k, kernel_impl.captured_constants(self.py_func), tuple(arrays), integer)
        entry = self._stage_funcs.get(key)
        if entry is None:
            namespace = dict(scope, _nmk_prange=prange)
            try:
                func, params = staging.reduction_function(
                    source, f"{self._stage_stem}_stage{k}_sum", namespace, set(arrays),
                    integer)
                entry = (Dispatcher(func, parallel=True, boundscheck=self.boundscheck,
                                    **self.options), params)
            except kernel_compiler.KernelCompileError:
                entry = False
            self._stage_funcs[key] = entry
        if entry is False:
            return NotImplemented
        sub, params = entry
        flat = [first.size] + [env[n].reshape((first.size,)) if n in arrays else env[n]
                               for n in source.inputs]
        try:
            total = sub._run(flat)
        except kernel_compiler.KernelCompileError:
            self._stage_funcs[key] = False        # not expressible per element
            return NotImplemented
        launches.append(dict(sub.last_launch, fused="map + sum"))
        if stage.op == "sum":
            # NumPy sums small integers in the platform integer
            out = np.dtype(np.int64) if dtype.kind in "ib" else \
                (np.dtype(np.uint64) if dtype.kind == "u" else dtype)
            return out.type(total)
        float_t = dtype.type if dtype.kind == "f" else np.float64
        return float_t(float_t(total) / float_t(first.size))

    def _stage_fused_axis_reduction(self, k, stage, env, scope, launches, arrays, dtype, axis):
        """np.sum / np.mean of a map along an axis of dense matrices of one
        shape.  Along the rows: one work-group per row with a work-group
        reduction.  Down the columns: chunks of rows per work-item, adjacent
        lanes on adjacent columns, partial sums added by the column-sum
        kernel."""
        source = stage.fused_map
        first = env[arrays[0]]
        if first.ndim != 2:
            return NotImplemented
        rows, cols = first.shape
        along_rows = axis in (1, -1)
        if along_rows and rows < 64:            # too few work-groups to fill the GPU
            return NotImplemented
        if dtype.kind == "u":
            return NotImplemented
        if not along_rows and cols % staging.COLUMNS_PER_ITEM:
            return NotImplemented
        integer = dtype.kind != "f"
        result_dtype = np.dtype(np.int64) if dtype.kind in "ib" else \
            (np.dtype(np.uint64) if dtype.kind == "u" else dtype)
        if stage.op == "mean":
            result_dtype = dtype if dtype.kind == "f" else np.dtype(np.float64)
        if along_rows and cols <= staging.SHORT_ROW and rows >= 4096:
            return NotImplemented
        key = ("axis", along_rows, k, kernel_impl.captured_constants(self.py_func),
               tuple(arrays), integer)
        entry = self._stage_funcs.get(key)
        if entry is None:
            namespace = dict(scope, _nmk_group_id=kernel_impl.get_group_id,
                             _nmk_local_id=kernel_impl.get_local_id,
                             _nmk_global_id=kernel_impl.get_global_id,
                             _nmk_group=kernel_impl.group)
            make = staging.row_sum_function if along_rows else staging.column_sum_function
            func, params = make(source, f"{self._stage_stem}_stage{k}_axis", namespace,
                                set(arrays), integer)
            entry = self._stage_funcs[key] = kernel_impl.Kernel(
                func, dict(boundscheck=self.boundscheck, **self.options))
        if entry is False:
            return NotImplemented
        inputs = [env[n] for n in source.inputs]
        ctx = first.ctx
        acc_dtype = np.int64 if integer else np.float64
        try:
            if along_rows:
                total = HipNdArray.empty((rows,), acc_dtype if stage.op == "mean" else
                                         result_dtype, device=ctx.device)
                launch = entry[(rows * staging.ROW_LANES,), (staging.ROW_LANES,)]
                launch(cols, *inputs, total)
            else:
                # (more chunks cost partial-sum traffic, fewer leave the GPU idle:
                # 256 chunks of 64 rows measured best for 16384 x 8192)
                chunks = max(1, min(256, rows // 64))
                chunk = -(-rows // chunks)
                chunks = -(-rows // chunk)
                partial = HipNdArray.empty((chunks, cols), acc_dtype, device=ctx.device)
                launch = entry[(chunks, cols // staging.COLUMNS_PER_ITEM), ()]
                launch(rows, chunk, *inputs, partial)
                total = ops.sum(partial, axis=0)
        except kernel_compiler.KernelCompileError:
            self._stage_funcs[key] = False        # not expressible per element
            return NotImplemented
        launches.append(dict(launch.last_launch, path="kernel", fused="map + axis sum"))
        if stage.op == "mean":
            return _DIVIDE_TO[result_dtype.type](total, result_dtype.type(
                cols if along_rows else rows))
        if total.dtype != result_dtype:
            return _CAST_TO[result_dtype.type](total)
        return total

    def _stage_alloc(self, stage, env, scope, call_args):
        """np.empty / zeros / ones (and *_like) on the device of the call's
        arrays (reference: numpy/funcs.py:581-640)."""
        def host(node):
            expr = ast.fix_missing_locations(ast.Expression(body=node))
            return eval(compile(expr, "<allocation argument>", "eval"), scope, dict(env))  # noqa: S307

        pos = [host(n) for n in stage.args[0]]
        kws = {k.arg: host(k.value) for k in stage.args[1]}
        where = f"{self.py_func.__name__}, line {stage.node.lineno}"
        unknown = set(kws) - {"shape", "dtype"}
        if unknown or len(pos) > 2:
            raise kernel_compiler.KernelCompileError(
                f"{where}: np.{stage.op}: only shape and dtype are supported")
        ctx = kernel_impl.check_device_args(
            [a for a in list(call_args) + list(env.values()) if isinstance(a, HipNdArray)])
        if stage.op.endswith("_like"):
            like = pos[0]
            shape = like.shape
            dtype = kws.get("dtype", pos[1] if len(pos) > 1 else None) or like.dtype
        else:
            shape = pos[0] if pos else kws["shape"]
            dtype = kws.get("dtype", pos[1] if len(pos) > 1 else None) or np.float64
        if isinstance(shape, (int, np.integer)):
            shape = (int(shape),)
        out = HipNdArray.empty(tuple(int(n) for n in shape), dtype, device=ctx.device)
        if not stage.op.startswith("empty") and out.size:
            _fill(out, out.dtype.type(1 if stage.op.startswith("ones") else 0))
        return out

    def _stage_make(self, stage, env, scope, call_args):
        """np.arange / eye / tril / triu / outer / cov / concatenate / hstack /
        vstack on the device of the call's arrays."""
        def host(node):
            expr = ast.fix_missing_locations(ast.Expression(body=node))
            return eval(compile(expr, "<argument>", "eval"), scope, dict(env))  # noqa: S307

        where = f"{self.py_func.__name__}, line {stage.node.lineno}"
        arrays = [env[name] for name in stage.operands]
        nodes, slots, keywords = stage.args
        pos = [arrays[slot] if slot is not None else host(node)
               for node, slot in zip(nodes, slots or [None] * len(nodes))]
        kws = {key: arrays[value] if isinstance(value, int) else host(value)
               for key, value in keywords}
        op = stage.op
        try:
            if any(not isinstance(a, HipNdArray) for a in arrays):
                raise TypeError("the array arguments must be device arrays")
            ctx = kernel_impl.check_device_args(
                [a for a in list(call_args) + list(env.values()) if isinstance(a, HipNdArray)])
            if op == "arange":
                return _arange(ctx, *pos, **kws)
            if op == "eye":
                return _eye(ctx, *pos, **kws)
            if op in ("tril", "triu"):
                k = pos[1] if len(pos) > 1 else kws.pop("k", 0)
                if kws or len(pos) > 2:
                    raise TypeError("takes an array and k")
                return _tri(pos[0], k, op == "tril")
            if op == "outer":
                if kws or len(pos) != 2:
                    raise TypeError("takes two arrays")
                return _outer(*pos)
            if op == "cov":
                return _cov(*pos, **kws)
            axis = pos[0] if pos else kws.pop("axis", 0)
            if kws or len(pos) > 1:
                raise TypeError("takes a tuple of arrays and an axis")
            if op == "concatenate":
                return _concatenate(arrays, axis)
            if pos:
                raise TypeError("takes a tuple of arrays")
            if op == "dstack":
                arrays = [a.reshape((1, a.size, 1)) if a.ndim < 2 else
                          a.reshape(a.shape + (1,)) if a.ndim == 2 else a for a in arrays]
                return _concatenate(arrays, 2)
            if op == "hstack":
                arrays = [a.reshape((1,)) if a.ndim == 0 else a for a in arrays]
                return _concatenate(arrays, 0 if arrays and arrays[0].ndim == 1 else 1)
            arrays = [a.reshape((1, a.size)) if a.ndim < 2 else a for a in arrays]
            return _concatenate(arrays, 0)
        except (TypeError, ValueError, NotImplementedError) as exc:
            raise kernel_compiler.KernelCompileError(f"{where}: np.{op}: {exc}") from exc

    def _stage_view(self, stage, env, scope):
        x = env[stage.operands[0]]
        where = f"{self.py_func.__name__}, line {stage.node.lineno}"
        if stage.op == "len":
            return len(x)
        if stage.op in staging.ARRAY_FACTS:
            if stage.op == "strides" and isinstance(x, HipNdArray):
                return tuple(st * x.dtype.itemsize for st in x.elem_strides)
            if stage.op == "itemsize" and isinstance(x, HipNdArray):
                return x.dtype.itemsize
            return getattr(x, stage.op)
        if stage.op == "getitem":
            node = ast.Subscript(value=ast.Name(id="_nmk_sliced", ctx=ast.Load()),
                                 slice=stage.args[0], ctx=ast.Load())
            expr = ast.fix_missing_locations(ast.Expression(body=node))
            try:
                view = eval(compile(expr, "<index>", "eval"), scope,  # noqa: S307
                            dict(env, _nmk_sliced=x))
                if isinstance(stage.node, ast.Assign) and isinstance(view, HipNdArray) and \
                        view.ndim == 0:
                    view = view.reshape((1,))       # the target of x[i, j] = value
                return view
            except (TypeError, ValueError, IndexError, NameError, NotImplementedError) as exc:
                raise kernel_compiler.KernelCompileError(f"{where}: {exc}") from exc
        args = []
        for node in stage.args:
            expr = ast.fix_missing_locations(ast.Expression(body=node))
            args.append(eval(compile(expr, "<view argument>", "eval"), scope, dict(env)))  # noqa: S307
        if not isinstance(x, HipNdArray):
            return getattr(np, stage.op)(x, *args)
        try:
            if stage.op == "reshape":
                return x.reshape(*args)
            if stage.op == "ravel":
                return x.reshape((x.size,))
            if stage.op in ("copy", "flatten"):
                if args:
                    raise NotImplementedError("the order argument is not supported")
                return _copy(x) if stage.op == "copy" else _copy(x).reshape((x.size,))
            if stage.op == "asfortranarray":
                # (numpy/funcs.py:1243-1246: a copy; the layout is the compiler's)
                return _copy(x.T).T
            if stage.op == "astype":
                if len(args) != 1:
                    raise TypeError("astype takes a type")
                return _astype(x, np.dtype(args[0]))
            if stage.op == "flip":
                # numpy.flip (numpy/funcs.py:236-253): negative strides
                if len(args) > 1 or (args and not (args[0] is None or
                                                   isinstance(args[0], (int, np.integer)))):
                    raise NotImplementedError("flip takes one integer axis or none")
                axis = args[0] if args else None
                if axis is not None and not -x.ndim <= axis < x.ndim:
                    raise ValueError("axis out of range")
                which = range(x.ndim) if axis is None else (axis % x.ndim,)
                return x[tuple(slice(None, None, -1) if d in which else slice(None)
                               for d in range(x.ndim))]
            return x.transpose(*args)
        except (TypeError, ValueError, NotImplementedError) as exc:
            raise kernel_compiler.KernelCompileError(f"{where}: {stage.op}: {exc}") from exc

    def _stage_library(self, stage, vals, launches, env):
        op, axis = stage.op, stage.kwargs.get("axis")
        where = f"{self.py_func.__name__}, line {stage.node.lineno}"
        try:
            out = env[stage.kwargs["out"]] if "out" in stage.kwargs else None
            if not any(isinstance(v, HipNdArray) for v in vals):
                launches.append({"path": "host scalar"})
                kwargs = dict(stage.kwargs, out=out) if out is not None else stage.kwargs
                return getattr(np, op)(*vals, **kwargs)
            ctx = next(v.ctx for v in vals if isinstance(v, HipNdArray))
            if op == "dot":
                result = _dot(*vals, out=out)
            else:
                x = vals[0]
                if op == "mean":
                    result = _mean(x, axis)
                else:
                    result = _reduce_nd(_REDUCE[op], x, axis)
                    if axis is None and isinstance(result, HipNdArray):
                        result = result.asnumpy().reshape(-1)[0]
            launches.append({"path": "library", "kernel": ctx.last_kernel()})
            return result
        except (TypeError, ValueError, NotImplementedError) as exc:
            raise kernel_compiler.KernelCompileError(f"{where}: np.{op}: {exc}") from exc

    # -- 4. elementwise fusion -----------------------------------------------
    def _refuse_sequential_array_loops(self, args):
        """A ``for ... in range(...)`` whose bounds are taken from an array
        argument (``x.shape[0]``, ``len(x)``, ``x.size``) walks that array in
        order: on the host that is a sequential loop, which is not offloaded
        -- as one work-item's loop inside a fused map it would run once per
        element.  Such a function must say ``prange``."""
        arrays = {name for name, a in zip(self._params(), args) if isinstance(a, HipNdArray)}

        def sized_by_array(node):
            for n in ast.walk(node):
                if isinstance(n, ast.Attribute) and n.attr in ("shape", "size") and \
                        isinstance(n.value, ast.Name) and n.value.id in arrays:
                    return n.value.id
                if isinstance(n, ast.Call) and isinstance(n.func, ast.Name) and \
                        n.func.id == "len" and len(n.args) == 1 and \
                        isinstance(n.args[0], ast.Name) and n.args[0].id in arrays:
                    return n.args[0].id
            return None

        # names bound to such extents first (n = len(x); for i in range(n))
        extents = {}
        for n in ast.walk(self._node):
            if isinstance(n, ast.Assign) and len(n.targets) == 1 and \
                    isinstance(n.targets[0], ast.Name):
                owner = sized_by_array(n.value)
                if owner:
                    extents[n.targets[0].id] = owner
        for n in ast.walk(self._node):
            if not (isinstance(n, ast.For) and isinstance(n.iter, ast.Call) and
                    self._callee(n.iter.func) is range):
                continue
            owner = None
            for a in n.iter.args:
                owner = owner or sized_by_array(a)
                for m in ast.walk(a):
                    if isinstance(m, ast.Name) and m.id in extents:
                        owner = owner or extents[m.id]
            if owner:
                raise kernel_compiler.KernelCompileError(
                    f"{self.py_func.__name__}, line {n.lineno}: a range loop over the extent of "
                    f"array argument '{owner}' is sequential and is not offloaded; write it "
                    "with prange")

    def _arrays_asked_about(self):
        """Parameters whose shape, size, length or single elements the body
        reads."""
        if self._asked is None:
            params, asked = set(self._params()), set()
            for n in ast.walk(self._node):
                if isinstance(n, ast.Attribute) and n.attr in staging.ARRAY_FACTS and \
                        isinstance(n.value, ast.Name):
                    asked.add(n.value.id)
                elif isinstance(n, ast.Call) and isinstance(n.func, ast.Name) and \
                        n.func.id == "len" and len(n.args) == 1 and \
                        isinstance(n.args[0], ast.Name):
                    asked.add(n.args[0].id)
                elif isinstance(n, ast.Subscript) and isinstance(n.ctx, ast.Load) and \
                        isinstance(n.value, ast.Name):
                    asked.add(n.value.id)
            self._asked = asked & params
        return self._asked

    def _elementwise(self, args):
        ctx = kernel_impl.check_device_args(args)
        # Everything but addresses and scalar values is fixed by the argument
        # types, shapes and strides: such a call replays a stored launch.
        key = (ctx, kernel_impl.plan_key(args),
               kernel_impl.captured_constants(self.py_func))
        entry = self._plans.get(key)
        if entry is not None:
            plan = entry["plan"]
            if plan is None:              # an argument is written: aliasing decides
                plan = entry["by_alias"].get(
                    hip.disjoint([a for a in args if isinstance(a, HipNdArray)]))
            if plan is not None:
                ret = None
                if entry["ret_dtype"] is not None:
                    ret = HipNdArray.empty(entry["shape"], entry["ret_dtype"],
                                           device=ctx.device)
                plan.run(args, ret)
                self.last_launch = dict(plan.info, path="elementwise")
                self.last_plan = plan
                return ret

        self._refuse_sequential_array_loops(args)
        arrays = [a for a in args if isinstance(a, HipNdArray)]
        shape = np.broadcast_shapes(*[a.shape for a in arrays])
        views = [a.broadcast_to(shape) if isinstance(a, HipNdArray) else a for a in args]
        dense = all(v.is_c_contiguous() for v in views if isinstance(v, HipNdArray))
        asked = [name for name, a in zip(self._params(), args)
                 if isinstance(a, HipNdArray) and name in self._arrays_asked_about()]
        if asked:
            # the body reads x.shape, len(x) or x[i, j] of an array argument:
            # the map must walk the arrays as they are, not merged into fewer
            # dimensions, and x must not be stretched to a larger shape
            for name, a in zip(self._params(), args):
                if name in asked and a.shape != tuple(shape):
                    raise kernel_compiler.KernelCompileError(
                        f"{self.py_func.__name__}: '{name}' of shape {a.shape} is broadcast "
                        f"to {tuple(shape)}; its shape, length or elements cannot be read "
                        "inside the map")
            if len(shape) > 3:
                raise kernel_compiler.KernelCompileError(
                    f"{self.py_func.__name__}: the shape, length or elements of an array of "
                    "more than 3 dimensions cannot be read inside a map")
            run_shape = tuple(shape)
        elif dense:                       # one long row: the cheapest indexing
            run_shape = (math.prod(shape),)
            views = [v.reshape(run_shape) if isinstance(v, HipNdArray) else v
                     for v in views]
        else:
            run_shape, views = _collapse(shape, views)
        if len(run_shape) > 3:
            return self._elementwise_slices(ctx, args, shape, run_shape, views)
        compiled = self._compile("elementwise", views, len(run_shape),
                                 kernel_impl.remap_mode(run_shape))
        for name, a, v in zip(self._params(), args, views):
            if isinstance(a, HipNdArray) and f"v_{name}" in compiled.written and \
                    a.shape != tuple(shape):
                raise ValueError(f"'{name}' is assigned but has shape {a.shape}, not the "
                                 f"broadcast shape {tuple(shape)}")
        ret = None
        if compiled.ret_dtype is not None:
            ret = HipNdArray.empty(shape, compiled.ret_dtype, device=ctx.device)
        ret_view = ret.reshape(run_shape) if ret is not None else ret
        plan = kernel_impl.plan_compiled(ctx, compiled, self.py_func.__name__,
                                         run_shape, views, ret_view)
        plan.run()
        self.last_launch = dict(plan.info, path="elementwise")
        self.last_plan = plan

        if len(self._plans) >= MAX_PLANS:
            self._plans.clear()
        writes = any(f"v_{name}" in compiled.written for name in self._params())
        entry = self._plans.setdefault(key, {
            "plan": None, "by_alias": {}, "shape": tuple(shape),
            "ret_dtype": compiled.ret_dtype})
        if writes:
            entry["by_alias"][hip.disjoint(arrays)] = plan
        else:
            entry["plan"] = plan
        return ret


    def _elementwise_slices(self, ctx, args, shape, run_shape, views):
        """More than three dimensions that do not merge: one launch of the 3-d
        kernel per index of the leading ones."""
        outer = run_shape[:-3]
        plan = ret = ret_view = None
        for index in np.ndindex(*outer):
            part = [v[index] if isinstance(v, HipNdArray) else v for v in views]
            if plan is None:
                compiled = self._compile("elementwise", part, 3,
                                         kernel_impl.remap_mode(run_shape[-3:]))
                for name, a in zip(self._params(), args):
                    if isinstance(a, HipNdArray) and f"v_{name}" in compiled.written and \
                            a.shape != tuple(shape):
                        raise ValueError(f"'{name}' is assigned but has shape {a.shape}, "
                                         f"not the broadcast shape {tuple(shape)}")
                if compiled.ret_dtype is not None:
                    ret = HipNdArray.empty(shape, compiled.ret_dtype, device=ctx.device)
                    ret_view = ret.reshape(run_shape)
                plan = kernel_impl.plan_compiled(
                    ctx, compiled, self.py_func.__name__, run_shape[-3:], part,
                    None if ret_view is None else ret_view[index])
                plan.run()
            else:
                plan.run(part, None if ret_view is None else ret_view[index])
        self.last_launch = dict(plan.info, path="elementwise", launches=math.prod(outer))
        return ret


def njit(signature_or_function=None, parallel=False, **options):
    """``@njit`` / ``@njit(parallel=True)``."""
    if inspect.isfunction(signature_or_function):
        return Dispatcher(signature_or_function, parallel=parallel, **options)

    def wrap(func):
        return Dispatcher(func, parallel=parallel, **options)

    return wrap


jit = njit
