"""Translates a Python ``@kernel`` body into a gfx950 kernel.

In the reference the body goes through Numba's front end, the plier and GPU
dialects and SPIR-V (reference: numba_mlir/numba_mlir/mlir/kernel_impl.py:97-206,
numba_mlir/mlir_compiler/lib/pipelines/LowerToGpu.cpp).  Here the body's
syntax tree is typed with the same rules and printed as one HIP ``__global__``
function, which hipcc compiles to a code object for ``gpuxModuleLoad``:

* types: Python ``int``/``float``/``bool`` literals and captured constants are
  int64/float64/bool; binary operators promote with ``numpy.promote_types``
  (linalg_builder.py:261-275); ``/`` on integers gives float64; a variable
  assigned values of several types takes their common type;
* one work-item per global id, dimension 0 on x, the tail guarded by
  ``id < global_size`` (LowerToGpu.cpp:1113-1137);
* the kernel's parameters are what the compiled host code passes
  (GpuRuntimeToLlvm.cpp:444-628): per array its pointer, shape and strides (in
  elements), scalars by value, one work-group-memory parameter per
  ``local.array``, then the three global sizes.

Supported syntax: assignments (also augmented and to array elements), ``if``,
``for ... in range(...)``, ``while``, ``break``/``continue``/``return``,
arithmetic with Python semantics for ``//``, ``%`` and ``**``, comparisons,
``and``/``or``/``not``, conditional expressions, indexing with integers,
tuples and slices (views), ``math``/``numpy`` scalar functions, casts, calls
of plain Python functions and lambdas (compiled as device functions), and the
kernel builtins: ids and sizes, ``atomic.add/sub``, ``barrier``/``mem_fence``,
``local.array``/``private.array``, ``group.reduce_*``.
"""

import ast
import hashlib
import inspect
import math
import os
import subprocess
import textwrap

import numpy as np


class KernelCompileError(Exception):
    pass


# ---------------------------------------------------------------------------
# Types
# ---------------------------------------------------------------------------

class Scalar:
    def __init__(self, name, ctype, dtype):
        self.name, self.ctype, self.dtype = name, ctype, np.dtype(dtype)
        self.kind = self.dtype.kind          # b, i, u, f
        self.is_float = self.kind == "f"
        self.is_int = self.kind in "iu"
        self.is_bool = self.kind == "b"

    def __repr__(self):
        return self.name


BOOL = Scalar("bool", "bool", np.bool_)
INT8 = Scalar("int8", "int8_t", np.int8)
INT16 = Scalar("int16", "int16_t", np.int16)
INT32 = Scalar("int32", "int32_t", np.int32)
INT64 = Scalar("int64", "int64_t", np.int64)
UINT8 = Scalar("uint8", "uint8_t", np.uint8)
UINT16 = Scalar("uint16", "uint16_t", np.uint16)
UINT32 = Scalar("uint32", "uint32_t", np.uint32)
UINT64 = Scalar("uint64", "uint64_t", np.uint64)
FLOAT32 = Scalar("float32", "float", np.float32)
FLOAT64 = Scalar("float64", "double", np.float64)
_SCALARS = {s.dtype: s for s in (BOOL, INT8, INT16, INT32, INT64, UINT8, UINT16,
                                 UINT32, UINT64, FLOAT32, FLOAT64)}


def scalar_of(dtype):
    try:
        return _SCALARS[np.dtype(dtype)]
    except (KeyError, TypeError):
        raise KernelCompileError(f"Unsupported element type: {dtype}")


def promote(a, b):
    return scalar_of(np.promote_types(a.dtype, b.dtype))


class Array:
    """``space``: global (an argument or a view of one), local or private.

    An argument can carry two facts the kernel is specialised on, as Numba
    specialises on layout: ``layout == "C"`` (dense row-major: the strides
    follow from the shape) and ``const_shape`` (the extent of a short trailing
    dimension, so that a loop over it unrolls)."""

    def __init__(self, elem, ndim, space="global", layout="A", const_shape=None):
        self.elem, self.ndim, self.space = elem, ndim, space
        self.layout = layout
        self.const_shape = tuple(const_shape) if const_shape else (None,) * ndim

    def key(self):
        return ("array", self.elem.name, self.ndim, self.space, self.layout,
                self.const_shape)

    def ctype(self):
        return f"nmkjit::View<{self.elem.ctype}, {self.ndim}>"

    def __eq__(self, other):
        return isinstance(other, Array) and self.key() == other.key()

    def __hash__(self):
        return hash(self.key())

    def __repr__(self):
        return f"array({self.elem}, {self.ndim}d, {self.space})"


class SliceArg:
    """A ``slice`` passed as a kernel argument: three int64 parameters."""

    def key(self):
        return ("slice",)

    def __eq__(self, other):
        return isinstance(other, SliceArg)

    def __hash__(self):
        return hash("slice")


def type_key(t):
    return t.name if isinstance(t, Scalar) else t.key()


SMALL_DIM = 8      # trailing dimensions up to this extent become constants


def type_of_argument(value, specialize=False):
    """Type of a launch argument (the unboxing of the reference's dispatcher).
    With ``specialize`` a device array also reports a dense row-major layout
    and the extents of its short non-leading dimensions."""
    if hasattr(value, "dtype") and hasattr(value, "ndim") and hasattr(value, "elem_strides"):
        if specialize and value.ndim >= 1:
            dense = bool(getattr(value, "is_c_contiguous", lambda: False)()) and \
                all(n > 0 for n in value.shape)
            const = [None] + [int(n) if 0 < n <= SMALL_DIM else None
                              for n in value.shape[1:]]
            return Array(scalar_of(value.dtype), value.ndim,
                         layout="C" if dense else "A", const_shape=const)
        return Array(scalar_of(value.dtype), value.ndim)
    if isinstance(value, slice):
        return SliceArg()
    if isinstance(value, (bool, np.bool_)):
        return BOOL
    if isinstance(value, np.generic):
        return scalar_of(value.dtype)
    if isinstance(value, int):
        return INT64
    if isinstance(value, float):
        return FLOAT64
    raise KernelCompileError(f"Unsupported kernel argument type: {type(value)}")


class Val:
    """A typed expression: C++ text, type, and what is known at compile time."""

    def __init__(self, code, type_, const=None, nonneg=False, items=None, pyobj=None,
                 slice_parts=None):
        self.code, self.type = code, type_
        self.const = const            # Python value of a compile-time constant
        self.nonneg = nonneg or (isinstance(const, (int, float)) and not
                                 isinstance(const, bool) and const >= 0)
        self.items = items            # tuple expression: list of Val
        self.pyobj = pyobj            # a Python object known at compile time
        self.slice_parts = slice_parts  # (start, stop, step) Vals or None each
        self.gid = None               # k: the value is global id k plus a constant
        self.arr = False              # elementwise mode: computed from array elements
        self.origin = None            # an array: the parameter this is, under any name
        # what the value was computed from, for the fused forms of
        # log(a / b), 1.0 / sqrt(x) and 0.5 + 0.5 * erf(x):
        # ("quot", a, b) | ("sqrt", x) | ("erf", x) | ("halferf", x)
        self.tag = None


class _Deferred(Exception):
    """A name is used before its type is known (resolved by a later pass)."""


_UNARY_MATH = {
    # python name -> C name; results are float32 for float32 input, else float64
    "sqrt": "sqrt", "exp": "exp", "log": "log", "log2": "log2", "log10": "log10",
    "log1p": "log1p", "expm1": "expm1", "sin": "sin", "cos": "cos", "tan": "tan",
    "asin": "asin", "acos": "acos", "atan": "atan", "sinh": "sinh", "cosh": "cosh",
    "tanh": "tanh", "asinh": "asinh", "acosh": "acosh", "atanh": "atanh",
    "erf": "erf", "erfc": "erfc", "gamma": "tgamma", "lgamma": "lgamma",
    "fabs": "fabs", "arcsin": "asin", "arccos": "acos", "arctan": "atan",
    "arcsinh": "asinh", "arccosh": "acosh", "arctanh": "atanh", "exp2": "exp2",
    "cbrt": "cbrt", "absolute": "fabs",
}
_BINARY_MATH = {"atan2": "atan2", "arctan2": "atan2", "pow": "pow",
                "hypot": "hypot", "copysign": "copysign", "fmod": "fmod"}
# NumPy's named forms of the operators (reference: numpy/funcs.py:362-383 and
# 457-562 register the same bodies under both names)
_UFUNC_BINOPS = {
    "add": ast.Add, "subtract": ast.Sub, "multiply": ast.Mult, "divide": ast.Div,
    "true_divide": ast.Div, "power": ast.Pow, "floor_divide": ast.FloorDiv,
    "remainder": ast.Mod, "mod": ast.Mod, "bitwise_and": ast.BitAnd,
    "bitwise_or": ast.BitOr, "bitwise_xor": ast.BitXor, "left_shift": ast.LShift,
    "right_shift": ast.RShift}
_UFUNC_COMPARE = {
    "less": ast.Lt, "less_equal": ast.LtE, "greater": ast.Gt, "greater_equal": ast.GtE,
    "equal": ast.Eq, "not_equal": ast.NotEq}
_UFUNC_UNARY = {"positive": ast.UAdd, "invert": ast.Invert, "bitwise_not": ast.Invert,
                "logical_not": ast.Not}
_ROUNDING = {"floor": "floor", "ceil": "ceil", "trunc": "trunc"}

_CAST_TYPES = {
    bool: BOOL, int: INT64, float: FLOAT64, np.bool_: BOOL, np.int8: INT8,
    np.int16: INT16, np.int32: INT32, np.int64: INT64, np.uint8: UINT8,
    np.uint16: UINT16, np.uint32: UINT32, np.uint64: UINT64,
    np.float32: FLOAT32, np.float64: FLOAT64,
}

_GROUP_NEUTRAL = {
    "add": lambda t: "0",
    "mul": lambda t: "1",
    "min": lambda t: _type_limit(t, True),
    "max": lambda t: _type_limit(t, False),
}
_GROUP_OPS = {"add": "AddOp", "mul": "MulOp", "min": "MinOp", "max": "MaxOp"}


def _type_limit(t, largest):
    if t.is_float:
        return "__builtin_inf()" if largest else "-__builtin_inf()"
    info = np.iinfo(t.dtype)
    v = info.max if largest else info.min
    if t is INT64 and not largest:
        return "INT64_MIN"
    suffix = "ull" if t is UINT64 else "ll"
    return f"{v}{suffix}"


def _float_literal(v, t):
    if math.isnan(v):
        return "__builtin_nan(\"\")" if t is FLOAT64 else "__builtin_nanf(\"\")"
    if math.isinf(v):
        s = "__builtin_inf()" if t is FLOAT64 else "__builtin_inff()"
        return s if v > 0 else "-" + s
    text = float(v).hex()
    return text if t is FLOAT64 else text + "f"


def cast(val, to):
    if val.type is to:
        return val
    if val.const is not None:
        return constant(_convert_const(val.const, to), to)
    return Val(f"(({to.ctype})({val.code}))", to, nonneg=val.nonneg and not to.is_bool)


def _convert_const(v, to):
    if to.is_bool:
        return bool(v)
    if to.is_float:
        return float(to.dtype.type(v))
    if isinstance(v, float):
        v = int(v) if math.isfinite(v) else 0
    return int(np.array(int(v), dtype=np.int64 if -2 ** 63 <= int(v) < 2 ** 63
                        else np.uint64).astype(to.dtype))


def constant(v, t=None):
    if isinstance(v, (bool, np.bool_)):
        t = t or BOOL
    elif isinstance(v, (int, np.integer)):
        t = t or (scalar_of(v.dtype) if isinstance(v, np.generic) else INT64)
    elif isinstance(v, (float, np.floating)):
        t = t or (scalar_of(v.dtype) if isinstance(v, np.generic) else FLOAT64)
    else:
        raise KernelCompileError(f"Unsupported constant: {v!r}")
    if t.is_bool:
        v = bool(v)
        return Val("true" if v else "false", t, const=v)
    if t.is_float:
        v = float(v)
        return Val(_float_literal(v, t), t, const=v)
    v = int(v)
    if t is INT64 and v == -2 ** 63:
        code = "INT64_MIN"
    elif t in (INT64,):
        code = f"((int64_t){v}ll)"
    elif t is UINT64:
        code = f"((uint64_t){v}ull)"
    else:
        code = f"(({t.ctype}){v})"
    return Val(code, t, const=v)


# ---------------------------------------------------------------------------
# Module: everything that ends up in one generated source file
# ---------------------------------------------------------------------------

class Module:
    def __init__(self, stubs, boundscheck=False):
        self.stubs = stubs              # kernel_impl module (the stub objects)
        self.boundscheck = boundscheck  # redirect and report out-of-range indices
        # set when the body can tell how work-items are grouped (local or
        # group ids, local sizes, barriers, fences, local arrays, group
        # reductions): only then does the item-to-lane mapping matter
        self.communicates = False
        self.device_funcs = {}          # (id(func), arg type keys) -> (name, ret type)
        self.device_code = []
        self.in_progress = set()
        self.counter = 0

    def fresh(self, prefix):
        self.counter += 1
        return f"{prefix}{self.counter}"


def _function_ast(func):
    """The FunctionDef or Lambda node of a Python function object."""
    node = getattr(func, "__nmk_ast__", None)    # a function built from a tree
    if node is not None:
        return node
    try:
        src = inspect.getsource(func)
    except (OSError, TypeError) as exc:
        raise KernelCompileError(
            f"No source available for {getattr(func, '__name__', func)!r}: {exc}")
    src = textwrap.dedent(src)
    try:
        tree = ast.parse(src)
    except SyntaxError:
        # the source lines of a lambda need not be a statement on their own
        # (a dictionary entry, an argument): parse from each `lambda` keyword
        found = []
        start = src.find("lambda")
        while start >= 0:
            for end in range(len(src), start + 6, -1):
                try:
                    node = ast.parse(src[start:end].strip().rstrip(","), mode="eval").body
                except SyntaxError:
                    continue
                if isinstance(node, ast.Lambda):
                    found.append(node)
                    break
            start = src.find("lambda", start + 6)
        tree = ast.Module(body=[ast.Expr(value=n) for n in found], type_ignores=[])
    name = func.__name__
    if name == "<lambda>":
        lambdas = [n for n in ast.walk(tree) if isinstance(n, ast.Lambda)]
        nargs = func.__code__.co_argcount
        names = func.__code__.co_varnames[:nargs]
        match = [n for n in lambdas if [a.arg for a in n.args.args] == list(names)]
        if len(match) != 1:
            # same parameter names: tell them apart by the names they use
            used = set(func.__code__.co_names) | set(func.__code__.co_freevars)
            match = [n for n in match if {x.id for x in ast.walk(n.body)
                                          if isinstance(x, ast.Name)} - set(names) == used]
        if len(match) != 1:
            raise KernelCompileError(
                "Cannot tell which lambda of the source line is meant; put each "
                "lambda on a line of its own")
        return match[0]
    for n in ast.walk(tree):
        if isinstance(n, (ast.FunctionDef,)) and n.name == name:
            return n
    raise KernelCompileError(f"Cannot find the definition of {name}")


def _unwrapped_unary(obj):
    """``def f(x): return g(x)`` (or the lambda, or the vectorize()d form of
    either) with ``g`` a function of the math or numpy module: ``g``.
    Anything else: ``obj`` itself."""
    func = getattr(obj, "_nmk_vectorized", None) or obj
    if not inspect.isfunction(func):
        return obj
    try:
        node = _function_ast(func)
    except KernelCompileError:
        return obj
    params = [a.arg for a in node.args.args]
    if len(params) != 1 or node.args.vararg or node.args.kwarg or node.args.kwonlyargs:
        return obj
    if isinstance(node, ast.Lambda):
        value = node.body
    else:
        body = [st for st in node.body
                if not (isinstance(st, ast.Expr) and isinstance(st.value, ast.Constant))]
        if len(body) != 1 or not isinstance(body[0], ast.Return):
            return obj
        value = body[0].value
    if not (isinstance(value, ast.Call) and len(value.args) == 1 and not value.keywords and
            isinstance(value.args[0], ast.Name) and value.args[0].id == params[0]):
        return obj
    target, scope = value.func, dict(getattr(func, "__globals__", {}))
    try:
        scope.update(inspect.getclosurevars(func).nonlocals)
    except (TypeError, ValueError):
        pass
    if isinstance(target, ast.Name):
        inner = scope.get(target.id)
    elif isinstance(target, ast.Attribute) and isinstance(target.value, ast.Name):
        inner = getattr(scope.get(target.value.id), target.attr, None)
    else:
        inner = None
    if inner is None:
        return obj
    mod = getattr(inner, "__module__", None)
    if (mod == "math" or mod == "numpy" or isinstance(inner, np.ufunc)) and \
            getattr(inner, "__name__", None) in _UNARY_MATH:
        return inner
    return obj


class _NotAdjacent(Exception):
    """The body does not fit the adjacent-elements form of a fused map."""


class FunctionTranslator:
    def __init__(self, module, func, arg_types, is_kernel, ndim=0):
        self.m = module
        self.func = func
        self.is_kernel = is_kernel
        self.ndim = ndim
        self.node = _function_ast(func)
        args = self.node.args
        if args.vararg or args.kwarg or args.kwonlyargs or args.defaults:
            raise KernelCompileError("Only plain positional parameters are supported")
        self.params = [a.arg for a in args.args]
        if len(self.params) != len(arg_types):
            raise KernelCompileError(
                f"{func.__name__} takes {len(self.params)} arguments, {len(arg_types)} given")
        self.arg_types = list(arg_types)
        cv = inspect.getclosurevars(func)
        self.outer = {}
        self.outer.update(cv.builtins)
        self.outer.update(cv.globals)
        self.outer.update(cv.nonlocals)
        # names that inspect does not report (used only inside nested scopes)
        self.func_globals = getattr(func, "__globals__", {})
        self.env = dict(zip(self.params, self.arg_types))   # name -> type
        self.assigned = self._assigned_names()
        self.ret_type = None
        self.lines = []
        self.indent = 1
        self.emitting = False
        self.local_arrays = []       # (elem Scalar, shape tuple) in source order
        self.group_sites = []        # (slot name, Scalar, op)
        self.private_decls = []
        # "kernel": an @kernel body; "elementwise": an @njit function of whole
        # arrays fused into one map (an array used as a value means its
        # element at the work-item's index); "parallel": an @njit function
        # whose top-level prange loop becomes the grid; "device" otherwise
        self.mode = "kernel" if is_kernel else "device"
        self.range_source = None     # parallel mode: source of the prange arguments
        self.grid_loops = []         # parallel mode: the perfectly nested prange loops
        self.grid_sources = []       # ... and the source of their range arguments
        self.reductions = {}         # parallel mode: reduction variable -> "add" | "mul"
        self.return_node = None      # parallel mode: the return after the loop
        self.allow_remap = False     # kernels only: see translate_kernel
        self.lanes_along_y = False   # remapped grids with a short x extent
        self.stages_table = False    # the kernel starts by copying a table into LDS
        self.reversed = False
        self.rows_per_lane = 1
        self.grid_stride = False
        self.stream = True           # with noalias: arrays too big to stay cached
        self.written_arrays = set()  # elementwise mode: arrays stored through [:]
        self.read_arrays = set()     # elementwise mode: arrays loaded as values
        self.noalias = False         # no two array arguments overlap (host-checked)
        self._store_only = None      # array parameters the body never reads
        self.last_elem_gid = None    # of the element subscript() resolved last
        self.last_elem_unit = "false"
        self.elements_per_thread = 1
        self.view_origin = {}        # array variable -> the parameter it is another name of
        self.written_origins = set() # parameters assigned through [:] under any name
        self.opaque_write = False    # [:] assignment to an array of unknown origin
        self.prefetched = {}         # parameter -> Array type: loaded ahead of the body
        self.ahead_nodes = {}        # parallel mode: id(p[i] node) -> parameter p
        self.loop_kinds = []         # enclosing loops, outermost first: "grid" | "sequential"
        self._lambda_body = None
        self.reduction_types = []    # (name, Scalar) in parameter order
        self.site_names = {}         # ast node -> stable names
        self.array_info = {}         # variable name -> Array type (views)
        # elementwise 1-d maps over dense arrays: a lane takes ADJACENT
        # elements, 128-bit loads and stores (see translate_kernel)
        self.adjacent = False
        self.unit_loop_var = None    # parallel mode: the variable of a prange(n) grid loop
        self.adjacent_outs = {}      # output array (code) -> (element ctype, pointer)
        self.speculates = False      # some call of the body has a plain and a careful form

    # -- helpers -----------------------------------------------------------
    def err(self, node, msg):
        line = getattr(node, "lineno", "?")
        raise KernelCompileError(f"{self.func.__name__}, line {line}: {msg}")

    def _assigned_names(self):
        names = set()
        self.store_count = {}
        body = self.node.body if isinstance(self.node.body, list) else []
        for n in ast.walk(ast.Module(body=body, type_ignores=[])):
            if isinstance(n, ast.Name) and isinstance(n.ctx, ast.Store):
                names.add(n.id)
                self.store_count[n.id] = self.store_count.get(n.id, 0) + 1
        # a name bound once, at the top level, to a constant is that constant
        # (array shapes and range bounds written through a local name)
        self.const_vars = {}
        # ... and one bound once, at the top level, to a global id (plus a
        # constant) is known to run along that grid dimension
        self.gid_vars = {}
        # elementwise mode: names that hold values computed from array
        # elements (they follow the array typing rules, see arith_type)
        self.array_valued = set()
        self.array_reads = 0         # how many such values expressions have read so far
        self.top_level = {id(s) for s in body}
        return names - set(self.params)

    def emit(self, text):
        if self.emitting:
            self.lines.append("  " * self.indent + text)

    def cname(self, name):
        if "." in name:                      # element k of the tuple variable
            base, k = name.split(".")
            return f"vt_{base}_{k}"
        return f"v_{name}"

    # -- name resolution ---------------------------------------------------
    def lookup(self, node):
        name = node.id
        if name in self.env:
            t = self.env[name]
            if isinstance(t, Scalar):
                if name in self.const_vars:
                    return constant(_convert_const(self.const_vars[name], t), t)
                v = Val(self.cname(name), t, nonneg=name in self.nonneg_vars)
                v.gid = self.gid_vars.get(name)
                v.arr = name in self.array_valued
                self.array_reads += v.arr
                return v
            if isinstance(t, Array):
                v = Val(self.cname(name), t)
                if name in self.params:
                    v.origin = name if not self.store_count.get(name) else None
                else:
                    v.origin = self.view_origin.get(name)
                return v
            if isinstance(t, SliceArg):
                c = self.cname(name)
                parts = tuple(Val(f"{c}_{k}", INT64) for k in ("start", "stop", "step"))
                return Val(c, t, slice_parts=parts)
            if isinstance(t, tuple) and t[0] == "tuple":
                items = [Val(self.cname(i), self.env[i], nonneg=i in self.nonneg_vars)
                         if isinstance(i, str) else i for i in self.tuple_vars[name]]
                return Val(None, t, items=items)
            raise KernelCompileError(f"Unsupported variable type for {name}")
        if name in self.params or name in self.assigned:
            raise _Deferred(name)
        if name in self.outer:
            return self.from_python(self.outer[name], node)
        if name in self.func_globals:
            return self.from_python(self.func_globals[name], node)
        import builtins
        if hasattr(builtins, name):
            return self.from_python(getattr(builtins, name), node)
        self.err(node, f"Unknown name '{name}'")

    def from_python(self, obj, node):
        if isinstance(obj, (bool, int, float, np.generic)) and not isinstance(obj, complex):
            return constant(obj)
        if isinstance(obj, tuple) and all(isinstance(x, (int, np.integer)) for x in obj):
            return Val(None, ("tuple",), items=[constant(int(x)) for x in obj])
        return Val(None, None, pyobj=obj)

    # -- expressions -------------------------------------------------------
    def expr(self, node):
        method = getattr(self, "expr_" + type(node).__name__, None)
        if method is None:
            self.err(node, f"Unsupported expression: {type(node).__name__}")
        reads = self.array_reads
        v = method(node)
        if self.array_reads > reads and isinstance(v, Val) and isinstance(v.type, Scalar):
            v.arr = True          # some operand was computed from array elements
        return v

    def scalar(self, node):
        v = self.expr(node)
        if isinstance(v.type, Array) and self.mode == "elementwise":
            return self.element_here(v, node)
        if not isinstance(v.type, Scalar):
            self.err(node, "A scalar value is required here")
        return v

    def element_here(self, arr, node):
        """Elementwise mode: the element of ``arr`` at this work-item's index
        (every array argument arrives broadcast to the iteration space)."""
        if arr.type.ndim != self.ndim:
            self.err(node, "Only whole arrays of the iteration space can be used "
                           "in an elementwise function")
        self.read_arrays.add(arr.code)
        if self.prefetches(arr):
            # loaded ahead of the body, for all of the lane's elements at once
            self.prefetched[arr.origin] = arr.type
            v = Val(f"nmk_pf_{arr.origin}", arr.type.elem)
            v.arr = True
            self.array_reads += 1
            return v
        if self.adjacent and self.emitting:
            raise _NotAdjacent(f"'{arr.code}' cannot be loaded ahead of the body")
        terms = [f"nmk_gid{d} * {arr.code}.stride[{d}]" for d in range(self.ndim)]
        ref = f"{arr.code}.p[{' + '.join(terms)}]"
        if self.noalias and self.stream and arr.code not in self.written_arrays:
            # read once, by this work-item only: no need to keep it cached
            ref = f"__builtin_nontemporal_load(&{ref})"
        v = Val(ref, arr.type.elem)
        v.arr = True
        self.array_reads += 1
        return v

    _PREFETCH_CTYPES = ("float", "double", "int32_t", "int64_t", "uint32_t", "uint64_t")

    def prefetches(self, arr):
        """A 1-d map that gives a lane several elements loads the lane's
        elements of its read-only array arguments before the first element's
        arithmetic: a body with branches (the range checks of log, exp, erf)
        would otherwise load, compute and store one element after the other,
        one memory latency each.  Needs arguments that do not overlap, and a
        parameter that no statement assigns through [:] under any name."""
        return (self.mode == "elementwise" and self.ndim == 1 and self.noalias and
                self.elements_per_thread > 1 and arr.origin is not None and
                arr.origin not in self.written_origins and not self.opaque_write and
                arr.type.elem.ctype in self._PREFETCH_CTYPES)

    def speculation(self):
        """Template argument of the routines that come in a plain and a
        careful form, where the body is computed under speculation (a fused
        map over adjacent elements), else the empty string."""
        if self.adjacent and self.mode in ("elementwise", "parallel") and self.is_kernel \
                and not self.reductions:
            # (a loop with reduction variables keeps them in registers of one
            # inlined body: no second, out-of-line form)
            self.speculates = True
            return "<decltype(nmk_careful)::value>"
        return ""

    def outputs_are_float32(self):
        """A fused map all of whose results are float32 arrays: its float64
        intermediates need float32's accuracy and a margin, not their own."""
        if self.is_kernel and self.mode == "parallel":
            # a loop without reductions that stores into float32 arrays only
            stored = {n.value.id for n in ast.walk(self.node)
                      if isinstance(n, ast.Subscript) and isinstance(n.ctx, ast.Store) and
                      isinstance(n.value, ast.Name)}
            types = dict(zip(self.params, self.arg_types))
            return bool(stored) and not self.reductions and all(
                isinstance(types.get(n), Array) and types[n].elem is FLOAT32 for n in stored)
        if not (self.is_kernel and self.mode == "elementwise") or self.opaque_write:
            return False
        outs = [t.elem for p, t in zip(self.params, self.arg_types)
                if isinstance(t, Array) and p in self.written_origins]
        if self.ret_type is not None:
            outs.append(self.ret_type)
        return bool(outs) and all(e is FLOAT32 for e in outs)

    _WORD_CTYPES = ("float", "int32_t", "uint32_t")

    def may_be_adjacent(self):
        """Whether the fused map can give each lane four ADJACENT elements:
        one dimension, dense arrays of 4-byte elements that do not overlap.
        (What the body does with them is found out while its statements are
        written: _NotAdjacent.  Maps over 8-byte elements measured faster with
        a lane's elements a block apart.)"""
        if not (self.is_kernel and self.mode in ("elementwise", "parallel") and
                self.ndim == 1 and self.noalias and self.elements_per_thread == 4) or \
                self.m.communicates or self.m.boundscheck or self.opaque_write:
            return False
        if self.reductions and self.mode != "parallel":
            return False
        if self.mode == "parallel":
            # one prange(n) loop: iteration g is work-item g.  Which arrays it
            # reads and stores at its own index is settled while the body is
            # written (check_adjacent_operands).
            return self.unit_loop_var is not None and len(self.grid_loops) == 1
        elems = [t.elem for t in self.arg_types if isinstance(t, Array)]
        if any(isinstance(t, Array) and (t.layout != "C" or t.ndim != 1)
               for t in self.arg_types):
            return False
        if self.ret_type is not None:
            elems.append(self.ret_type)
        return all(e.ctype in self._WORD_CTYPES for e in elems)

    def check_adjacent_operands(self):
        """After the body has been written: every array loaded ahead of it and
        every array it stores must be dense with 4-byte elements, and
        something must be stored."""
        types = dict(zip(self.params, self.arg_types))
        for name in self.prefetched:
            t = types.get(name)
            if not (isinstance(t, Array) and t.layout == "C" and t.ndim == 1 and
                    t.elem.ctype in self._WORD_CTYPES):
                raise _NotAdjacent(f"'{name}' is not a dense array of 4-byte elements")
        if not self.adjacent_outs and not (self.reductions and self.prefetched):
            raise _NotAdjacent("no array is assigned at every index")
        for ctype, _ in self.adjacent_outs.values():
            if ctype not in self._WORD_CTYPES:
                raise _NotAdjacent("an assigned array has 8-byte elements")

    def adjacent_rounds(self, pf, body):
        """The rounds of a fused map over adjacent elements.  A lane loads its
        four elements of every operand in one 128-bit word, computes the four
        results and stores them the same way.  Calls with a plain and a
        careful form run plain first (``nmk_ok`` records whether every operand
        was in range); a wave in which some lane's was not computes its
        elements again the careful way before anything is stored.  Words need
        16-byte aligned arrays: otherwise, and for the last n % 4 elements,
        lanes take single elements."""
        nt = self.stream
        outs = sorted(self.adjacent_outs.items())
        ins = [(n, ct, self.cname(n)) for n, ct, _ in pf]
        pointers = [f"{c}_p" for _, _, c in ins] + [ptr for _, (_, ptr) in outs]
        out = [
            "  const int64_t nmk_gid1 = 0, nmk_gid2 = 0;",
            "  (void)nmk_gid1; (void)nmk_gid2;",
            "  struct nmk_results {",
        ] + [f"    {ct} {code};" for code, (ct, _) in outs] + [
            "  };",
        ]
        for n, ct, _ in ins:
            out.append(f"  typedef {ct} nmk_in_t_{n} __attribute__((ext_vector_type(4)));")
        for code, (ct, _) in outs:
            out.append(f"  typedef {ct} nmk_out_t_{code} __attribute__((ext_vector_type(4)));")
        extra = "".join(f", const {ct} nmk_pf_{n}" for n, ct, _ in ins)
        names = "".join(f", nmk_pf_{n}" for n, _, _ in ins)
        # The careful form is kept out of line (and the closures hold copies,
        # not addresses): inlined, it would cost the plain form registers.
        # With reduction variables there is one form only, inlined, that adds
        # to them where they are.
        reducing = bool(self.reductions)
        out += [
            f"  auto nmk_item = [{'&' if reducing else '='}](const int64_t nmk_gid0, "
            f"auto nmk_careful, bool &nmk_ok{extra}) -> nmk_results {{",
            "    (void)nmk_gid0; (void)nmk_ok;",
            "    nmk_results nmk_out = {};",
        ] + body + [
            "    return nmk_out;",
            "  };",
        ]
        if reducing:
            out += [
                f"  auto nmk_item_careful = [&](const int64_t nmk_gid0{extra}) -> nmk_results {{",
                "    bool nmk_unused = true;",
                f"    return nmk_item(nmk_gid0, nmkjit::Yes(), nmk_unused{names});",
                "  };",
            ]
        else:
            out += [
                f"  auto nmk_item_careful = [=](const int64_t nmk_gid0{extra}) "
                "__attribute__((noinline)) -> nmk_results {",
                "    bool nmk_unused = true;",
                f"    return nmk_item(nmk_gid0, nmkjit::Yes(), nmk_unused{names});",
                "  };",
            ]
        out += [
            "  const bool nmk_words = ((" + " | ".join(
                f"reinterpret_cast<uintptr_t>({p})" for p in pointers) + ") & 15u) == 0;",
            "  const int64_t nmk_nvec = nmk_words ? nmk_gsz0 / 4 : 0;",
            "  const int64_t nmk_lane = nmk_grp0 * nmk_lsz0 + nmk_lid0;",
            "  const int64_t nmk_lanes = int64_t(gridDim.x) * nmk_lsz0;",
        ]
        # (two words of every operand in flight a lane were measured for loops
        # that only reduce: slower, 88 against 79 us for 512 MiB)
        if self.stages_table:
            # Every block copies a table into workgroup memory first, so the
            # launcher runs half the blocks, two trips a lane; the two trips
            # lie 128 pieces (of one word a lane of a block) apart, not a grid
            # apart: the fastest walk measured for such kernels (the
            # Black-Scholes body over 2^24 options: 55.8 against 57.2 us).
            # Written without divisions: one of 64-bit integers is some 150
            # scalar instructions at the head of every wave.
            out += [
                "  const int64_t nmk_sweep = nmk_lanes;    // words a trip of the whole grid takes",
                "  const bool nmk_paired = gridDim.x % 128 == 0 && nmk_nvec > nmk_sweep && "
                "nmk_nvec <= 2 * nmk_sweep;",
                "  const int64_t nmk_step = nmk_paired ? 128 * nmk_lsz0 : nmk_sweep;",
                "  const int64_t nmk_first = nmk_paired ? (((nmk_grp0 >> 7) << 8) + "
                "(nmk_grp0 & 127)) * nmk_lsz0 + nmk_lid0 : nmk_lane;",
                "  const int64_t nmk_behind = nmk_paired ? nmk_first + 2 * nmk_step : nmk_nvec;",
                "  for (int64_t nmk_i = nmk_first; nmk_i < nmk_nvec && nmk_i < nmk_behind; "
                "nmk_i += nmk_step) {",
            ]
        else:
            out.append("  for (int64_t nmk_i = nmk_lane; nmk_i < nmk_nvec; nmk_i += nmk_lanes) {")
        for n, ct, c in ins:
            src = f"reinterpret_cast<const nmk_in_t_{n} *>({c}_p) + nmk_i"
            load = f"__builtin_nontemporal_load({src})" if nt else f"*({src})"
            out.append(f"    const nmk_in_t_{n} nmk_in_{n} = {load};")
        out += [f"    nmk_out_t_{code} nmk_vec_{code};" for code, _ in outs]
        args = "".join(f", nmk_in_{n}[nmk_k]" for n, _, _ in ins)
        keep = [f"      nmk_vec_{code}[nmk_k] = nmk_r.{code};" for code, _ in outs]
        out += [
            "    bool nmk_ok = true;",
            "#pragma unroll",
            "    for (int nmk_k = 0; nmk_k < 4; ++nmk_k) {",
            f"      const nmk_results nmk_r = nmk_item(nmk_i * 4 + nmk_k, nmkjit::No(), nmk_ok"
            f"{args});",
            "      (void)nmk_r;",
        ] + keep + [
            "    }",
        ]
        if self.speculates:
            out += [
                "    if (__builtin_amdgcn_ballot_w64(!nmk_ok) != 0) {",
                "#pragma unroll 1",
                "      for (int nmk_k = 0; nmk_k < 4; ++nmk_k) {",
                f"        const nmk_results nmk_r = nmk_item_careful(nmk_i * 4 + nmk_k{args});",
            ] + ["  " + line for line in keep] + [
                "      }",
                "    }",
            ]
        for code, (_, ptr) in outs:
            dst = f"reinterpret_cast<nmk_out_t_{code} *>({ptr}) + nmk_i"
            out.append(f"    __builtin_nontemporal_store(nmk_vec_{code}, {dst});" if nt else
                       f"    *({dst}) = nmk_vec_{code};")
        scalars = "".join(f", {c}_p[g]" for _, _, c in ins)
        out += [
            "  }",
            "  for (int64_t g = nmk_nvec * 4 + nmk_lane; g < nmk_gsz0; g += nmk_lanes) {",
            f"    const nmk_results nmk_r = nmk_item_careful(g{scalars});",
            "    (void)nmk_r;",
        ] + [f"    {ptr}[g] = nmk_r.{code};" for code, (_, ptr) in outs] + [
            "  }",
        ]
        return out

    def store_here(self, arr_code, elem, value_code, origin=None):
        """Elementwise mode: the store of this work-item's element.  An array
        that is only written, and that no other argument overlaps, is streamed
        past the caches."""
        if self.adjacent and self.emitting:
            # the lane's four values of an output array leave in one store,
            # after the last of them is computed
            if arr_code in self.read_arrays or origin is None:
                raise _NotAdjacent(f"'{arr_code}' is read as well as assigned")
            if self.indent != 2:
                raise _NotAdjacent(f"'{arr_code}' is assigned under a condition")
            pointer = "nmk_ret_p" if origin == "nmk_ret" else f"{self.cname(origin)}_p"
            self.adjacent_outs[arr_code] = (elem.ctype, pointer)
            self.emit(f"nmk_out.{arr_code} = ({elem.ctype})({value_code});")
            return
        terms = [f"nmk_gid{d} * {arr_code}.stride[{d}]" for d in range(self.ndim)]
        dst = f"{arr_code}.p[{' + '.join(terms)}]"
        if self.noalias and self.stream and arr_code not in self.read_arrays:
            last = self.ndim - 1
            # (the returned array is allocated dense by the caller)
            unit = "true" if arr_code == "nmk_ret" else f"{arr_code}.stride[{last}] == 1"
            self.emit(f"NMK_STORE_ALONG{last}(&{dst}, ({elem.ctype})({value_code}), "
                      f"{unit});")
        else:
            self.emit(f"{dst} = {value_code};")

    @staticmethod
    def is_whole_slice(node):
        def full(n):
            return (isinstance(n, ast.Slice) and n.lower is None and n.upper is None
                    and n.step is None) or \
                   (isinstance(n, ast.Constant) and n.value is Ellipsis)
        if isinstance(node, ast.Tuple):
            return all(full(e) for e in node.elts)
        return full(node)

    def expr_Constant(self, node):
        v = node.value
        if v is None:
            return Val(None, None, pyobj=None)
        if isinstance(v, (bool, int, float)):
            return constant(v)
        self.err(node, f"Unsupported constant {v!r}")

    def expr_Name(self, node):
        return self.lookup(node)

    def extent(self, base, k):
        known = base.type.const_shape[k]
        if known is not None:
            return constant(known)
        return Val(f"{base.code}.shape[{k}]", INT64, nonneg=True)

    def expr_Attribute(self, node):
        base = self.expr(node.value)
        if isinstance(base.type, Array):
            if node.attr == "shape":
                items = [self.extent(base, k) for k in range(base.type.ndim)]
                return Val(None, ("tuple",), items=items)
            if node.attr == "ndim":
                return constant(base.type.ndim)
            if node.attr == "size":
                code = " * ".join(self.extent(base, k).code for k in range(base.type.ndim))
                return Val(f"({code})", INT64, nonneg=True)
            self.err(node, f"Unsupported array attribute '{node.attr}'")
        if base.type is None and base.pyobj is not None:
            try:
                return self.from_python(getattr(base.pyobj, node.attr), node)
            except AttributeError:
                self.err(node, f"{base.pyobj!r} has no attribute '{node.attr}'")
        self.err(node, f"Unsupported attribute access '.{node.attr}'")

    def expr_Tuple(self, node):
        return Val(None, ("tuple",), items=[self.expr(e) for e in node.elts])

    def expr_Slice(self, node):
        parts = tuple(self.scalar(p) if p is not None else None
                      for p in (node.lower, node.upper, node.step))
        return Val(None, SliceArg(), slice_parts=parts)

    def expr_UnaryOp(self, node):
        v = self.scalar(node.operand)
        if isinstance(node.op, ast.Not):
            b = self.truth(v)
            if b.const is not None:
                return constant(not b.const)
            return Val(f"(!{b.code})", BOOL)
        if isinstance(node.op, ast.UAdd):
            return cast(v, INT64) if v.type.is_bool else v
        if isinstance(node.op, ast.USub):
            if v.type.is_bool:
                v = cast(v, INT64)
            if v.const is not None:
                return constant(-v.const, v.type)
            return Val(f"(-{v.code})", v.type)
        if isinstance(node.op, ast.Invert):
            if v.type.is_float:
                self.err(node, "~ needs an integer")
            if v.type.is_bool and v.const is None:
                # an element of a boolean array: numpy.invert is logical not
                return Val(f"(!{v.code})", BOOL)
            if v.type.is_bool:
                v = cast(v, INT64)        # ~True of Python is -2
            return Val(f"(~{v.code})", v.type)
        self.err(node, "Unsupported unary operator")

    def truth(self, v):
        if v.type.is_bool:
            return v
        if v.const is not None:
            return constant(bool(v.const))
        return Val(f"({v.code} != 0)", BOOL)

    def expr_BoolOp(self, node):
        vals = [self.scalar(e) for e in node.values]
        if not all(v.type.is_bool for v in vals):
            # Python's and / or return one of the operands, not a truth value
            self.err(node, "'and' / 'or' are supported between boolean values only")
        op = " && " if isinstance(node.op, ast.And) else " || "
        return Val("(" + op.join(v.code for v in vals) + ")", BOOL)

    def expr_Compare(self, node):
        ops = {ast.Lt: "<", ast.LtE: "<=", ast.Gt: ">", ast.GtE: ">=",
               ast.Eq: "==", ast.NotEq: "!="}
        left = self.scalar(node.left)
        parts = []
        for op, right_node in zip(node.ops, node.comparators):
            right = self.scalar(right_node)
            if type(op) not in ops:
                self.err(node, "Unsupported comparison")
            t = self.arith_type(left.type, right.type)
            a, b = cast(left, t), cast(right, t)
            parts.append(f"({a.code} {ops[type(op)]} {b.code})")
            left = right
        return Val("(" + " && ".join(parts) + ")", BOOL)

    def arith_type(self, a, b, arrays=False):
        """Result type of arithmetic on types ``a`` and ``b``.  Between values
        computed from array elements (``arrays``) a float meeting an integer
        keeps its own width, as the reference's array operators do
        (_select_float_type, numpy/funcs.py:402-418: float32 array * 2 and
        float32 array + int array are float32); scalars follow Numba's scalar
        rules (numpy.promote_types)."""
        if arrays and a is not b:
            if a.is_float and not b.is_float:
                return a
            if b.is_float and not a.is_float:
                return b
        t = promote(a, b)
        return INT64 if t.is_bool else t

    def common_type(self, a, b):
        """The type two alternatives (of a selection, a minimum ...) share."""
        if (a.arr or b.arr) and a.type is not b.type:
            if a.type.is_float and not b.type.is_float:
                return a.type
            if b.type.is_float and not a.type.is_float:
                return b.type
        return promote(a.type, b.type)

    def expr_IfExp(self, node):
        c = self.truth(self.scalar(node.test))
        a, b = self.scalar(node.body), self.scalar(node.orelse)
        t = self.common_type(a, b)
        return Val(f"({c.code} ? {cast(a, t).code} : {cast(b, t).code})", t,
                   nonneg=a.nonneg and b.nonneg)

    def expr_BinOp(self, node):
        return self.binop(node.op, self.scalar(node.left), self.scalar(node.right), node)

    def binop(self, op, a, b, node):
        v = self._binop(op, a, b, node)
        v.arr = a.arr or b.arr
        return v

    def _binop(self, op, a, b, node):
        t = self.arith_type(a.type, b.type, a.arr or b.arr)
        if isinstance(op, ast.Div):
            if not t.is_float:
                t = FLOAT64
            x, y = cast(a, t), cast(b, t)
            if t is FLOAT64 and x.const == 1.0 and b.type is FLOAT64 and b.tag and \
                    b.tag[0] == "sqrt":
                # 1.0 / sqrt(z): the reciprocal square root and one correction
                # instead of a square root and a division
                spec = self.speculation()
                return Val(f"nmkjit::rsqrtF64m{spec}({b.tag[1]}, nmk_ok)" if spec else
                           f"nmk::rsqrtF64({b.tag[1]})", t, nonneg=True)
            v = Val(f"({x.code} / {y.code})", t, nonneg=a.nonneg and b.nonneg)
            if t is FLOAT32:
                v.tag = ("quot", x.code, y.code)
            return v
        if isinstance(op, ast.Pow):
            if t.is_float:
                x, y = cast(a, t), cast(b, t)
                if b.const is not None and not isinstance(b.const, bool) and \
                        b.const in (1, 2, 3, 4) and a.const is None:
                    # a small whole power is a product (as NumPy evaluates x ** 2)
                    self.m.counter += 1
                    tmp = f"nmk_pw{self.m.counter}"
                    chain = {1: "{0}", 2: "{0} * {0}", 3: "{0} * {0} * {0}",
                             4: "({0} * {0}) * ({0} * {0})"}[int(b.const)].format(tmp)
                    return Val(f"([&] {{ const {t.ctype} {tmp} = {x.code}; return {chain}; }}())",
                               t, nonneg=int(b.const) % 2 == 0 or a.nonneg)
                return Val(f"pow({x.code}, {y.code})", t)
            x, y = cast(a, t), cast(b, t)
            return Val(f"nmkjit::powInt<{t.ctype}>({x.code}, {y.code})", t,
                       nonneg=a.nonneg)
        if isinstance(op, (ast.BitAnd, ast.BitOr, ast.BitXor, ast.LShift, ast.RShift)):
            if t.is_float:
                self.err(node, "Bitwise operators need integers")
            if a.type.is_bool and b.type.is_bool and not isinstance(op, (ast.LShift, ast.RShift)):
                t = BOOL
            sym = {ast.BitAnd: "&", ast.BitOr: "|", ast.BitXor: "^", ast.LShift: "<<",
                   ast.RShift: ">>"}[type(op)]
            x, y = cast(a, t), cast(b, t)
            return Val(f"(({t.ctype})({x.code} {sym} {y.code}))", t,
                       nonneg=a.nonneg and b.nonneg)
        x, y = cast(a, t), cast(b, t)
        if isinstance(op, (ast.Add, ast.Sub, ast.Mult)):
            sym = {ast.Add: "+", ast.Sub: "-", ast.Mult: "*"}[type(op)]
            if x.const is not None and y.const is not None and t.is_int:
                r = {"+": x.const + y.const, "-": x.const - y.const,
                     "*": x.const * y.const}[sym]
                if -2 ** 63 <= r < 2 ** 63:
                    return constant(r, t)
            nonneg = a.nonneg and b.nonneg and sym != "-"
            code = f"({x.code} {sym} {y.code})"
            if t is FLOAT64 and sym in "+*":
                # 0.5 + 0.5 * erf(x): one table lookup for the whole term
                for half, other in ((x, b), (y, a)):
                    if half.const == 0.5 and other.type is FLOAT64 and other.tag:
                        if sym == "*" and other.tag[0] == "erf":
                            v = Val(code, t)
                            v.tag = ("halferf", other.tag[1])
                            return v
                        if sym == "+" and other.tag[0] == "halferf" and \
                                self.emitting and self.outputs_are_float32():
                            spec = self.speculation()
                            return Val(f"nmkjit::cdfTermF64m{spec}({other.tag[1]}, nmk_ok)" if spec
                                       else f"nmkjit::cdfTermF64({other.tag[1]})", t, nonneg=True)
            gid = None
            if t is INT64:                # id + constant still runs along the id
                if sym in "+-" and a.gid is not None and y.const is not None:
                    gid = a.gid
                elif sym == "+" and b.gid is not None and x.const is not None:
                    gid = b.gid
            if t.dtype.itemsize < 4:      # C promotes narrow integers to int
                code = f"(({t.ctype}){code})"
            v = Val(code, t, nonneg=nonneg)
            v.gid = gid
            return v
        if isinstance(op, ast.FloorDiv):
            if t.is_float:
                return Val(f"nmkjit::floordivFloat<{t.ctype}>({x.code}, {y.code})", t)
            if x.const is not None and y.const is not None and y.const != 0:
                return constant(x.const // y.const, t)
            if a.nonneg and b.nonneg and y.const:
                return Val(f"({x.code} / {y.code})", t, nonneg=True)
            return Val(f"nmkjit::floordivInt<{t.ctype}>({x.code}, {y.code})", t,
                       nonneg=a.nonneg and b.nonneg)
        if isinstance(op, ast.Mod):
            if t.is_float:
                return Val(f"nmkjit::modFloat<{t.ctype}>({x.code}, {y.code})", t,
                           nonneg=b.nonneg)
            if x.const is not None and y.const is not None and y.const != 0:
                return constant(x.const % y.const, t)
            if a.nonneg and b.nonneg and y.const:
                return Val(f"({x.code} % {y.code})", t, nonneg=True)
            return Val(f"nmkjit::modInt<{t.ctype}>({x.code}, {y.code})", t, nonneg=b.nonneg)
        self.err(node, f"Unsupported operator {type(op).__name__}")

    # -- indexing ----------------------------------------------------------
    def index_items(self, node):
        v = self.expr(node)
        return v.items if v.items is not None else [v]

    def normalise_index(self, idx, base, dim):
        idx = cast(idx, INT64) if idx.type is not INT64 else idx
        if idx.const is not None:
            if idx.const < 0:
                idx = Val(f"({base.code}.shape[{dim}] + {idx.code})", INT64)
        elif not idx.nonneg:
            idx = Val(f"nmkjit::wrap({idx.code}, {base.code}.shape[{dim}])", INT64)
        if self.m.boundscheck:
            idx = Val(f"nmkjit::checked({idx.code}, {base.code}.shape[{dim}], nmk_oob)",
                      INT64, nonneg=True)
        return idx

    def subscript(self, node):
        """Returns ("elem", lvalue code, elem type) or ("view", Val)."""
        base = self.expr(node.value)
        if base.items is not None:            # tuple[constant]
            k = self.expr(node.slice)
            if k.const is None:
                self.err(node, "A tuple can only be indexed by a constant")
            return ("value", base.items[k.const])
        if not isinstance(base.type, Array):
            self.err(node, "Only arrays and tuples can be indexed")
        items = self.index_items(node.slice)
        ndim = base.type.ndim
        if len(items) > ndim:
            self.err(node, f"Too many indices for a {ndim}-d array")
        if all(isinstance(i.type, Scalar) for i in items) and len(items) == ndim:
            terms = []
            for d, i in enumerate(items):
                i = self.normalise_index(i, base, d)
                terms.append(f"{i.code} * {base.code}.stride[{d}]")
            # the grid dimension the innermost index runs along, if any
            self.last_elem_gid = i.gid
            self.last_elem_unit = f"{base.code}.stride[{ndim - 1}] == 1"
            return ("elem", f"{base.code}.p[{' + '.join(terms)}]", base.type.elem)
        # a view: integers drop a dimension, slices keep it
        cur, cur_t, dim = base.code, base.type, 0
        for i in items:
            if isinstance(i.type, Scalar):
                i = self.normalise_index(i, Val(cur, cur_t), dim)
                cur = f"nmkjit::subAt({cur}, {dim}, {i.code})"
                cur_t = Array(cur_t.elem, cur_t.ndim - 1, cur_t.space)
            elif isinstance(i.type, SliceArg):
                parts = [cast(p, INT64).code if p is not None else "nmkjit::kNone"
                         for p in i.slice_parts]
                cur = f"nmkjit::slice({cur}, {dim}, {', '.join(parts)})"
                dim += 1
            else:
                self.err(node, "Unsupported index")
        if cur_t.ndim == 0:
            self.err(node, "Too many indices")
        return ("view", Val(cur, cur_t))

    def expr_Subscript(self, node):
        if self.mode == "elementwise" and self.is_whole_slice(node.slice):
            return self.expr(node.value)          # a[:] is a itself
        param = self.ahead_nodes.get(id(node))
        if param is not None:
            t = self.arg_types[self.params.index(param)]
            self.prefetched[param] = t
            return Val(f"nmk_pf_{param}", t.elem)
        kind, *rest = self.subscript(node)
        if kind == "elem":
            code, elem = rest
            return Val(code, elem)
        return rest[0]

    # -- calls -------------------------------------------------------------
    def expr_Call(self, node):
        fn = self.expr(node.func)
        if fn.type is not None or fn.pyobj is None:
            self.err(node, "Only functions known at compile time can be called")
        obj = fn.pyobj
        kwargs = {k.arg: k.value for k in node.keywords}
        stubs = self.m.stubs
        ids = {
            stubs.get_global_id: ("gid", True), stubs.get_local_id: ("lid", True),
            stubs.get_group_id: ("grp", True), stubs.get_global_size: ("gsz", True),
            stubs.get_local_size: ("lsz", True),
        }
        if inspect.isfunction(obj) and obj in ids:
            axis = self.expr(node.args[0])
            if axis.const is None or not 0 <= axis.const <= 2:
                self.err(node, "The axis must be a constant 0, 1 or 2")
            if ids[obj][0] in ("lid", "grp", "lsz"):
                self.m.communicates = True
            v = Val(f"nmk_{ids[obj][0]}{axis.const}", INT64, nonneg=True)
            if ids[obj][0] == "gid":
                v.gid = axis.const
            return v
        if obj is stubs.atomic.add or obj is stubs.atomic.sub:
            return self.call_atomic(node, obj is stubs.atomic.sub)
        if obj is stubs.barrier or obj is stubs.mem_fence:
            self.m.communicates = True
            flags = node.args[0] if node.args else kwargs.get("flags")
            if flags is not None:
                f = self.expr(flags)
                if f.const is None and not (f.type is None and f.pyobj is None):
                    self.err(node, "The fence flags must be a constant")
            self.emit("__syncthreads();" if obj is stubs.barrier else
                      "__threadfence_block();")
            return Val(None, None, pyobj=None)
        if obj is stubs.local.array or obj is stubs.private.array:
            self.err(node, "local.array / private.array must be assigned to a variable")
        for opname in _GROUP_OPS:
            if obj is getattr(stubs.group, "reduce_" + opname):
                return self.call_group(node, opname)
        if obj is stubs.kernel_func:
            self.err(node, "kernel_func cannot be called inside a kernel")
        if isinstance(obj, type) and obj in _CAST_TYPES:
            if len(node.args) != 1:
                self.err(node, "A cast takes one argument")
            return cast(self.scalar(node.args[0]), _CAST_TYPES[obj])
        if obj is abs or obj is np.abs or obj is np.absolute or obj is math.fabs:
            v = self.scalar(node.args[0])
            if obj is math.fabs and not v.type.is_float:
                v = cast(v, FLOAT64)
            if v.type.is_float:
                return Val(f"fabs({v.code})", v.type, nonneg=True)
            if v.type.is_bool or v.type.kind == "u":
                return v
            return Val(f"({v.code} < 0 ? ({v.type.ctype})(-{v.code}) : {v.code})", v.type,
                       nonneg=True)
        if any(obj is f for f in (min, max, np.minimum, np.maximum)):
            vals = [self.scalar(a) for a in node.args]
            if len(vals) < 2:
                self.err(node, "min/max need at least two scalar arguments")
            is_min = obj is min or obj is np.minimum
            acc = vals[0]
            for v in vals[1:]:
                t = self.common_type(acc, v)
                a, b = cast(acc, t), cast(v, t)
                cmp = "<" if is_min else ">"
                # Python keeps the first of equal arguments
                acc = Val(f"({b.code} {cmp} {a.code} ? {b.code} : {a.code})", t,
                          nonneg=(acc.nonneg and v.nonneg) if is_min else
                          (acc.nonneg or v.nonneg))
            return acc
        if obj is len:
            v = self.expr(node.args[0])
            if isinstance(v.type, Array):
                return self.extent(v, 0)
            if v.items is not None:
                return constant(len(v.items))
            self.err(node, "len() needs an array or a tuple")
        if obj is range:
            self.err(node, "range() is only supported as the iterable of a for loop")
        if len(node.args) == 1 and not kwargs:
            # def f(x): return math.erf(x) -- and its vectorize()d form -- is
            # the function it wraps
            obj = _unwrapped_unary(obj)
        name = getattr(obj, "__name__", None)
        mod = getattr(obj, "__module__", None)
        is_np = isinstance(obj, np.ufunc) or mod == "numpy"
        if (mod == "math" or is_np) and name in _UNARY_MATH and len(node.args) == 1:
            v = self.scalar(node.args[0])
            t = FLOAT32 if v.type is FLOAT32 else FLOAT64
            v = cast(v, t)
            spec = self.speculation()
            if name == "sqrt" and t is FLOAT64:
                # same rounding as the library routine at half its cost
                r = Val(f"nmkjit::sqrtF64m{spec}({v.code}, nmk_ok)" if spec else
                        f"nmk::sqrtF64({v.code})", t, nonneg=True)
                r.tag = ("sqrt", v.code)
                return r
            if name == "erf" and t is FLOAT64:
                # table in workgroup memory, loaded at kernel entry
                r = Val(f"nmkjit::erfF64({v.code})", t)
                r.tag = ("erf", v.code)
                return r
            if name == "log" and t is FLOAT32 and v.tag and v.tag[0] == "quot":
                # log(a / b): the quotient feeds nothing else
                _, qa, qb = v.tag
                return Val(f"nmkjit::logQuotientF32m{spec}({qa}, {qb}, nmk_ok)" if spec else
                           f"nmk::logQuotientF32({qa}, {qb})", t)
            if name in ("log", "exp") and t is FLOAT32:
                # the library routine's own arithmetic, its range handling
                # only where the argument needs it
                return Val(f"nmkjit::{name}F32m{spec}({v.code}, nmk_ok)" if spec else
                           f"nmk::{name}F32({v.code})", t, nonneg=name == "exp")
            return Val(f"{_UNARY_MATH[name]}({v.code})", t)
        if (mod == "math" or is_np) and name in _ROUNDING and len(node.args) == 1:
            v = self.scalar(node.args[0])
            if not v.type.is_float:
                return cast(v, INT64) if mod == "math" else cast(v, FLOAT64)
            r = Val(f"{_ROUNDING[name]}({v.code})", v.type)
            return cast(r, INT64) if mod == "math" else r
        if is_np and name in _UFUNC_BINOPS and len(node.args) == 2:
            return self.binop(_UFUNC_BINOPS[name](), self.scalar(node.args[0]),
                              self.scalar(node.args[1]), node)
        if is_np and name in _UFUNC_COMPARE and len(node.args) == 2:
            return self.expr(ast.copy_location(ast.Compare(
                left=node.args[0], ops=[_UFUNC_COMPARE[name]()],
                comparators=[node.args[1]]), node))
        if is_np and name in _UFUNC_UNARY and len(node.args) == 1:
            return self.expr(ast.copy_location(ast.UnaryOp(
                op=_UFUNC_UNARY[name](), operand=node.args[0]), node))
        if is_np and name in ("logical_and", "logical_or", "logical_xor") and \
                len(node.args) == 2:
            a = self.truth(self.scalar(node.args[0]))
            b = self.truth(self.scalar(node.args[1]))
            sym = {"logical_and": "&&", "logical_or": "||", "logical_xor": "!="}[name]
            return Val(f"({a.code} {sym} {b.code})", BOOL)
        if is_np and name == "clip" and len(node.args) == 3:
            # min(a_max, max(a, a_min)) in the operands' common type
            # (reference: numpy/funcs.py:571-578)
            a, lo, hi = (self.scalar(x) for x in node.args)
            t = self.common_type(a, lo)
            t = self.common_type(Val("", t), hi) if not (a.arr or lo.arr) else \
                self.arith_type(t, hi.type, True)
            t = INT64 if t.is_bool else t
            a, lo, hi = cast(a, t), cast(lo, t), cast(hi, t)
            # (a NaN element stays NaN, as in NumPy)
            inner = f"({a.code} < {lo.code} ? {lo.code} : {a.code})"
            return Val(f"({inner} > {hi.code} ? {hi.code} : {inner})", t,
                       nonneg=hi.nonneg and (a.nonneg or lo.nonneg))
        if (mod == "math" or is_np) and name in _BINARY_MATH and len(node.args) == 2:
            a, b = self.scalar(node.args[0]), self.scalar(node.args[1])
            t = self.common_type(a, b)
            t = t if t.is_float else FLOAT64
            return Val(f"{_BINARY_MATH[name]}({cast(a, t).code}, {cast(b, t).code})", t)
        if mod == "math" and name in ("isnan", "isinf", "isfinite") or \
                is_np and name in ("isnan", "isinf", "isfinite"):
            v = self.scalar(node.args[0])
            if not v.type.is_float:
                return constant(name == "isfinite")
            return Val(f"(bool)__builtin_{name}({v.code})", BOOL)
        if is_np and name == "where" and len(node.args) == 3:
            c = self.truth(self.scalar(node.args[0]))
            a, b = self.scalar(node.args[1]), self.scalar(node.args[2])
            t = self.common_type(a, b)
            return Val(f"({c.code} ? {cast(a, t).code} : {cast(b, t).code})", t,
                       nonneg=a.nonneg and b.nonneg)
        if is_np and name == "square" and len(node.args) == 1:
            v = self.scalar(node.args[0])
            return self.binop(ast.Mult(), v, v, node)
        if is_np and name == "negative" and len(node.args) == 1:
            v = self.scalar(node.args[0])
            return Val(f"(-{v.code})", INT64 if v.type.is_bool else v.type)
        if getattr(obj, "_nmk_vectorized", None) is not None:
            return self.call_device(node, obj._nmk_vectorized)
        if inspect.isfunction(obj):
            return self.call_device(node, obj)
        self.err(node, f"Unsupported call target {obj!r}")

    def call_atomic(self, node, negate):
        if len(node.args) != 3:
            self.err(node, "atomic.add/sub take (array, index, value)")
        arr = self.expr(node.args[0])
        if not isinstance(arr.type, Array):
            self.err(node, "The first argument of an atomic must be an array")
        elem = arr.type.elem
        if elem not in (INT32, INT64, FLOAT32, FLOAT64):
            self.err(node, f"Atomics on {elem} are not supported")
        items = self.index_items(node.args[1])
        if len(items) != arr.type.ndim:
            self.err(node, "An atomic needs a full index")
        terms = []
        for d, i in enumerate(items):
            i = self.normalise_index(i, arr, d)
            terms.append(f"{i.code} * {arr.code}.stride[{d}]")
        val = cast(self.scalar(node.args[2]), elem)
        v = f"(-{val.code})" if negate else val.code
        return Val(f"nmkjit::atomicAddT(&{arr.code}.p[{' + '.join(terms)}], "
                   f"({elem.ctype}){v})", elem)

    def call_group(self, node, opname):
        self.m.communicates = True
        if not self.is_kernel:
            self.err(node, "group reductions are only supported in the kernel body")
        v = self.scalar(node.args[0])
        t = INT64 if v.type.is_bool else v.type
        if t.dtype.itemsize < 4:
            t = INT32 if t.kind == "i" else UINT32
        v = cast(v, t)
        if node not in self.site_names:
            self.site_names[node] = self.m.fresh("nmk_group")
        slot = self.site_names[node]
        if self.emitting and all(s[0] != slot for s in self.group_sites):
            neutral = _GROUP_NEUTRAL[opname](t)
            if t is FLOAT32 and "inf" in neutral:
                neutral = neutral.replace("__builtin_inf()", "__builtin_inff()")
            self.group_sites.append((slot, t, neutral))
        tmp = self.m.fresh("nmk_t")
        self.emit(f"const {t.ctype} {tmp} = nmkjit::groupReduce({slot}, {v.code}, "
                  f"nmk_clipped != 0, nmkjit::{_GROUP_OPS[opname]}());")
        return Val(tmp, t)

    def call_device(self, node, obj):
        if node.keywords:
            self.err(node, "Keyword arguments are not supported in device calls")
        args = [self.expr(a) for a in node.args]
        if self.mode == "elementwise":
            args = [self.element_here(a, node) if isinstance(a.type, Array) else a
                    for a in args]
        for a in args:
            if not isinstance(a.type, (Scalar, Array)):
                self.err(node, "Device functions take scalars and arrays")
        key = (obj, tuple(type_key(a.type) for a in args))
        if key in self.m.in_progress:
            self.err(node, "Recursive device functions are not supported")
        if key not in self.m.device_funcs:
            self.m.in_progress.add(key)
            try:
                tr = FunctionTranslator(self.m, obj, [a.type for a in args], False)
                name = self.m.fresh(f"nmk_dev_{_safe(obj.__name__)}_")
                code, ret = tr.translate_device(name)
            finally:
                self.m.in_progress.discard(key)
            self.m.device_funcs[key] = (name, ret)
            self.m.device_code.append(code)
        name, ret = self.m.device_funcs[key]
        actual = [a.code for a in args] + (["nmk_oob"] if self.m.boundscheck else [])
        call = f"{name}({', '.join(actual)})"
        if ret is None:
            self.emit(call + ";")
            return Val(None, None, pyobj=None)
        return Val(call, ret)

    # -- statements --------------------------------------------------------
    def stmt(self, node):
        method = getattr(self, "stmt_" + type(node).__name__, None)
        if method is None:
            self.err(node, f"Unsupported statement: {type(node).__name__}")
        try:
            method(node)
        except _Deferred:
            if self.emitting:
                raise
            self.deferred = True

    def block(self, stmts):
        self.indent += 1
        for s in stmts:
            self.stmt(s)
        self.indent -= 1

    def stmt_Pass(self, node):
        pass

    def stmt_Expr(self, node):
        if isinstance(node.value, ast.Constant):
            return                                     # docstring
        v = self.expr(node.value)
        if v.code is not None and isinstance(v.type, Scalar):
            self.emit(f"(void)({v.code});")

    def bind(self, name, t, node):
        """Records that ``name`` receives a value of type ``t``."""
        old = self.env.get(name)
        if name in self.params and not isinstance(old, Scalar):
            self.err(node, f"Cannot rebind the array argument '{name}'")
        if isinstance(t, Scalar):
            if old is None:
                new = t
            elif isinstance(old, Scalar):
                new = promote(old, t)
            else:
                self.err(node, f"'{name}' is used both as a scalar and as an array")
            if new is not old:
                self.env[name] = new
                self.changed = True
        else:
            if isinstance(old, Scalar):
                self.err(node, f"'{name}' is used both as a scalar and as an array")
            if old is not None and old != t:
                self.err(node, f"'{name}' is bound to arrays of different types")
            if old is None:
                self.env[name] = t
                self.changed = True

    def special_array_call(self, value):
        """local.array / private.array call nodes, else None."""
        if not isinstance(value, ast.Call):
            return None
        try:
            fn = self.expr(value.func)
        except (_Deferred, KernelCompileError):
            return None
        stubs = self.m.stubs
        if fn.pyobj is stubs.local.array:
            return "local"
        if fn.pyobj is stubs.private.array:
            return "private"
        return None

    def array_alloc(self, name, node, space):
        call = node.value
        args = list(call.args)
        kwargs = {k.arg: k.value for k in call.keywords}
        shape_node = args[0] if args else kwargs.get("shape")
        dtype_node = args[1] if len(args) > 1 else kwargs.get("dtype")
        if shape_node is None or dtype_node is None:
            self.err(node, "array(shape, dtype) needs both arguments")
        shape = self.expr(shape_node)
        dims = shape.items if shape.items is not None else [shape]
        if any(d.const is None or isinstance(d.const, float) for d in dims):
            self.err(node, "The shape of a local or private array must be constant")
        dims = tuple(int(d.const) for d in dims)
        if isinstance(dtype_node, ast.Constant) and isinstance(dtype_node.value, str):
            elem = scalar_of(dtype_node.value)
        else:
            dt = self.expr(dtype_node)
            if dt.pyobj is None:
                self.err(node, "The dtype must be a NumPy type or its name")
            elem = scalar_of(dt.pyobj)
        t = Array(elem, len(dims), space)
        self.bind(name, t, node)
        if not self.emitting:
            return
        strides = []
        acc = 1
        for d in reversed(dims):
            strides.insert(0, acc)
            acc *= d
        total = acc
        shape_c = ", ".join(str(d) for d in dims)
        stride_c = ", ".join(str(s) for s in strides)
        c = self.cname(name)
        if space == "local":
            self.m.communicates = True
            if not self.is_kernel:
                self.err(node, "local.array is only supported in the kernel body")
            k = len(self.local_arrays)
            self.local_arrays.append((elem, dims))
            self.emit(f"{c} = {{reinterpret_cast<{elem.ctype} *>(nmk_dyn_lds + nmk_lds{k}), "
                      f"{{{shape_c}}}, {{{stride_c}}}}};")
        else:
            store = self.m.fresh("nmk_priv")
            self.private_decls.append(f"{elem.ctype} {store}[{max(total, 1)}] = {{}};")
            self.emit(f"{c} = {{{store}, {{{shape_c}}}, {{{stride_c}}}}};")

    def stmt_Assign(self, node):
        if len(node.targets) != 1:
            self.err(node, "Chained assignment is not supported")
        target = node.targets[0]
        if isinstance(target, ast.Name) and target.id in self.reductions and \
                id(node) in self.top_level:
            v = self.scalar(node.value)           # the host applies the start value
            self.bind(target.id, v.type, node)
            self.maybe_negative.add(target.id)
            return
        if isinstance(target, ast.Name):
            space = self.special_array_call(node.value)
            if space:
                return self.array_alloc(target.id, node, space)
            v = self.expr(node.value)
            self.assign_name(target.id, v, node)
        elif isinstance(target, ast.Subscript):
            v = self.expr(node.value)
            self.assign_subscript(target, v, node)
        elif isinstance(target, ast.Tuple):
            v = self.expr(node.value)
            if v.items is None or len(v.items) != len(target.elts):
                self.err(node, "Tuple assignment needs a tuple of the same length")
            if not all(isinstance(e, ast.Name) for e in target.elts):
                self.err(node, "Only names can be unpacked into")
            # evaluate everything first (a, b = b, a)
            tmps = []
            for e, item in zip(target.elts, v.items):
                if isinstance(item.type, Scalar) and self.emitting:
                    tmp = self.m.fresh("nmk_t")
                    self.emit(f"const {item.type.ctype} {tmp} = {item.code};")
                    item = Val(tmp, item.type, const=item.const, nonneg=item.nonneg)
                tmps.append(item)
            for e, item in zip(target.elts, tmps):
                self.assign_name(e.id, item, node)
        else:
            self.err(node, "Unsupported assignment target")

    def assign_name(self, name, v, node):
        if v.items is not None:
            if name in self.env and not (isinstance(self.env[name], tuple)):
                self.err(node, f"'{name}' changes from a scalar to a tuple")
            # the scalar elements are stored now (a later change of what they
            # were computed from must not show); views and slices are kept as
            # expressions
            items = []
            for k, item in enumerate(v.items):
                if isinstance(item.type, Scalar) and item.const is None:
                    slot = f"{name}.{k}"
                    self.assigned.add(slot)
                    self.bind(slot, item.type, node)
                    if not item.nonneg:
                        self.maybe_negative.add(slot)
                    if self.emitting:
                        self.emit(f"{self.cname(slot)} = {cast(item, self.env[slot]).code};")
                    items.append(slot)
                else:
                    items.append(item)
            old = self.tuple_vars.get(name)
            if old is not None and len(old) != len(items):
                self.err(node, f"'{name}' is bound to tuples of different lengths")
            self.tuple_vars[name] = items
            self.env[name] = ("tuple",)
            return
        if isinstance(v.type, SliceArg):
            self.err(node, "Slices cannot be stored in variables")
        if v.type is None:
            self.err(node, "This value cannot be assigned to a variable")
        self.bind(name, v.type, node)
        if v.arr and name not in self.array_valued:
            self.array_valued.add(name)
            self.changed = True
        if isinstance(v.type, Array) and v.origin is not None and \
                self.store_count.get(name) == 1 and id(node) in self.top_level and \
                name not in self.params:
            self.view_origin[name] = v.origin      # P = price: P is price
        if isinstance(v.type, Scalar):
            if (v.const is not None and self.store_count.get(name) == 1 and
                    id(node) in self.top_level and name not in self.params):
                self.const_vars[name] = v.const
            if (v.gid is not None and self.store_count.get(name) == 1 and
                    id(node) in self.top_level and name not in self.params):
                self.gid_vars[name] = v.gid
            if not v.nonneg:
                self.maybe_negative.add(name)
            if self.emitting:
                t = self.env[name]
                self.emit(f"{self.cname(name)} = {cast(v, t).code};")
        else:
            self.emit(f"{self.cname(name)} = {v.code};")

    def assign_subscript(self, target, v, node):
        if self.mode == "elementwise" and self.is_whole_slice(target.slice):
            arr = self.expr(target.value)
            if not isinstance(arr.type, Array):
                self.err(node, "Only arrays can be assigned through [:]")
            if isinstance(v.type, Array):
                v = self.element_here(v, node)
            if arr.type.ndim != self.ndim:
                self.err(node, "Only whole arrays of the iteration space can be assigned")
            self.written_arrays.add(arr.code)
            if arr.origin is not None:
                self.written_origins.add(arr.origin)
            else:
                self.opaque_write = True
            self.store_here(arr.code, arr.type.elem, cast(v, arr.type.elem).code,
                            origin=arr.origin)
            return
        kind, *rest = self.subscript(target)
        if kind != "elem":
            self.err(node, "Only single elements can be assigned")
        code, elem = rest
        if not isinstance(v.type, Scalar):
            self.err(node, "Only scalars can be stored into an array element")
        if self.adjacent and self.emitting:
            # a prange(n) loop that stores p[i] = value for its own i, in the
            # loop body itself: the lane's four values leave in one store
            name = target.value.id if isinstance(target.value, ast.Name) else None
            t = dict(zip(self.params, self.arg_types)).get(name)
            if not (self.mode == "parallel" and self.unit_loop_var is not None and
                    isinstance(target.slice, ast.Name) and
                    target.slice.id == self.unit_loop_var and
                    self.loop_kinds == ["grid"] and self.indent == 2 and
                    name in self.store_only_params() and isinstance(t, Array) and
                    t.ndim == 1 and t.layout == "C"):
                raise _NotAdjacent("the body stores single elements")
            c = self.cname(name)
            self.adjacent_outs[c] = (elem.ctype, f"{c}_p")
            self.emit(f"nmk_out.{c} = ({elem.ctype})({cast(v, elem).code});")
            return
        if self.noalias and self.stream and self.last_elem_gid is not None and \
                isinstance(target.value, ast.Name) and \
                target.value.id in self.store_only_params():
            # read by nobody in this launch: past the caches when adjacent
            # lanes write adjacent elements (see translate_kernel)
            self.emit(f"NMK_STORE_ALONG{self.last_elem_gid}(&{code}, "
                      f"({elem.ctype})({cast(v, elem).code}), {self.last_elem_unit});")
            return
        self.emit(f"{code} = {cast(v, elem).code};")

    def store_only_params(self):
        """Array parameters of a kernel (or loop function) that the body only
        stores elements into: every use is ``p[...] = value``, ``p.shape`` /
        ``p.size`` / ``p.ndim`` / ``p.dtype`` or ``len(p)``.  Handing the array
        to anything else (a view, another name, a call, an atomic, ``+=``)
        counts as reading it."""
        if self._store_only is not None:
            return self._store_only
        names = {p for p, t in zip(self.params, self.arg_types)
                 if isinstance(t, Array) and t.space == "global"}
        if not self.is_kernel:
            names = set()
        parents = {}
        for parent in ast.walk(self.node):
            for child in ast.iter_child_nodes(parent):
                parents[id(child)] = parent
        for n in ast.walk(self.node):
            if not (isinstance(n, ast.Name) and n.id in names):
                continue
            parent = parents.get(id(n))
            if isinstance(n.ctx, ast.Load):
                if isinstance(parent, ast.Subscript) and parent.value is n and \
                        isinstance(parent.ctx, ast.Store) and \
                        isinstance(parents.get(id(parent)), ast.Assign):
                    continue
                if isinstance(parent, ast.Attribute) and \
                        parent.attr in ("shape", "size", "ndim", "dtype"):
                    continue
                if isinstance(parent, ast.Call) and isinstance(parent.func, ast.Name) and \
                        parent.func.id == "len" and len(parent.args) == 1:
                    continue
            names.discard(n.id)
        self._store_only = names
        return names

    def stmt_AugAssign(self, node):
        if isinstance(node.target, ast.Name):
            cur = self.expr(ast.Name(id=node.target.id, ctx=ast.Load(),
                                     lineno=node.lineno, col_offset=0))
            if not isinstance(cur.type, Scalar):
                self.err(node, "Augmented assignment needs a scalar variable")
            v = self.binop(node.op, cur, self.scalar(node.value), node)
            self.assign_name(node.target.id, v, node)
        elif isinstance(node.target, ast.Subscript):
            kind, *rest = self.subscript(node.target)
            if kind != "elem":
                self.err(node, "Only single elements can be updated")
            code, elem = rest
            v = self.binop(node.op, Val(code, elem), self.scalar(node.value), node)
            self.emit(f"{code} = {cast(v, elem).code};")
        else:
            self.err(node, "Unsupported augmented assignment target")

    def stmt_If(self, node):
        c = self.truth(self.scalar(node.test))
        self.emit(f"if ({c.code}) {{")
        self.block(node.body)
        if node.orelse:
            self.emit("} else {")
            self.block(node.orelse)
        self.emit("}")

    def stmt_For(self, node):
        if node.orelse:
            self.err(node, "for ... else is not supported")
        it = node.iter
        is_range = is_prange = False
        if isinstance(it, ast.Call) and not it.keywords and 1 <= len(it.args) <= 3:
            try:
                fn = self.expr(it.func)
            except KernelCompileError:
                fn = None
            if fn is not None and fn.type is None:
                is_range = fn.pyobj is range
                is_prange = bool(getattr(fn.pyobj, "_nmk_prange", False))
        if not (is_range or is_prange):
            self.err(node, "Only 'for x in range(...)' loops are supported")
        if not isinstance(node.target, ast.Name):
            self.err(node, "The loop variable must be a name")
        a = [cast(self.scalar(x), INT64) for x in it.args]
        start = a[0] if len(a) > 1 else constant(0)
        stop = a[1] if len(a) > 1 else a[0]
        step = a[2] if len(a) > 2 else constant(1)
        name = node.target.id
        depth = self.grid_depth(node) if (is_prange and self.mode == "parallel") else None
        if depth is not None:
            # a grid loop: work-item g of dimension `depth` runs iteration g
            if step.const is None or step.const <= 0:
                self.err(node, "A prange step must be a positive constant")
            if depth == 0:
                if self.range_source is not None and self.range_source[0] is not node:
                    self.err(node, "Only one top-level prange loop is offloaded")
                self.range_source = (node, [ast.unparse(x) for x in it.args])
                self.grid_loops = [node]
                self.grid_sources = [self.range_source[1]]
            elif node not in self.grid_loops:
                self.grid_loops.append(node)
                self.grid_sources.append([ast.unparse(x) for x in it.args])
            self.bind(name, INT64, node)
            if not start.nonneg:
                self.maybe_negative.add(name)
            if step.const == 1 and self.store_count.get(name) == 1:
                self.gid_vars[name] = depth
            if depth == 0 and self.ndim == 1 and self.noalias and start.const == 0 and \
                    step.const == 1 and self.elements_per_thread > 1 and \
                    not self.m.boundscheck:
                # what every iteration reads at its own index is loaded for
                # all of a lane's iterations before the first one runs
                self.ahead_nodes = self.loads_ahead_of(node)
                if self.store_count.get(name) == 1:
                    self.unit_loop_var = name      # iteration g is work-item g
            if self.emitting:
                self.emit(f"{self.cname(name)} = {start.code} + nmk_gid{depth} * {step.code};")
            self.indent -= 1
            self.loop_kinds.append("grid")
            self.block(node.body)
            self.loop_kinds.pop()
            self.indent += 1
            return
        self.bind(name, INT64, node)
        if not (start.nonneg and step.const is not None and step.const > 0):
            self.maybe_negative.add(name)
        itv = self.m.fresh("nmk_it")
        stopv, stepv = self.m.fresh("nmk_stop"), self.m.fresh("nmk_step")
        self.emit("{")
        self.indent += 1
        self.emit(f"const int64_t {stopv} = {stop.code}, {stepv} = {step.code};")
        if step.const is not None and step.const > 0:
            cond = f"{itv} < {stopv}"
        elif step.const is not None and step.const < 0:
            cond = f"{itv} > {stopv}"
        else:
            cond = f"({stepv} > 0 ? {itv} < {stopv} : {itv} > {stopv})"
        self.emit(f"for (int64_t {itv} = {start.code}; {cond}; {itv} += {stepv}) {{")
        self.indent += 1
        if self.emitting:
            t = self.env[name]
            self.emit(f"{self.cname(name)} = ({t.ctype}){itv};")
        self.indent -= 1
        self.loop_kinds.append("sequential")
        self.block(node.body)
        self.loop_kinds.pop()
        self.emit("}")
        self.indent -= 1
        self.emit("}")

    def loads_ahead_of(self, loop):
        """prange loop of a 1-d launch, iterations 0, 1, 2 ...: the reads
        ``p[i]`` of parameter arrays that every iteration performs, whatever
        its data -- in a statement of the loop body itself, outside ``x if c
        else y`` and ``and`` / ``or``, in a body without continue / break /
        return.  ``p`` must be used for nothing but element reads and its
        shape in the whole function.  Returns {id(subscript node): parameter}."""
        var = loop.target.id
        if self.store_count.get(var) != 1:
            return {}
        for n in ast.walk(ast.Module(body=loop.body, type_ignores=[])):
            if isinstance(n, (ast.Continue, ast.Break, ast.Return)):
                return {}
        arrays = {p for p, t in zip(self.params, self.arg_types)
                  if isinstance(t, Array) and t.space == "global" and t.ndim == 1 and
                  t.elem.ctype in self._PREFETCH_CTYPES and not self.store_count.get(p)}
        parents = {}
        for parent in ast.walk(self.node):
            for child in ast.iter_child_nodes(parent):
                parents[id(child)] = parent
        for n in ast.walk(self.node):
            if isinstance(n, ast.Name) and n.id in arrays:
                parent = parents.get(id(n))
                if isinstance(parent, ast.Subscript) and parent.value is n and \
                        isinstance(parent.ctx, ast.Load):
                    continue
                if isinstance(parent, ast.Attribute) and \
                        parent.attr in ("shape", "size", "ndim", "dtype"):
                    continue
                if isinstance(parent, ast.Call) and isinstance(parent.func, ast.Name) and \
                        parent.func.id == "len" and len(parent.args) == 1:
                    continue
                arrays.discard(n.id)
        found = {}

        def scan(n):
            if isinstance(n, ast.IfExp):
                scan(n.test)
                return
            if isinstance(n, ast.BoolOp):
                scan(n.values[0])
                return
            if isinstance(n, (ast.Lambda, ast.ListComp, ast.GeneratorExp, ast.SetComp,
                              ast.DictComp)):
                return
            if isinstance(n, ast.Subscript) and isinstance(n.ctx, ast.Load) and \
                    isinstance(n.value, ast.Name) and n.value.id in arrays and \
                    isinstance(n.slice, ast.Name) and n.slice.id == var:
                found[id(n)] = n.value.id
                return
            for child in ast.iter_child_nodes(n):
                scan(child)

        for stmt in loop.body:
            if isinstance(stmt, (ast.Assign, ast.AugAssign, ast.AnnAssign, ast.Expr)):
                scan(stmt.value)
        return found

    def grid_depth(self, node):
        """Which grid dimension a prange loop is, or None for a sequential one:
        the top-level loop is dimension 0; a prange loop that is the whole body
        of grid loop k is dimension k + 1 (a perfect nest), while the launch
        has that many dimensions."""
        if id(node) in self.top_level:
            return 0
        for k, outer in enumerate(self.grid_loops):
            if k + 1 < self.ndim and len(outer.body) == 1 and outer.body[0] is node:
                return k + 1
        return None

    def stmt_While(self, node):
        if node.orelse:
            self.err(node, "while ... else is not supported")
        c = self.truth(self.scalar(node.test))
        self.emit(f"while ({c.code}) {{")
        self.loop_kinds.append("sequential")
        self.block(node.body)
        self.loop_kinds.pop()
        self.emit("}")

    def stmt_Break(self, node):
        if self.loop_kinds and self.loop_kinds[-1] == "grid":
            self.err(node, "A prange loop cannot be left with break")
        self.emit("break;")

    def stmt_Continue(self, node):
        # an iteration of a prange loop is one call of the work-item body
        grid = self.loop_kinds and self.loop_kinds[-1] == "grid"
        self.emit("return;" if grid else "continue;")

    def stmt_Return(self, node):
        if node is self.return_node:
            return                                 # evaluated by the host
        if node.value is None or (isinstance(node.value, ast.Constant) and
                                  node.value.value is None):
            if not self.is_kernel and self.ret_type is not None:
                self.err(node, "A device function must return a value on every path")
            self.emit("return;")
            return
        if self.mode == "elementwise":
            if id(node) not in self.top_level:
                self.err(node, "An elementwise function returns at its end only")
            v = self.scalar(node.value)
            if self.ret_type is None:
                self.ret_type = v.type
                self.changed = True
            elif self.ret_type is not v.type:
                self.err(node, "An elementwise function has one return statement")
            self.store_here("nmk_ret", self.ret_type, v.code, origin="nmk_ret")
            return
        if self.is_kernel:
            self.err(node, "A kernel cannot return a value")
        v = self.scalar(node.value)
        new = v.type if self.ret_type is None else promote(self.ret_type, v.type)
        if new is not self.ret_type:
            self.ret_type = new
            self.changed = True
        self.emit(f"return {cast(v, self.ret_type).code};")

    # -- driving -----------------------------------------------------------
    def infer(self, body):
        """Fixed point of the variable types."""
        self.tuple_vars = {}
        self.maybe_negative = set(self.params)
        self.nonneg_vars = set()
        for _ in range(12):
            self.changed = False
            self.deferred = False
            self.emitting = False
            for s in body:
                self.stmt(s)
            if not self.changed:
                break
        else:
            raise KernelCompileError("Type inference did not converge")
        missing = [n for n in self.assigned if n not in self.env]
        if self.deferred and missing:
            raise KernelCompileError(
                f"{self.func.__name__}: cannot type {', '.join(sorted(missing))} "
                "(used before assignment?)")
        # Which integer variables can never be negative (their indices need no
        # wrap-around): the greatest fixed point, starting from "all of them".
        scalars = {n for n, t in self.env.items()
                   if isinstance(t, Scalar) and n not in self.params}
        self.nonneg_vars = set(scalars)
        for _ in range(12):
            self.maybe_negative = set(self.params)
            for s in body:
                self.stmt(s)
            new = scalars - self.maybe_negative
            if new == self.nonneg_vars:
                break
            self.nonneg_vars = new
        else:
            self.nonneg_vars = set()

    def body_stmts(self):
        if isinstance(self.node, ast.Lambda):
            if self._lambda_body is None:
                self._lambda_body = [ast.Return(value=self.node.body,
                                                lineno=self.node.lineno, col_offset=0)]
                self.top_level.add(id(self._lambda_body[0]))
            return self._lambda_body
        return self.node.body

    def declarations(self):
        out = []
        for name in sorted(self.assigned):
            t = self.env.get(name)
            if name in self.reductions:
                continue                           # lives at kernel scope
            if isinstance(t, Scalar):
                out.append(f"{t.ctype} {self.cname(name)} = 0;")
            elif isinstance(t, Array):
                out.append(f"{t.ctype()} {self.cname(name)} = {{}};")
        return out

    def run_emit(self, body):
        self.emitting = True
        self.prefetched = {}        # (the passes before knew less of what is written)
        self.adjacent_outs = {}
        self.speculates = False
        self.lines = []
        self.group_sites = []
        self.local_arrays = []
        self.private_decls = []
        self.indent = 2 if self.is_kernel else 1
        for s in body:
            self.stmt(s)
        return self.lines

    def translate_device(self, cname):
        body = self.body_stmts()
        self.infer(body)
        lines = self.run_emit(body)
        ret = self.ret_type
        params = []
        for p, t in zip(self.params, self.arg_types):
            ct = t.ctype if isinstance(t, Scalar) else t.ctype()
            params.append(f"{ct} {self.cname(p)}")
        if self.m.boundscheck:
            params.append("int *nmk_oob")
        head = (f"__device__ __forceinline__ {ret.ctype if ret else 'void'} "
                f"{cname}({', '.join(params)}) {{")
        decls = ["  " + d for d in self.declarations() + self.private_decls]
        return "\n".join([head] + decls + lines + ["}"]), ret

    def translate_kernel(self, cname):
        body = self.body_stmts()
        self.infer(body)
        self.adjacent = self.may_be_adjacent()
        if self.adjacent:
            try:
                lines = self.run_emit(body)
                self.check_adjacent_operands()
            except _NotAdjacent:
                self.adjacent = False
        if not self.adjacent:
            lines = self.run_emit(body)
        params, views = [], []
        # (a kernel whose work-items exchange data through memory keeps plain
        # pointers)
        restrict = "__restrict__ " if self.noalias and not (
            self.mode == "kernel" and self.m.communicates) else ""
        for p, t in zip(self.params, self.arg_types):
            c = self.cname(p)
            if isinstance(t, Array):
                params.append(f"{t.elem.ctype} *{restrict}{c}_p")
                params += [f"int64_t {c}_s{k}" for k in range(t.ndim)]
                params += [f"int64_t {c}_t{k}" for k in range(t.ndim)]
                if t.ndim == 0:
                    self.err(self.node, "0-d array arguments are not supported")
                dims = [str(t.const_shape[k]) if t.const_shape[k] is not None
                        else f"{c}_s{k}" for k in range(t.ndim)]
                if t.layout == "C":
                    # dense row-major: the strides follow from the extents
                    strides = ["1"] * t.ndim
                    for k in range(t.ndim - 2, -1, -1):
                        strides[k] = f"{strides[k + 1]} * {dims[k + 1]}"
                else:
                    strides = [f"{c}_t{k}" for k in range(t.ndim)]
                views.append(f"{t.ctype()} {c} = {{{c}_p, {{{', '.join(dims)}}}, "
                             f"{{{', '.join(strides)}}}}};")
            elif isinstance(t, SliceArg):
                params += [f"int64_t {c}_start", f"int64_t {c}_stop", f"int64_t {c}_step"]
            else:
                if p in self.assigned:
                    params.append(f"{t.ctype} {c}_arg")
                    views.append(f"{self.env[p].ctype} {c} = {c}_arg;")
                else:
                    params.append(f"{t.ctype} {c}")
        if self.mode == "elementwise" and self.ret_type is not None:
            # the array an elementwise function returns: allocated by the
            # caller, passed after the function's own arguments
            n = self.ndim
            params.append(f"{self.ret_type.ctype} *{restrict}nmk_ret_p")
            params += [f"int64_t nmk_ret_s{k}" for k in range(n)]
            params += [f"int64_t nmk_ret_t{k}" for k in range(n)]
            # (allocated dense by the caller: the strides follow from the
            # extents, which lets adjacent stores of a lane merge)
            dense = ["1"] * n
            for k in range(n - 2, -1, -1):
                dense[k] = f"{dense[k + 1]} * nmk_ret_s{k + 1}"
            views.append(f"nmkjit::View<{self.ret_type.ctype}, {n}> nmk_ret = {{nmk_ret_p, "
                         f"{{{', '.join(f'nmk_ret_s{k}' for k in range(n))}}}, "
                         f"{{{', '.join(dense)}}}}};")
        # one partial result per block and reduction variable, after the
        # function's own arguments (the host folds them in block order)
        red = []
        for name in sorted(self.reductions):
            t = self.env.get(name)
            if not isinstance(t, Scalar):
                self.err(self.node, f"The reduction variable '{name}' has no scalar type")
            t = INT64 if t.is_bool else t
            neutral = "0" if self.reductions[name] == "add" else "1"
            red.append((name, t, neutral))
            params.append(f"{t.ctype} *nmk_part_{name}")
        if red:
            # (zeroed counters, one set per launch plan: which block finishes)
            params.append("uint32_t *nmk_ticket")
        self.reduction_types = [(n, t) for n, t, _ in red]
        params += [f"uint64_t nmk_lds{k}" for k in range(len(self.local_arrays))]
        params += ["int64_t nmk_gsz0", "int64_t nmk_gsz1", "int64_t nmk_gsz2"]
        if self.m.boundscheck:
            params.append("int *nmk_oob")
        # (the launcher picks the block of a fused map: never above 256 lanes,
        # and a tighter bound wins)
        bound = 256 if self.adjacent else 1024
        out = [f'extern "C" __global__ __launch_bounds__({bound}) void {cname}(',
               "    " + ", ".join(params) + ") {"]
        # Work-items that cannot tell how they are grouped may be laid out on
        # the lanes in any order: put the LAST global dimension on x, so that
        # adjacent lanes touch adjacent elements of row-major arrays.
        self.reversed = (self.allow_remap and not self.m.communicates and self.ndim > 1)
        hw = "xyz"
        dim = [hw[self.ndim - 1 - k] if (self.reversed and k < self.ndim) else hw[k]
               for k in range(3)]
        # Stores nobody reads back go past the caches only along the grid
        # dimension that lies on x (adjacent lanes), and only into unit-stride
        # rows: scattered stores are left for L2 to combine.
        out = [f"#define NMK_STORE_ALONG{k}(p, v, unit) " +
               ("nmkjit::streamStore(p, v, unit)" if dim[k] == "x" else "(*(p) = (v))")
               for k in range(3)] + out
        # A 1-d map whose work-items cannot observe their grouping may give
        # several elements to a lane, a block apart (coalesced); unrolled, with
        # non-overlapping arrays, their loads are in flight together.
        ept = self.elements_per_thread
        if self.m.communicates or self.ndim != 1 or self.mode == "kernel":
            ept = self.elements_per_thread = 1
        # A remapped grid of two or three dimensions runs flat blocks (x only)
        # and gives each lane ROWS_PER_LANE work-items along hardware y: what
        # they load by the x index alone (a row vector against a matrix, the
        # second operand of an outer product) is then loaded once, and the
        # index on y is uniform over the wave.
        rows = ROWS_PER_LANE if self.reversed else 1
        self.rows_per_lane = rows
        flat = self.reversed
        # Where the extent along x is shorter than a wave (a tall result of a
        # few columns), a flat block would leave most lanes of its wave idle:
        # the block then has lanes along hardware y too -- a wave covers whole
        # neighbouring rows -- and a lane's work-items lie a block's rows apart.
        tall = self.lanes_along_y = bool(self.reversed and self.lanes_along_y)
        thin = lambda k: flat and dim[k] != "x" and not (tall and dim[k] == "y")
        out += [
            "  const int64_t " + ", ".join(
                f"nmk_lid{k} = " + ("0" if thin(k) else f"threadIdx.{dim[k]}")
                for k in range(3)) + ";",
            # (a launch has 65535 blocks along y and z: a grid of one or two
            # dimensions with more along y goes on along z)
            "  const int64_t " + ", ".join(
                f"nmk_grp{k} = " + (
                    f"blockIdx.{dim[k]}" if self.ndim == 3 or dim[k] == "x" else
                    "int64_t(blockIdx.y) + int64_t(gridDim.y) * blockIdx.z" if dim[k] == "y"
                    else "0") for k in range(3)) + ";",
            "  const int64_t " + ", ".join(
                f"nmk_lsz{k} = " + ("1" if thin(k) else f"blockDim.{dim[k]}")
                for k in range(3)) + ";",
            "  (void)nmk_lid0; (void)nmk_lid1; (void)nmk_lid2; (void)nmk_grp0; (void)nmk_grp1;",
            "  (void)nmk_grp2; (void)nmk_lsz0; (void)nmk_lsz1; (void)nmk_lsz2;",
        ]
        for name, t, neutral in red:
            out.append(f"  {t.ctype} {self.cname(name)} = ({t.ctype}){neutral};")
        # tables in workgroup memory, staged by the routines' users
        text = "\n".join(self.m.device_code + lines)
        self.stages_table = False
        if "nmkjit::erfF64(" in text:
            out.append("  nmkjit::erfTableLoad();")
            self.stages_table = True
        if "nmkjit::cdfTermF64(" in text or "nmkjit::cdfTermF64m<" in text:
            out.append("  nmkjit::cdfTableLoad();")
            self.stages_table = True
        body = ["    " + v for v in views]
        body += ["    " + d for d in self.declarations() + self.private_decls]
        body += lines
        if rows > 1:
            ky = dim.index("y")
            others = [k for k in range(3) if k != ky]
            out += [f"  const int64_t nmk_gid{k} = nmk_grp{k} * nmk_lsz{k} + nmk_lid{k};"
                    for k in others]
            # (flat blocks: a lane's rows are adjacent; with lanes along y they
            # are a block's rows apart, so that each access of a wave covers
            # adjacent rows)
            first = f"nmk_grp{ky} * {rows}"
            last = f"nmk_first + {rows}"
            step = ""
            if tall:
                first = f"nmk_grp{ky} * ({rows} * nmk_lsz{ky}) + nmk_lid{ky}"
                last = f"(nmk_grp{ky} + 1) * ({rows} * nmk_lsz{ky})"
                step = f" * nmk_lsz{ky}"
            out += [
                f"  const int64_t nmk_first = {first};",
                f"  auto nmk_item = [&](const int64_t nmk_gid{ky}, auto nmk_guarded) {{",
                f"    if (decltype(nmk_guarded)::value && !(nmk_gid{ky} < nmk_gsz{ky})) return;",
            ] + body + [
                "  };",
                "  if (" + " && ".join(f"nmk_gid{k} < nmk_gsz{k}" for k in others) + ") {",
                f"    if ({last} <= nmk_gsz{ky}) {{",
                "#pragma unroll",
                f"      for (int nmk_row = 0; nmk_row < {rows}; ++nmk_row)",
                f"        nmk_item(nmk_first + nmk_row{step}, nmkjit::No());",
                "    } else {",
                "#pragma unroll",
                f"      for (int nmk_row = 0; nmk_row < {rows}; ++nmk_row)",
                f"        nmk_item(nmk_first + nmk_row{step}, nmkjit::Yes());",
                "    }",
                "  }",
            ]
        else:
            # 1-d loops and maps stride over the iteration space by whole
            # grids: the launcher may run fewer blocks than cover it (it does
            # for reductions, whose per-block epilogue then runs once per many
            # elements).  A lane takes `ept` elements a block apart (each
            # access of the wave is contiguous on its own); a round that lies
            # wholly inside the iteration space runs them unguarded, so a
            # straight-line body has all its loads in flight together.
            strided = self.ndim == 1 and not self.m.communicates and self.mode != "kernel"
            self.grid_stride = strided
            if strided:
                # (name, element type, address of the element at index g)
                pf = []
                for name in [p for p in self.params if p in self.prefetched and ept > 1]:
                    t, c = self.prefetched[name], self.cname(name)
                    step = "" if t.layout == "C" else f" * {c}_t0"
                    addr = f"&{c}_p[g{step}]"
                    # (a loop's other iterations may read the element too)
                    load = f"__builtin_nontemporal_load({addr})" \
                        if self.stream and self.mode == "elementwise" else f"*({addr})"
                    pf.append((name, t.elem.ctype, load))
                if self.prefetched and not pf:
                    self.err(self.node, "internal: elements loaded ahead in a kernel that "
                                        "takes one element per lane")
                extra = "".join(f", const {ct} nmk_pf_{n}" for n, ct, _ in pf)
                if self.adjacent:
                    out += self.adjacent_rounds(pf, body)
                    strided = False       # (the rounds are written)
                if strided:
                  out += [
                      "  const int64_t nmk_gid1 = 0, nmk_gid2 = 0;",
                      "  (void)nmk_gid1; (void)nmk_gid2;",
                      f"  auto nmk_item = [&](const int64_t nmk_gid0, auto nmk_guarded{extra}) {{",
                      "    if (decltype(nmk_guarded)::value && !(nmk_gid0 < nmk_gsz0)) return;",
                  ] + body + [
                      "  };",
                      f"  for (int64_t nmk_round = nmk_grp0; nmk_round * {ept} * nmk_lsz0 < "
                      "nmk_gsz0; nmk_round += gridDim.x) {",
                      f"    const int64_t nmk_base = nmk_round * {ept} * nmk_lsz0 + nmk_lid0;",
                      f"    if ((nmk_round + 1) * {ept} * nmk_lsz0 <= nmk_gsz0) {{",
                  ]
                  if pf:
                      # The empty asm statements keep the optimizer from moving
                      # each load back down to its first use.
                      out += [f"      {ct} nmk_ahead_{n}[{ept}];" for n, ct, _ in pf]
                      out += [
                          "#pragma unroll",
                          f"      for (int nmk_rep = 0; nmk_rep < {ept}; ++nmk_rep) {{",
                          "        const int64_t g = nmk_base + nmk_rep * nmk_lsz0;",
                      ] + [f"        nmk_ahead_{n}[nmk_rep] = {load};" for n, _, load in pf] + [
                          "      }",
                          "#pragma unroll",
                          f"      for (int nmk_rep = 0; nmk_rep < {ept}; ++nmk_rep) {{",
                      ] + [f'        asm volatile("" : "+v"(nmk_ahead_{n}[nmk_rep]));'
                           for n, _, _ in pf] + [
                          "      }",
                      ]
                  ahead = "".join(f", nmk_ahead_{n}[nmk_rep]" for n, _, _ in pf)
                  out += [
                      "#pragma unroll",
                      f"      for (int nmk_rep = 0; nmk_rep < {ept}; ++nmk_rep)",
                      f"        nmk_item(nmk_base + nmk_rep * nmk_lsz0, nmkjit::No(){ahead});",
                      "    } else {",
                      "#pragma unroll 1",
                      f"      for (int nmk_rep = 0; nmk_rep < {ept}; ++nmk_rep) {{",
                      "        const int64_t g = nmk_base + nmk_rep * nmk_lsz0;",
                      "        if (g < nmk_gsz0)",
                      "          nmk_item(g, nmkjit::No()" +
                      "".join(f", {load}" for _, _, load in pf) + ");",
                      "      }",
                      "    }",
                      "  }",
                  ]
            else:
                out += [
                    "  const int64_t nmk_gid0 = nmk_grp0 * nmk_lsz0 + nmk_lid0;",
                    "  const int64_t nmk_gid1 = nmk_grp1 * nmk_lsz1 + nmk_lid1;",
                    "  const int64_t nmk_gid2 = nmk_grp2 * nmk_lsz2 + nmk_lid2;",
                    "  const bool nmk_active = nmk_gid0 < nmk_gsz0 && nmk_gid1 < nmk_gsz1 && "
                    "nmk_gid2 < nmk_gsz2;",
                ]
                if self.group_sites:
                    out.append("  __shared__ int nmk_clipped;")
                    for slot, t, _ in self.group_sites:
                        out.append(f"  __shared__ {t.ctype} {slot}[nmkjit::kMaxGroup];")
                    out.append("  if (nmkjit::linearLocalId() == 0) nmk_clipped = 0;")
                    out.append("  __syncthreads();")
                    out.append("  if (!nmk_active) nmk_clipped = 1;")
                    for slot, t, neutral in self.group_sites:
                        out.append(f"  nmkjit::groupInit<{t.ctype}>({slot}, "
                                   f"({t.ctype}){neutral});")
                    out.append("  __syncthreads();")
                out.append("  if (nmk_active) {")
                out += body
                out.append("  }")
        for name, t, _ in red:
            op = "AddOp" if self.reductions[name] == "add" else "MulOp"
            out.append(f"  nmkjit::blockReduceStore<{t.ctype}>({self.cname(name)}, "
                       f"nmkjit::{op}(), nmk_part_{name});")
        if red:
            # the block that arrives last adds up the blocks' results: each
            # array of partial results has one more element, for the total
            out.append("  if (nmkjit::drewLastTicket(nmk_ticket)) {")
            for name, t, neutral in red:
                op = "AddOp" if self.reductions[name] == "add" else "MulOp"
                out.append(f"    nmkjit::foldPartials<{t.ctype}>(nmk_part_{name}, nmkjit::{op}(), "
                           f"({t.ctype}){neutral});")
            out.append("  }")
        out.append("}")
        return "\n".join(out)


ROWS_PER_LANE = 4     # work-items per lane along hardware y of a remapped grid


def _safe(name):
    return "".join(ch if ch.isalnum() else "_" for ch in name)


HEADER = """// Generated from the Python @kernel '{name}'; do not edit.
#include "jit_support.h"
extern __shared__ __attribute__((aligned(16))) unsigned char nmk_dyn_lds[];
"""


class CompiledKernel:
    def __init__(self, name, source, local_arrays):
        self.name, self.source = name, source
        # bytes of each work-group-memory parameter, in parameter order
        self.local_bytes = [int(np.prod(shape, dtype=np.int64)) * elem.dtype.itemsize
                            for elem, shape in local_arrays]


def translate(func, arg_types, ndim, stubs, boundscheck=False, remap=False,
              mode="kernel", noalias=False, elements_per_thread=1, stream=True):
    """Python function + argument types -> CompiledKernel (source only).

    With ``boundscheck`` every index is tested against its dimension: an
    index outside it is replaced by 0 and the flag the kernel's last
    parameter points at is set, so the launch can raise IndexError instead
    of faulting the GPU.  With ``remap`` a body whose work-items cannot
    observe their grouping gets global dimension ``ndim - 1`` on x
    (``reversed_dims`` of the result tells the launcher); ``remap="tall"``
    says that this dimension is shorter than a wave, and the blocks get lanes
    along the next dimension too (``lanes_along_y``).

    ``mode``: "kernel" for an @kernel body; "elementwise" for a function of
    whole arrays fused into one map over ``ndim`` dimensions (``ret_dtype`` of
    the result is the dtype of the returned array, if any); "parallel" for a
    function whose top-level prange loop becomes a 1-d grid (``range_source``
    holds the source text of the prange arguments for the host to evaluate).
    ``noalias`` promises that no two array arguments overlap (pointers become
    ``__restrict__``); with ``stream`` as well -- the caller found the arrays
    too large to stay in the memory-side cache between launches -- arrays the
    body only stores into are written past the caches and a fused map reads
    its operands with streaming loads.  For the last two modes ``elements_per_thread`` asks for that
    many elements per lane of a 1-d grid (the result says what it got: the launcher divides the grid
    by it)."""
    module = Module(stubs, boundscheck)
    tr = FunctionTranslator(module, func, arg_types, True, ndim)
    tr.allow_remap = bool(remap)
    tr.lanes_along_y = remap == "tall"
    tr.mode = mode
    tr.noalias = noalias
    tr.stream = stream
    if mode != "kernel":
        tr.elements_per_thread = max(1, int(elements_per_thread))
    if mode == "parallel":
        _check_parallel_shape(tr)
    digest = hashlib.sha256()
    body = tr.translate_kernel("NMK_KERNEL_NAME")
    text = "\n\n".join(module.device_code + [body])
    digest.update(text.encode())
    name = f"nmkjit_{_safe(func.__name__)}_{digest.hexdigest()[:12]}"
    source = HEADER.format(name=func.__name__) + "\n" + text.replace("NMK_KERNEL_NAME", name) + "\n"
    compiled = CompiledKernel(name, source, tr.local_arrays)
    compiled.boundscheck = boundscheck
    # translated for arguments that do not overlap (__restrict__ pointers,
    # streaming stores, loads ahead of the body): launches must keep to that
    compiled.noalias = bool(noalias)
    compiled.reversed_dims = tr.reversed
    # a remapped kernel runs blocks of shape (n, 1, 1) and gives each lane this
    # many work-items along hardware y: the launcher divides that grid
    # dimension by it
    compiled.rows_per_lane = tr.rows_per_lane
    # ... unless the grid is short along x: then the block has lanes along
    # hardware y as well (x extent times as many as fill 256)
    compiled.lanes_along_y = tr.lanes_along_y
    # a 1-d loop or map that strides over its iteration space by whole grids:
    # any number of blocks computes the same thing
    compiled.grid_stride = tr.grid_stride
    # every block first copies a table into workgroup memory: worth two trips
    # a lane instead of one
    compiled.stages_table = tr.stages_table
    compiled.ret_dtype = tr.ret_type.dtype if (mode == "elementwise" and tr.ret_type) else None
    compiled.range_source = tr.range_source[1] if tr.range_source else None
    compiled.grid_sources = list(tr.grid_sources)   # per grid dimension
    compiled.written = sorted(tr.written_arrays)
    compiled.elements_per_thread = tr.elements_per_thread
    # parallel mode: (name, dtype, "add" | "mul") per reduction, in the order
    # of their partial-result parameters, and the source of the final return
    compiled.reductions = [(n, t.dtype, tr.reductions[n]) for n, t in tr.reduction_types]
    compiled.return_source = (ast.unparse(tr.return_node.value)
                              if tr.return_node is not None else None)
    # parallel mode: what precedes the loop, for the host to evaluate the
    # loop bounds that depend on it (n = len(x); for i in prange(n))
    compiled.preamble_source = []
    if tr.range_source:
        for stmt in tr.body_stmts():
            if stmt is tr.range_source[0]:
                break
            compiled.preamble_source.append(ast.unparse(stmt))
    if mode == "parallel" and compiled.range_source is None:
        raise KernelCompileError(f"{func.__name__}: no top-level prange loop to offload")
    return compiled


def _check_parallel_shape(tr):
    """A parallel function is: assignments, one prange loop, then at most a
    ``return``.  Scalars that the loop only updates with ``+=`` / ``*=`` and
    that are set before it are reductions: every lane accumulates its share,
    blocks reduce theirs, the host folds the per-block partials and evaluates
    the ``return`` expression."""
    body = tr.body_stmts()
    loop = None
    before = set()
    for stmt in body:
        if isinstance(stmt, ast.For):
            if loop is not None:
                tr.err(stmt, "Only one top-level loop is offloaded")
            loop = stmt
        elif loop is not None:
            if isinstance(stmt, ast.Return) and tr.return_node is None:
                tr.return_node = stmt if stmt.value is not None else None
            elif not isinstance(stmt, ast.Pass):
                tr.err(stmt, "Statements after the parallel loop are not supported")
        elif isinstance(stmt, ast.Assign):
            before |= {t.id for t in stmt.targets if isinstance(t, ast.Name)}
        elif not isinstance(stmt, (ast.AugAssign, ast.Expr, ast.Pass)):
            tr.err(stmt, "Only assignments may precede the parallel loop")
    if loop is None:
        return
    ops = {ast.Add: "add", ast.Mult: "mul"}
    for node in ast.walk(loop):
        if isinstance(node, ast.AugAssign) and isinstance(node.target, ast.Name) and \
                node.target.id in before:
            name = node.target.id
            if type(node.op) not in ops or tr.reductions.get(name, ops[type(node.op)]) != \
                    ops[type(node.op)]:
                tr.err(node, f"'{name}' is set before the parallel loop and updated in it: "
                             "only '+=' or only '*=' make it a reduction")
            tr.reductions[name] = ops[type(node.op)]
    for node in ast.walk(loop):
        if isinstance(node, ast.Name) and node.id in tr.reductions and \
                isinstance(node.ctx, ast.Load):
            tr.err(node, f"The reduction variable '{node.id}' cannot be read inside the loop")
        if isinstance(node, ast.Assign) and any(isinstance(t, ast.Name) and
                                                t.id in tr.reductions for t in node.targets):
            tr.err(node, "A reduction variable can only be updated with '+=' or '*='")
    if tr.return_node is not None:
        for node in ast.walk(tr.return_node.value):
            if isinstance(node, ast.Name) and node.id in tr.assigned and \
                    node.id not in tr.reductions and node.id not in before:
                tr.err(node, f"'{node.id}' is computed inside the loop; only reductions and "
                             "what precedes the loop can be returned")


# ---------------------------------------------------------------------------
# Source -> code object
# ---------------------------------------------------------------------------

_HERE = os.path.dirname(os.path.abspath(__file__))
_KERNELS_DIR = os.path.join(os.path.dirname(_HERE), "csrc", "kernels")
CACHE_DIR = os.environ.get(
    "NUMBA_MLIR_KERNEL_CACHE", os.path.join(os.path.dirname(_HERE), "kernel_cache"))


def _hipcc():
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    return os.environ.get("HIPCC", os.path.join(rocm, "bin", "hipcc"))


_FLAGS = ["--genco", "--no-gpu-bundle-output", "--offload-arch=gfx950", "-O3",
          "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang",
          "-packed-fp32-ops", "-std=c++17"]


def build_code_object(compiled):
    """Compiles the generated source with hipcc; code objects are cached on
    disk under the hash of (source, support header, flags)."""
    support = b""
    for header in ("jit_support.h", "fast_math.h", "erf_taylor.inc", "erf_table.inc"):
        with open(os.path.join(_KERNELS_DIR, header), "rb") as f:
            support += f.read()
    digest = hashlib.sha256()
    flags = list(_FLAGS)
    if getattr(compiled, "fastmath", False):
        # fastmath=True (reference: test_gpu.py:980-1008 expects a * b + c to
        # become one fma): contraction only, no value-changing shortcuts
        flags[flags.index("-ffp-contract=off")] = "-ffp-contract=fast"
    for part in (compiled.source.encode(), support, " ".join(flags).encode()):
        digest.update(part)
    key = digest.hexdigest()[:24]
    os.makedirs(CACHE_DIR, exist_ok=True)
    obj = os.path.join(CACHE_DIR, f"{compiled.name}_{key}.hsaco")
    if not os.path.exists(obj):
        src = os.path.join(CACHE_DIR, f"{compiled.name}_{key}.hip")
        with open(src, "w") as f:
            f.write(compiled.source)
        tmp = obj + f".tmp{os.getpid()}"
        proc = subprocess.run([_hipcc(), *flags, f"-I{_KERNELS_DIR}", "-o", tmp, src],
                              capture_output=True, text=True)
        if proc.returncode != 0:
            raise KernelCompileError(
                f"hipcc failed for {compiled.name}:\n{proc.stderr}\n--- source ---\n"
                f"{compiled.source}")
        os.replace(tmp, obj)
    with open(obj, "rb") as f:
        return f.read()
