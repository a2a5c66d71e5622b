"""Splits a straight-line function of whole-array expressions at its
reductions and contractions.

The reference lowers ``np.sqrt(np.sum(a * b, axis=1)) / n`` to a chain of
linalg.generic ops -- a map, a reduction, a map -- and fuses what it can
(numba_mlir/mlir/numpy/funcs.py:163-229 builds the reductions,
linalg_builder.py:297-325 the maps).  Here the same chain is made explicit:
every ``np.sum / prod / min / max / mean`` (function or array method),
``np.dot`` and ``@`` becomes a *library* stage served by a hand-written
kernel, and the expressions between them become *map* stages, each fused into
one generated kernel.  Operands of a library stage that are expressions are
materialised by a map stage first.

Only straight-line bodies qualify: assignments to names, whole-array stores
(``out[:] = ...``), augmented assignments of names and one final ``return``.
"""

import ast

REDUCTIONS = ("sum", "prod", "min", "max", "amin", "amax", "mean")
CONTRACTIONS = ("dot",)
VIEWS = ("reshape", "transpose", "ravel", "flip",     # no data moves
         "copy", "flatten", "astype",                 # a dense copy
         "asfortranarray")
# what an array says about itself: host values (numpy/funcs.py:1197-1300)
ARRAY_FACTS = ("shape", "size", "ndim", "itemsize", "strides", "dtype")
# np.<name>(...) that builds a new array on the device: which positional
# arguments are arrays ("tuple": the first is a tuple of them)
MAKERS = {"arange": (), "eye": (), "tril": (0,), "triu": (0,), "outer": (0, 1),
          "cov": (0, 1), "concatenate": "tuple", "hstack": "tuple", "vstack": "tuple", "dstack": "tuple"}
ALLOCATIONS = ("empty", "zeros", "ones", "empty_like", "zeros_like", "ones_like")
# NumPy functions that take an `out` array after this many operands
# (reference: numpy/funcs.py registers them with out="out")
OUT_AFTER = dict(
    [(n, 1) for n in ("sqrt", "square", "log", "sin", "cos", "exp", "tanh", "abs",
                      "absolute", "negative", "positive", "logical_not", "invert")] +
    [(n, 2) for n in ("add", "subtract", "multiply", "true_divide", "divide", "power",
                      "arctan2", "minimum", "maximum", "logical_and", "logical_or",
                      "logical_xor", "less", "greater", "less_equal", "greater_equal",
                      "equal", "not_equal", "bitwise_and", "bitwise_or", "bitwise_xor",
                      "left_shift", "right_shift", "floor_divide", "remainder", "mod")] +
    [("clip", 3)])


class Stage:
    """kind: "map" (target = expr), "store" (target[...] = expr), "lib"
    (target = op(operands, **kwargs)), "alloc" (target = a new array; ``args``
    are the call's positional and keyword expressions, of host values), "view"
    (target = operand reshaped or
    transposed; ``args`` are expressions of host values), "call" (target =
    another compiled function applied to whole arrays; ``args`` are names),
    "return" (expr is a Name or an expression of names)."""

    def __init__(self, kind, target=None, expr=None, op=None, operands=(), kwargs=None,
                 node=None):
        self.kind, self.target, self.expr = kind, target, expr
        self.op, self.operands, self.kwargs = op, list(operands), kwargs or {}
        self.node = node            # the source node, for messages
        self.inputs = []            # local names the expression reads (map / store)
        self.args = []              # view / call stages: see above
        self.deferred = False       # a map that the next stage evaluates itself
        self.fused_map = None       # ... and that stage's link to it

    def __repr__(self):
        if self.kind == "lib":
            return f"{self.target} = {self.op}({', '.join(self.operands)}, {self.kwargs})"
        text = ast.unparse(self.expr) if self.expr is not None else ""
        return " ".join(part for part in (self.kind, self.target, text) if part)


class NotStraightLine(Exception):
    pass


def _is_whole_slice(node):
    def full(n):
        return (isinstance(n, ast.Slice) and n.lower is None and n.upper is None
                and n.step is None) or \
               (isinstance(n, ast.Constant) and n.value is Ellipsis)
    if isinstance(node, ast.Tuple):
        return len(node.elts) > 0 and all(full(e) for e in node.elts)
    return full(node)


class _Splitter(ast.NodeTransformer):
    def __init__(self, plan):
        self.plan = plan

    def _operand(self, node):
        """A name holding the operand's value (materialised if needed)."""
        if isinstance(node, ast.Name):
            return node.id
        name = self.plan.fresh()
        self.plan.add(Stage("map", name, node, node=node))
        return name

    def _literal_kwargs(self, node, positional, keywords):
        kwargs = {}
        for key, value in list(zip(("axis",), positional)) + \
                [(k.arg, k.value) for k in keywords]:
            if key != "axis":
                raise NotStraightLine(f"line {node.lineno}: only 'axis' is supported here")
            try:
                kwargs[key] = ast.literal_eval(value)
            except ValueError:
                raise NotStraightLine(f"line {node.lineno}: the axis must be a literal")
            if not (kwargs[key] is None or isinstance(kwargs[key], int)):
                raise NotStraightLine(f"line {node.lineno}: the axis must be one integer")
        return kwargs

    def visit_Call(self, node):
        self.generic_visit(node)              # innermost stages first
        func = node.func
        if isinstance(func, ast.Name) and func.id == "len" and "len" not in self.plan.locals \
                and len(node.args) == 1 and not node.keywords and \
                isinstance(node.args[0], ast.Name) and node.args[0].id in self.plan.locals:
            return self._fact(node, "len", node.args[0].id)
        if not isinstance(func, ast.Attribute):
            return node
        name = func.attr
        if name in VIEWS:
            return self._view(node, name)
        numpy_function = isinstance(func.value, ast.Name) and \
            func.value.id not in self.plan.locals and self.plan.is_numpy(func.value.id)
        if numpy_function and name in ALLOCATIONS:
            stage = Stage("alloc", self.plan.fresh(), op=name, node=node)
            stage.args = (list(node.args), list(node.keywords))
            self.plan.add(stage)
            self.plan.library_stages += 1
            return ast.copy_location(ast.Name(id=stage.target, ctx=ast.Load()), node)
        if numpy_function and name in MAKERS:
            return self._make(node, name)
        if numpy_function and name in OUT_AFTER:
            return self._with_out(node, OUT_AFTER[name])
        if name not in REDUCTIONS + CONTRACTIONS:
            return node
        base = func.value
        if isinstance(base, ast.Name) and base.id not in self.plan.locals:
            if not self.plan.is_numpy(base.id):
                return node                   # math.prod, some other module
            args = list(node.args)            # np.<name>(x, ...)
        else:
            args = [base] + list(node.args)   # <expr>.<name>(...)
        count = 2 if name in CONTRACTIONS else 1
        if len(args) < count:
            return node
        operands = [self._operand(a) for a in args[:count]]
        if name in CONTRACTIONS:
            # np.dot(a, b, c) / np.dot(a, b, out=c) write into an existing array
            extra = list(args[count:]) + [k.value for k in node.keywords if k.arg == "out"]
            if len(extra) > 1 or any(k.arg != "out" for k in node.keywords) or \
                    not all(isinstance(e, ast.Name) for e in extra):
                raise NotStraightLine(f"line {node.lineno}: np.dot takes two arrays and "
                                      "an optional out array here")
            kwargs = {"out": extra[0].id} if extra else {}
        else:
            kwargs = self._literal_kwargs(node, args[count:], node.keywords)
        target = self.plan.fresh()
        self.plan.add(Stage("lib", target, op=name, operands=operands, kwargs=kwargs,
                            node=node))
        self.plan.library_stages += 1
        return ast.copy_location(ast.Name(id=target, ctx=ast.Load()), node)

    def _make(self, node, name):
        """np.arange / eye / tril / triu / outer / cov / concatenate / hstack /
        vstack (reference: numpy/funcs.py:255-310, 642-700, 1536-1549): the
        array arguments become operands, the others stay host expressions."""
        where = MAKERS[name]
        args = list(node.args)
        operands, slots = [], []          # slots: per positional, operand index or None
        if where == "tuple":
            if not args or not isinstance(args[0], (ast.Tuple, ast.List)):
                raise NotStraightLine(f"line {node.lineno}: np.{name} takes a tuple of "
                                      "arrays here")
            operands = [self._operand(e) for e in args[0].elts]
            args = args[1:]
        else:
            for at, arg in enumerate(args):
                is_none = isinstance(arg, ast.Constant) and arg.value is None
                if at in where and not is_none:
                    slots.append(len(operands))
                    operands.append(self._operand(arg))
                else:
                    slots.append(None)
        keywords = []
        for k in node.keywords:
            if name == "cov" and k.arg == "y" and \
                    not (isinstance(k.value, ast.Constant) and k.value.value is None):
                keywords.append(("y", len(operands)))
                operands.append(self._operand(k.value))
            else:
                keywords.append((k.arg, k.value))
        stage = Stage("make", self.plan.fresh(), op=name, operands=operands, node=node)
        stage.args = (args, slots, keywords)
        self.plan.add(stage)
        self.plan.library_stages += 1
        return ast.copy_location(ast.Name(id=stage.target, ctx=ast.Load()), node)

    def visit_Subscript(self, node):
        """x[a:b], x[:, j], x[::2], x[i] of a local array: a view (of one
        element when every axis is indexed)."""
        self.generic_visit(node)
        if not isinstance(node.ctx, ast.Load) or not isinstance(node.value, ast.Name) or \
                node.value.id not in self.plan.locals or _is_whole_slice(node.slice):
            return node
        stage = Stage("view", self.plan.fresh(), op="getitem", operands=[node.value.id],
                      node=node)
        stage.args = [node.slice]
        self.plan.add(stage)
        self.plan.library_stages += 1
        return ast.copy_location(ast.Name(id=stage.target, ctx=ast.Load()), node)

    def _with_out(self, node, operands):
        """np.add(a, b, out) / np.add(a, b, out=out): a store into ``out``,
        whose value the call then is."""
        out = [k.value for k in node.keywords if k.arg == "out"]
        if len(node.args) == operands + 1 and not out:
            out, args = [node.args[-1]], node.args[:-1]
        else:
            args = node.args
        if not out or (isinstance(out[0], ast.Constant) and out[0].value is None):
            return node
        if not isinstance(out[0], ast.Name) or len(args) != operands or \
                any(k.arg != "out" for k in node.keywords):
            raise NotStraightLine(f"line {node.lineno}: out must be a named array")
        value = ast.copy_location(ast.Call(func=node.func, args=list(args), keywords=[]), node)
        self.plan.add(Stage("store", out[0].id, value, node=node))
        self.plan.library_stages += 1
        return ast.copy_location(ast.Name(id=out[0].id, ctx=ast.Load()), node)

    def _view(self, node, name):
        base = node.func.value
        if isinstance(base, ast.Name) and base.id not in self.plan.locals:
            if not self.plan.is_numpy(base.id) or not node.args:
                return node
            array, args = node.args[0], list(node.args[1:])    # np.reshape(x, shape)
        else:
            array, args = base, list(node.args)                # x.reshape(...)
        if node.keywords:
            raise NotStraightLine(f"line {node.lineno}: keywords are not supported here")
        stage = Stage("view", self.plan.fresh(), op=name, operands=[self._operand(array)],
                      node=node)
        stage.args = args
        self.plan.add(stage)
        self.plan.library_stages += 1
        return ast.copy_location(ast.Name(id=stage.target, ctx=ast.Load()), node)

    def _fact(self, node, name, operand):
        """x.shape, len(x), ...: a host value taken from the array as it is at
        that point (inside a fused map the array is seen per element, through
        a view with its dimensions merged)."""
        stage = Stage("view", self.plan.fresh(), op=name, operands=[operand], node=node)
        self.plan.add(stage)
        self.plan.library_stages += 1
        return ast.copy_location(ast.Name(id=stage.target, ctx=ast.Load()), node)

    def visit_Attribute(self, node):
        self.generic_visit(node)
        if node.attr in ARRAY_FACTS and isinstance(node.ctx, ast.Load) and \
                isinstance(node.value, ast.Name) and node.value.id in self.plan.locals:
            return self._fact(node, node.attr, node.value.id)
        if node.attr != "T" or not isinstance(node.ctx, ast.Load):
            return node
        if isinstance(node.value, ast.Name) and node.value.id not in self.plan.locals:
            return node
        stage = Stage("view", self.plan.fresh(), op="transpose",
                      operands=[self._operand(node.value)], node=node)
        self.plan.add(stage)
        self.plan.library_stages += 1
        return ast.copy_location(ast.Name(id=stage.target, ctx=ast.Load()), node)

    def visit_BinOp(self, node):
        self.generic_visit(node)
        if not isinstance(node.op, ast.MatMult):
            return node
        operands = [self._operand(node.left), self._operand(node.right)]
        target = self.plan.fresh()
        self.plan.add(Stage("lib", target, op="dot", operands=operands, node=node))
        self.plan.library_stages += 1
        return ast.copy_location(ast.Name(id=target, ctx=ast.Load()), node)


class Plan:
    """The stages of one function, in execution order."""

    def __init__(self, node, is_numpy, is_compiled=lambda name: False):
        self.is_numpy = is_numpy            # name -> bool: bound to the numpy module
        self.is_compiled = is_compiled      # name -> bool: another compiled function
        self.stages = []
        self.library_stages = 0
        self.counter = 0
        self.params = [a.arg for a in node.args.args]
        self.locals = set(self.params)
        body = node.body if isinstance(node.body, list) else [ast.Return(value=node.body)]
        for stmt in body:
            for n in ast.walk(stmt):
                if isinstance(n, ast.Name) and isinstance(n.ctx, ast.Store):
                    self.locals.add(n.id)
        splitter = _Splitter(self)
        returned = False
        for stmt in body:
            if returned:
                raise NotStraightLine("statements after the return")
            if isinstance(stmt, ast.Expr) and isinstance(stmt.value, ast.Constant):
                continue                                       # a docstring
            if isinstance(stmt, ast.AugAssign) and isinstance(stmt.target, ast.Subscript) and \
                    isinstance(stmt.target.value, ast.Name) and \
                    not _is_whole_slice(stmt.target.slice):
                # x[1:] += ...: x[1:] = x[1:] + ...
                import copy
                load = copy.deepcopy(stmt.target)
                load.ctx = ast.Load()
                value = ast.copy_location(ast.BinOp(left=load, op=stmt.op, right=stmt.value),
                                          stmt)
                stmt = ast.copy_location(ast.Assign(targets=[stmt.target], value=value), stmt)
            if isinstance(stmt, ast.AugAssign) and isinstance(stmt.target, ast.Name):
                load = ast.copy_location(ast.Name(id=stmt.target.id, ctx=ast.Load()), stmt)
                value = ast.copy_location(ast.BinOp(left=load, op=stmt.op, right=stmt.value),
                                          stmt)
                stmt = ast.copy_location(ast.Assign(targets=[stmt.target], value=value), stmt)
            call = stmt.value if isinstance(stmt, (ast.Expr, ast.Assign)) else None
            if isinstance(call, ast.Call) and isinstance(call.func, ast.Name) and \
                    call.func.id not in self.locals and self.is_compiled(call.func.id) and \
                    not call.keywords and \
                    (isinstance(stmt, ast.Expr) or
                     (len(stmt.targets) == 1 and isinstance(stmt.targets[0], ast.Name))):
                # another compiled function applied to whole arrays
                target = stmt.targets[0].id if isinstance(stmt, ast.Assign) else None
                stage = Stage("call", target, op=call.func.id, node=stmt)
                stage.args = [splitter._operand(splitter.visit(a)) for a in call.args]
                self.add(stage)
                self.library_stages += 1
                continue
            if isinstance(stmt, ast.Expr):
                # a call made for its effect: np.add(a, b, out)
                if isinstance(splitter.visit(stmt.value), ast.Name):
                    continue
                raise NotStraightLine(f"line {stmt.lineno}: an expression without effect")
            if isinstance(stmt, ast.Assign) and len(stmt.targets) == 1:
                target = stmt.targets[0]
                value = splitter.visit(stmt.value)
                if isinstance(target, ast.Name):
                    self.add(Stage("map", target.id, value, node=stmt))
                    continue
                if isinstance(target, ast.Subscript) and isinstance(target.value, ast.Name) \
                        and _is_whole_slice(target.slice):
                    self.add(Stage("store", target.value.id, value, node=stmt))
                    continue
                if isinstance(target, ast.Subscript) and isinstance(target.value, ast.Name) \
                        and target.value.id in self.locals:
                    # x[1:5] = ..., x[:, 3] = ..., x[5] = ...: a store into a view of x
                    view = Stage("view", self.fresh(), op="getitem",
                                 operands=[target.value.id], node=stmt)
                    view.args = [splitter.visit(target.slice)]
                    self.add(view)
                    self.library_stages += 1
                    self.add(Stage("store", view.target, value, node=stmt))
                    continue
            elif isinstance(stmt, ast.Return):
                if stmt.value is not None:
                    self.add(Stage("return", None, splitter.visit(stmt.value), node=stmt))
                returned = True
                continue
            raise NotStraightLine(f"line {stmt.lineno}: not an assignment, a whole-array "
                                  "store or a return")
        for stage in self.stages:
            if stage.expr is not None:
                seen = []
                for n in ast.walk(stage.expr):
                    if isinstance(n, ast.Name) and n.id in self.locals and n.id not in seen:
                        seen.append(n.id)
                stage.inputs = seen
        self._mark_fused_reductions()

    def _mark_fused_reductions(self):
        """np.sum / np.mean -- over everything, or along an axis of a matrix --
        of an expression materialised just for it: the map can run inside the
        reduction (one pass over the operands instead of a pass, a temporary
        and a second pass).  The map
        stage is marked ``deferred`` and the library stage gets it as
        ``fused_map``; the executor falls back to the two stages when the
        operands do not all have one dense shape."""
        uses = {}
        for stage in self.stages:
            for name in list(stage.inputs) + list(stage.operands) + \
                    [a for a in stage.args if isinstance(a, str)] + \
                    ([stage.kwargs["out"]] if "out" in stage.kwargs else []):
                uses[name] = uses.get(name, 0) + 1
            if stage.kind in ("view", "alloc", "make"):
                # their argument expressions may name anything
                if stage.kind == "alloc":
                    nodes = stage.args[0] + [k.value for k in stage.args[1]]
                elif stage.kind == "make":
                    nodes = [a for a, slot in zip(stage.args[0], stage.args[1] or
                                                  [None] * len(stage.args[0])) if slot is None] + \
                        [v for _, v in stage.args[2] if isinstance(v, ast.AST)]
                else:
                    nodes = stage.args
                for node in nodes:
                    for n in ast.walk(node):
                        if isinstance(n, ast.Name):
                            uses[n.id] = uses.get(n.id, 0) + 2
        for before, stage in zip(self.stages, self.stages[1:]):
            if stage.kind == "lib" and stage.op in ("sum", "mean") and \
                    stage.kwargs.get("axis") in (None, 0, 1, -1, -2) and \
                    before.kind == "map" and \
                    before.target == stage.operands[0] and \
                    before.target.startswith("_nmk_t") and uses.get(before.target) == 1 and \
                    not isinstance(before.expr, ast.Name):
                before.deferred = True
                stage.fused_map = before

    def fresh(self):
        self.counter += 1
        name = f"_nmk_t{self.counter}"
        self.locals.add(name)
        return name

    def add(self, stage):
        self.stages.append(stage)


def plan_of(node, is_numpy, is_compiled=lambda name: False):
    """The Plan of a FunctionDef / Lambda node, or None when the body is not
    straight-line or holds nothing to split at (a reduction, a contraction, a
    view, a call of another compiled function)."""
    try:
        import copy
        plan = Plan(copy.deepcopy(node), is_numpy, is_compiled)
    except NotStraightLine:
        return None
    return plan if plan.library_stages else None


def stage_function(stage, name, scope):
    """A Python function computing one map or store stage (its source is
    attached as ``__nmk_ast__`` for the kernel compiler)."""
    args = ast.arguments(posonlyargs=[], args=[], kwonlyargs=[], kw_defaults=[], defaults=[])
    params = list(stage.inputs)
    if stage.kind == "store":
        params = [stage.target] + [p for p in params if p != stage.target]
        body = ast.Assign(
            targets=[ast.Subscript(value=ast.Name(id=stage.target, ctx=ast.Load()),
                                   slice=ast.Constant(value=Ellipsis), ctx=ast.Store())],
            value=stage.expr)
    else:
        body = ast.Return(value=stage.expr)
    args.args = [ast.arg(arg=p) for p in params]
    fn = ast.FunctionDef(name=name, args=args, body=[body], decorator_list=[])
    ast.copy_location(fn, stage.node)
    ast.copy_location(body, stage.node)
    module = ast.fix_missing_locations(ast.Module(body=[fn], type_ignores=[]))
    namespace = dict(scope)
    exec(compile(module, f"<stage of {name}>", "exec"), namespace)    # noqa: S102
    func = namespace[name]
    func.__nmk_ast__ = fn
    return func, params


def reduction_function(stage, name, scope, arrays, integer):
    """A Python function summing one map stage's expression over dense 1-d
    operands in a parallel loop: ``arrays`` are the inputs that are arrays
    (indexed by the loop variable), the others stay scalars.  ``integer``
    selects an integer accumulator."""
    class Index(ast.NodeTransformer):
        def visit_Name(self, node):
            if node.id in arrays and isinstance(node.ctx, ast.Load):
                return ast.copy_location(ast.Subscript(
                    value=node, slice=ast.Name(id="_nmk_i", ctx=ast.Load()), ctx=ast.Load()),
                    node)
            return node

    import copy
    expr = Index().visit(copy.deepcopy(stage.expr))
    params = ["_nmk_n"] + list(stage.inputs)
    args = ast.arguments(posonlyargs=[], args=[ast.arg(arg=p) for p in params],
                         kwonlyargs=[], kw_defaults=[], defaults=[])
    body = [
        ast.Assign(targets=[ast.Name(id="_nmk_acc", ctx=ast.Store())],
                   value=ast.Constant(value=0 if integer else 0.0)),
        ast.For(target=ast.Name(id="_nmk_i", ctx=ast.Store()),
                iter=ast.Call(func=ast.Name(id="_nmk_prange", ctx=ast.Load()),
                              args=[ast.Name(id="_nmk_n", ctx=ast.Load())], keywords=[]),
                body=[ast.AugAssign(target=ast.Name(id="_nmk_acc", ctx=ast.Store()),
                                    op=ast.Add(), value=expr)],
                orelse=[]),
        ast.Return(value=ast.Name(id="_nmk_acc", ctx=ast.Load())),
    ]
    fn = ast.FunctionDef(name=name, args=args, body=body, decorator_list=[])
    for node in [fn] + body:
        ast.copy_location(node, stage.node)
    module = ast.fix_missing_locations(ast.Module(body=[fn], type_ignores=[]))
    namespace = dict(scope)
    exec(compile(module, f"<stage of {name}>", "exec"), namespace)    # noqa: S102
    func = namespace[name]
    func.__nmk_ast__ = fn
    return func, params


def _indexed(expr, arrays, index):
    """``expr`` with every array name replaced by its element at ``index``
    (a list of expression nodes)."""
    import copy

    class Index(ast.NodeTransformer):
        def visit_Name(self, node):
            if node.id in arrays and isinstance(node.ctx, ast.Load):
                sub = ast.Tuple(elts=[copy.deepcopy(i) for i in index], ctx=ast.Load()) \
                    if len(index) > 1 else copy.deepcopy(index[0])
                return ast.copy_location(
                    ast.Subscript(value=node, slice=sub, ctx=ast.Load()), node)
            return node

    return Index().visit(copy.deepcopy(expr))


def _function(name, params, body_source, exprs, stage, scope):
    """Parses ``body_source`` (with the placeholders NMK_EXPR0, NMK_EXPR1, ...
    where the indexed expressions go) into a function and attaches its
    tree."""
    text = f"def {name}({', '.join(params)}):\n" + body_source
    module = ast.parse(text)

    class Put(ast.NodeTransformer):
        def visit_Name(self, node):
            if node.id.startswith("NMK_EXPR"):
                return exprs[int(node.id[len("NMK_EXPR"):])]
            return node

    module = Put().visit(module)
    fn = module.body[0]
    for node in ast.walk(fn):
        if not hasattr(node, "lineno"):
            continue
        node.lineno = node.end_lineno = stage.node.lineno
    ast.fix_missing_locations(module)
    namespace = dict(scope)
    exec(compile(module, f"<stage of {name}>", "exec"), namespace)    # noqa: S102
    func = namespace[name]
    func.__nmk_ast__ = fn
    return func


def _offset(name, k):
    node = ast.Name(id=name, ctx=ast.Load())
    return node if k == 0 else ast.BinOp(left=node, op=ast.Add(), right=ast.Constant(value=k))


ROW_LANES = 256       # work-group of the row-sum kernel


def row_sum_function(stage, name, scope, arrays, integer):
    """A @kernel body summing one map stage's expression along the rows of
    dense matrices: one work-group per row, lanes stride over the columns
    (four columns a work-group apart in flight), one work-group reduction.
    Parameters: the column count, the stage's inputs, the output vector.
    ``scope`` must bind _nmk_group_id, _nmk_local_id and _nmk_group (the
    kernel API)."""
    row = ast.Name(id="_nmk_row", ctx=ast.Load())
    exprs = [_indexed(stage.expr, arrays, [row, _offset("_nmk_j", k * ROW_LANES)])
             for k in range(4)]
    params = ["_nmk_cols"] + list(stage.inputs) + ["_nmk_out"]
    zero = "0" if integer else "0.0"
    body = f"""    _nmk_row = _nmk_group_id(0)
    _nmk_lid = _nmk_local_id(0)
    _nmk_a0 = {zero}
    _nmk_a1 = {zero}
    _nmk_a2 = {zero}
    _nmk_a3 = {zero}
    _nmk_whole = _nmk_cols - _nmk_cols % {4 * ROW_LANES}
    for _nmk_j in range(_nmk_lid, _nmk_whole, {4 * ROW_LANES}):
        _nmk_a0 += NMK_EXPR0
        _nmk_a1 += NMK_EXPR1
        _nmk_a2 += NMK_EXPR2
        _nmk_a3 += NMK_EXPR3
    for _nmk_j in range(_nmk_whole + _nmk_lid, _nmk_cols, {ROW_LANES}):
        _nmk_a0 += NMK_EXPR0
    _nmk_total = _nmk_group.reduce_add((_nmk_a0 + _nmk_a1) + (_nmk_a2 + _nmk_a3))
    if _nmk_lid == 0:
        _nmk_out[_nmk_row] = _nmk_total
"""
    return _function(name, params, body, exprs, stage, scope), params


# Thousands of rows of up to this many columns are not summed inside the map: a work-group
# per row would be mostly idle lanes and a work-item per row reads a cache
# line per lane and trip (1,048,576 x 16 float64: 1244 and 133 us); the map
# and the reduction kernels' short-row route take 45 + 42 us.
SHORT_ROW = 64


COLUMNS_PER_ITEM = 4      # adjacent columns per work-item of the column-sum kernel


def column_sum_function(stage, name, scope, arrays, integer):
    """A @kernel body summing one map stage's expression down the columns of
    dense matrices in chunks of rows: work-item (chunk, q) adds its chunk's
    rows of columns 4q .. 4q + 3 (a wave reads 256 adjacent columns of a row,
    two rows in flight) into partial[chunk, column]; the partial sums are
    added by the column-sum kernel.  The column count must be a multiple of
    four.  ``scope`` must bind _nmk_global_id."""
    n = COLUMNS_PER_ITEM
    exprs = [_indexed(stage.expr, arrays, [_offset("_nmk_i", r), _offset("_nmk_col", k)])
             for r in range(2) for k in range(n)]
    params = ["_nmk_rows", "_nmk_chunk"] + list(stage.inputs) + ["_nmk_part"]
    zero = "0" if integer else "0.0"
    lines = ["    _nmk_c = _nmk_global_id(0)", f"    _nmk_col = _nmk_global_id(1) * {n}"]
    lines += [f"    _nmk_a{k} = {zero}" for k in range(2 * n)]
    lines += ["    _nmk_first = _nmk_c * _nmk_chunk",
              "    _nmk_last = min(_nmk_first + _nmk_chunk, _nmk_rows)",
              "    _nmk_whole = _nmk_last - (_nmk_last - _nmk_first) % 2",
              "    for _nmk_i in range(_nmk_first, _nmk_whole, 2):"]
    lines += [f"        _nmk_a{k} += NMK_EXPR{k}" for k in range(2 * n)]
    lines += ["    for _nmk_i in range(_nmk_whole, _nmk_last):"]
    lines += [f"        _nmk_a{k} += NMK_EXPR{k}" for k in range(n)]
    lines += [f"    _nmk_part[_nmk_c, _nmk_col + {k}] = _nmk_a{k} + _nmk_a{k + n}"
              for k in range(n)]
    return _function(name, params, "\n".join(lines) + "\n", exprs, stage, scope), params
