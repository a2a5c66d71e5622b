"""GPU parity: randomly generated straight-line array functions under ``njit``
against the same functions run by NumPy.

Each function mixes broadcasting maps, NumPy's named functions, reductions
along an axis or over everything and matrix products, so it exercises the
splitting of a body into fused map kernels and library kernels, merged
dimensions, scalar stages on the host and the typing rules.  The generator is
seeded: the set of functions is fixed."""

import importlib.util
import os

import numpy as np
import pytest

from numba_mlir_amd.decorators import njit

pytestmark = pytest.mark.gpu

N_FUNCTIONS = 36
ROWS, COLS = 37, 53          # deliberately not multiples of the lane tiling


class _Gen:
    """Expressions are (source, kind): kind "m" is a [ROWS, COLS] matrix, "r" a
    [COLS] row, "c" a [ROWS, 1] column, "s" a scalar."""

    def __init__(self, rng):
        self.rng = rng

    def pick(self, items):
        return items[int(self.rng.integers(len(items)))]

    def leaf(self, kind):
        if kind == "m":
            return self.pick(["a", "b", "(a - b)"])
        if kind == "r":
            return self.pick(["r", "(r * 0.5)"])
        if kind == "c":
            return "c"
        return self.pick(["2.0", "0.25", "s", "3"])

    def expr(self, kind, depth):
        if depth == 0 or self.rng.random() < 0.15:
            return self.leaf(kind)
        choice = self.rng.random()
        if kind == "s":
            if choice < 0.45:
                red = self.pick(["np.sum", "np.max", "np.min", "np.mean"])
                return f"{red}({self.expr(self.pick(['m', 'r']), depth - 1)})"
            if choice < 0.6:
                return f"np.dot({self.expr('r', depth - 1)}, {self.expr('r', depth - 1)})"
            op = self.pick(["+", "-", "*"])
            return f"({self.expr('s', depth - 1)} {op} {self.leaf('s')})"
        if kind == "r" and choice < 0.3:
            red = self.pick(["np.sum", "np.max", "np.mean", "np.min"])
            return f"{red}({self.expr('m', depth - 1)}, axis=0)"
        if kind == "r" and choice < 0.4:
            return f"np.dot({self.expr('r', depth - 1)}, mm)"
        if kind == "c" and choice < 0.4:
            red = self.pick(["np.sum", "np.max", "np.mean"])
            return f"{red}({self.expr('m', depth - 1)}, axis=1).reshape({ROWS}, 1)"
        if kind == "m" and choice < 0.12:
            return f"np.dot({self.expr('m', depth - 1)}, mm)"
        if choice < 0.6:
            op = self.pick(["+", "-", "*"])
            other = self.pick({"m": ["m", "r", "c", "s"], "r": ["r", "s"],
                               "c": ["c", "s"]}[kind])
            x, y = self.expr(kind, depth - 1), self.expr(other, depth - 1)
            return f"({x} {op} {y})" if self.rng.random() < 0.5 else f"({y} {op} {x})"
        if choice < 0.8:
            fn = self.pick(["np.sin", "np.cos", "np.abs", "np.tanh", "np.square",
                            "np.negative"])
            return f"{fn}({self.expr(kind, depth - 1)})"
        if choice < 0.9:
            fn = self.pick(["np.maximum", "np.minimum", "np.add", "np.subtract"])
            return f"{fn}({self.expr(kind, depth - 1)}, {self.expr(kind, depth - 1)})"
        x, y = self.expr(kind, depth - 1), self.expr(kind, depth - 1)
        return f"np.where({x} > {y}, {x}, {y} * 0.5)"

    def function(self, index):
        lines = [f"def f{index}(a, b, r, c, mm, s):"]
        names = {"m": ["a", "b"], "r": ["r"], "c": ["c"], "s": ["s"]}
        for k in range(int(self.rng.integers(1, 4))):
            kind = self.pick(["m", "r", "c", "s"])
            lines.append(f"    t{k} = {self.expr(kind, 3)}")
            names[kind].append(f"t{k}")
        kind = self.pick(["m", "m", "r", "c", "s"])
        ret = self.expr(kind, 2)
        # fold the temporaries in so that none is dead
        for k_kind, k_names in names.items():
            for name in k_names:
                if name.startswith("t"):
                    if k_kind == kind or kind == "m" or k_kind == "s":
                        ret = f"({ret} + {name})"
                    else:
                        ret = f"({ret} + np.sum({name}))"
        lines.append(f"    return {ret}")
        return "\n".join(lines)


@pytest.fixture(scope="module")
def functions(tmp_path_factory):
    gen = _Gen(np.random.default_rng(2024))
    source = "import numpy as np\n\n\n" + "\n\n\n".join(
        gen.function(k) for k in range(N_FUNCTIONS)) + "\n"
    path = os.path.join(tmp_path_factory.mktemp("random_njit"), "random_functions.py")
    with open(path, "w") as f:
        f.write(source)
    spec = importlib.util.spec_from_file_location("random_functions", path)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module, source


@pytest.mark.parametrize("index", range(N_FUNCTIONS))
def test_random_function(hip, functions, index):
    module, source = functions
    func = getattr(module, f"f{index}")
    rng = np.random.default_rng(100 + index)
    a, b = rng.uniform(-1, 1, (ROWS, COLS)), rng.uniform(-1, 1, (ROWS, COLS))
    r, c = rng.uniform(-1, 1, COLS), rng.uniform(-1, 1, (ROWS, 1))
    mm = rng.uniform(-1, 1, (COLS, COLS)) / COLS
    s = 0.75
    want = func(a, b, r, c, mm, s)
    got = njit(func)(hip.asarray(a), hip.asarray(b), hip.asarray(r), hip.asarray(c),
                     hip.asarray(mm), s)
    got = got.asnumpy() if hasattr(got, "asnumpy") else got
    text = source.split(f"def f{index}(")[1].split("\n\n\n")[0]
    assert np.shape(got) == np.shape(want), text
    # sums of ~2000 terms in another order, products through the MFMA kernel
    np.testing.assert_allclose(got, want, rtol=1e-9, atol=1e-9, err_msg=text)
