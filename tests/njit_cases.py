"""Functions shared by the CPU (translate + compile) and GPU (run) tests of
``njit``.  The Black-Scholes bodies restate the formula of the reference's
fused-loop test (numba_mlir/numba_mlir/mlir/tests/test_numpy.py:2827-2852),
once over whole arrays and once as a prange loop."""

import math

import numpy as np

from numba_mlir_amd.decorators import prange, vectorize


@vectorize(nopython=True)
def _erf(x):
    return math.erf(x)


def black_scholes_arrays(price, strike, t, rate, volatility, call, put):
    mr = -rate
    sig_sig_two = volatility * volatility * 2
    P = price
    S = strike
    T = t
    a = np.log(P / S)
    b = T * mr
    z = T * sig_sig_two
    c = 0.25 * z
    y = 1.0 / np.sqrt(z)
    w1 = (a - b + c) * y
    w2 = (a - b - c) * y
    d1 = 0.5 + 0.5 * _erf(w1)
    d2 = 0.5 + 0.5 * _erf(w2)
    Se = np.exp(b) * S
    r = P * d1 - Se * d2
    call[:] = r
    put[:] = r - P + Se


def black_scholes_loop(nopt, price, strike, t, rate, volatility, call, put):
    mr = -rate
    sig_sig_two = volatility * volatility * 2
    for i in prange(nopt):
        P = price[i]
        S = strike[i]
        T = t[i]
        a = math.log(P / S)
        b = T * mr
        z = T * sig_sig_two
        c = 0.25 * z
        y = 1.0 / math.sqrt(z)
        w1 = (a - b + c) * y
        w2 = (a - b - c) * y
        d1 = 0.5 + 0.5 * math.erf(w1)
        d2 = 0.5 + 0.5 * math.erf(w2)
        Se = math.exp(b) * S
        r = P * d1 - Se * d2
        call[i] = r
        put[i] = r - P + Se


def add(a, b):
    return a + b


def fused_map(a, b, c, scale):
    t = a * scale + np.sin(b)
    u = np.where(t > c, t, c) / (1.0 + np.abs(c))
    return np.maximum(u, 0.25) ** 2 - t


def fused_store(x, y, out_f, out_i):
    s = x + y
    out_f[:] = np.sqrt(np.abs(s)) * 0.5
    out_i[...] = x // 3 + y % 5


def saxpy_loop(alpha, x, y, out):
    n = len(x)
    for i in prange(n):
        out[i] = alpha * x[i] + y[i]


def strided_loop(x, out):
    for i in prange(1, x.shape[0] - 1, 2):
        acc = 0.0
        for k in range(x.shape[1]):
            acc += x[i, k] * (x[i - 1, k] + x[i + 1, k])
        out[i] = acc


def row_sums(x):
    return np.sum(x, axis=1)


def col_sums(x):
    return x.sum(axis=0)


def norm(x):
    return np.sqrt(np.sum(x * x))


def matmul(a, b):
    return a @ b


def dot(a, b):
    return np.dot(a, b)


def statements_after_loop(x, out):
    for i in prange(len(x)):
        out[i] = x[i]
    out[0] = 0.0


def two_returns(a):
    if True:
        return a + 1
    return a


def no_loop(x):
    y = 1


def sum_of_squares(x):
    s = 0.0
    for i in prange(len(x)):
        s += x[i] * x[i]
    return math.sqrt(s)


def mean_and_count(x, threshold):
    total = 0.0
    above = 0
    n = x.shape[0]
    for i in prange(n):
        total += x[i]
        if x[i] > threshold:
            above += 1
    return total / n, above


def int_dot(a, b):
    acc = 10
    for i in prange(len(a)):
        acc += a[i] * b[i]
    return acc


def product(x):
    p = 2.0
    for i in prange(x.shape[0]):
        p *= x[i]
    return p


def reduction_read_in_loop(x):
    s = 0.0
    for i in prange(len(x)):
        s += x[i]
        x[i] = s
    return s


def parfor_add(a, b, c):
    for i in prange(len(a)):
        c[i] = a[i] + b[i]


def parfor_scalar(a, b, c, d):
    for i in prange(len(a)):
        c[i] = a[i] + b[i] + d


def nested_prange(a):
    ah, aw = a.shape
    for h in prange(ah):
        for w in prange(aw):
            a[h, w] = w + h * aw


def scale_into(a, b):
    b[:] = a * 2


def add_into(a, b, c):
    c[:] = a + b


def loop_reads(n, a, b, c, out):
    for i in prange(n):
        x = a[i] + out[i]
        y = b[i] if x > 0 else 0.0
        if y > 1.0:
            y = c[i]
        out[i] = x + y


def loop_leaves_early(n, a, out):
    for i in prange(n):
        if i % 2:
            continue
        out[i] = a[i]


def scale_in_place(a, b):
    x = a
    x[:] = a * b + 1.0


def fill(a):
    a[:] = 42


def _smoothstep(x, lo, hi):
    t = min(max((x - lo) / (hi - lo), 0.0), 1.0)
    return t * t * (3.0 - 2.0 * t)



# NumPy's named forms of the operators (the reference registers each body under
# both names, numpy/funcs.py:362-383 and 457-562), one per line so that each
# lambda's source is found.  (name, function, operand kinds)
NAMED_UFUNCS = [
    ("add", lambda a, b: np.add(a, b), "fi"),
    ("subtract", lambda a, b: np.subtract(a, b), "fi"),
    ("multiply", lambda a, b: np.multiply(a, b), "fi"),
    ("true_divide", lambda a, b: np.true_divide(a, b), "fi"),
    ("power", lambda a, b: np.power(a, b), "p"),
    ("arctan2", lambda a, b: np.arctan2(a, b), "f"),
    ("minimum", lambda a, b: np.minimum(a, b), "fi"),
    ("maximum", lambda a, b: np.maximum(a, b), "fi"),
    ("logical_and", lambda a, b: np.logical_and(a, b), "fib"),
    ("logical_or", lambda a, b: np.logical_or(a, b), "fib"),
    ("logical_xor", lambda a, b: np.logical_xor(a, b), "fib"),
    ("less", lambda a, b: np.less(a, b), "fi"),
    ("greater", lambda a, b: np.greater(a, b), "fi"),
    ("less_equal", lambda a, b: np.less_equal(a, b), "fi"),
    ("greater_equal", lambda a, b: np.greater_equal(a, b), "fi"),
    ("equal", lambda a, b: np.equal(a, b), "fib"),
    ("not_equal", lambda a, b: np.not_equal(a, b), "fib"),
    ("bitwise_and", lambda a, b: np.bitwise_and(a, b), "ib"),
    ("bitwise_or", lambda a, b: np.bitwise_or(a, b), "ib"),
    ("bitwise_xor", lambda a, b: np.bitwise_xor(a, b), "ib"),
    ("left_shift", lambda a, b: np.left_shift(a, b), "s"),
    ("right_shift", lambda a, b: np.right_shift(a, b), "s"),
    ("floor_divide", lambda a, b: np.floor_divide(a, b), "fi"),
    ("remainder", lambda a, b: np.remainder(a, b), "fi"),
]

NAMED_UNARY = [
    ("sqrt", lambda a: np.sqrt(a), "p"),
    ("square", lambda a: np.square(a), "fi"),
    ("log", lambda a: np.log(a), "p"),
    ("sin", lambda a: np.sin(a), "f"),
    ("cos", lambda a: np.cos(a), "f"),
    ("exp", lambda a: np.exp(a), "f"),
    ("tanh", lambda a: np.tanh(a), "f"),
    ("abs", lambda a: np.abs(a), "fi"),
    ("negative", lambda a: np.negative(a), "fi"),
    ("positive", lambda a: np.positive(a), "fi"),
    ("logical_not", lambda a: np.logical_not(a), "fib"),
    ("invert", lambda a: np.invert(a), "i"),
    ("neg", lambda a: -a, "fi"),
    ("pos", lambda a: +a, "fi"),
    ("inv", lambda a: ~a, "i"),
]


def clip_scalars(a):
    return np.clip(a, -0.5, 0.75)


def clip_arrays(a, lo, hi):
    return np.clip(a, lo, hi)


def mean_all(x):
    return np.mean(x)


def mean_rows(x):
    return x.mean(axis=1)


def mean_cols(x):
    return np.mean(x, axis=0)


# straight-line bodies that mix maps with reductions / contractions
def l2_norm_rows(a):
    return np.sqrt(np.square(a).sum(axis=1))


def softmax(x):
    e = np.exp(x - np.max(x))
    return e / np.sum(e)


def standardise(x):
    m = np.mean(x, axis=0)
    d = x - m
    return d / np.sqrt(np.mean(d * d, axis=0))


def affine(a, b, c):
    return np.dot(a, b) + c


def chain(a, b, c):
    return a @ b @ c


def cosine(x, y):
    return np.dot(x, y) / (np.sqrt(np.sum(x * x)) * np.sqrt(np.sum(y * y)))


def weighted_rows(a, w, out):
    s = np.sum(a * w, axis=1)
    s += 1.0
    out[:] = s * 2.0


def matvec(a, v):
    return np.dot(a, v * 2.0) - 1.0


def column_range(x):
    return x.max(axis=0) - np.min(x, axis=0)


def dot_out_positional(a, b, c):
    return np.dot(a, b, c)


def dot_out_keyword(a, b, c):
    return np.dot(a, b, out=c)


def reshape_fill(a):
    b = a.reshape(17, 23, 56)
    b[:] = 42


def transposed_sum(a):
    return np.sum(a.T * 2.0, axis=1)


def pairwise_loop(X1, X2, D):
    X1_rows = X1.shape[0]
    X2_rows = X2.shape[0]
    X1_cols = X1.shape[1]

    for i in prange(X1_rows):
        for j in prange(X2_rows):
            d = 0.0
            for k in range(X1_cols):
                tmp = X1[i, k] - X2[j, k]
                d += tmp * tmp
            D[i, j] = np.sqrt(d)


def batchnorm(x, eps=1e-5):
    # test_numpy.py's test_batchnorm body
    mean = np.empty(x.shape, dtype=x.dtype)
    mean[:] = np.sum(x, axis=0) / x.shape[0]
    std = np.empty(x.shape, dtype=x.dtype)
    std[:] = np.sqrt(np.sum((x - mean) ** 2, axis=0) / x.shape[0])
    return (x - mean) / np.sqrt(std + eps)


def batchnorm4(x, eps):
    mean = np.empty(x.shape, dtype=x.dtype)
    mean[:] = np.sum(x, axis=0) / x.shape[0]
    std = np.empty(x.shape, dtype=x.dtype)
    std[:] = np.sqrt(np.sum((x - mean) ** 2, axis=0) / x.shape[0])
    return (x - mean) / np.sqrt(std + eps)


def broadcast_setitem(a, b):
    a[:] = b
    return a


OUT_FORMS = [
    ("add", lambda a, b, c: np.add(a, b, c)),
    ("subtract", lambda a, b, c: np.subtract(a, b, out=c)),
    ("multiply", lambda a, b, c: np.multiply(a, b, c)),
    ("true_divide", lambda a, b, c: np.true_divide(a, b, c)),
    ("power", lambda a, b, c: np.power(a, b, c)),
    ("minimum", lambda a, b, c: np.minimum(a, b, c)),
    ("maximum", lambda a, b, c: np.maximum(a, b, out=c)),
    ("sqrt", lambda a, b, c: np.sqrt(a, c)),
    ("exp", lambda a, b, c: np.exp(b, out=c)),
]


def clip_out(a, lo, hi, out):
    return np.clip(a, lo, hi, out=out)


def zeros_ones(x):
    z = np.zeros(x.shape, dtype=np.float32)
    o = np.ones_like(x)
    e = np.empty_like(x)
    e[:] = x + o
    return e * 2 + z


TRANSPOSES = [
    ((0, 1, 2), lambda a: np.transpose(a, (0, 1, 2))),
    ((0, 2, 1), lambda a: np.transpose(a, (0, 2, 1))),
    ((1, 0, 2), lambda a: np.transpose(a, (1, 0, 2))),
    ((1, 2, 0), lambda a: np.transpose(a, (1, 2, 0))),
    ((2, 0, 1), lambda a: np.transpose(a, (2, 0, 1))),
    ((2, 1, 0), lambda a: np.transpose(a, (2, 1, 0))),
    ("T", lambda a: a.T),
    ("method", lambda a: a.transpose(1, 0, 2) * 2),
]

FLIPS = [
    ("all", lambda a: np.flip(a)),
    ("axis0", lambda a: np.flip(a, 0)),
    ("axis1", lambda a: np.flip(a, 1)),
    ("axis-1", lambda a: np.flip(a, -1)),
    ("flip+map", lambda a: np.flip(a, 1) + a),
]


def l2_norm_rows_product(a):
    return np.sqrt(np.sum(a * a, axis=1))


# reductions over everything of a map: one pass over the operands
def frobenius(a, b):
    return np.sqrt(np.sum((a - b) ** 2))


def mean_abs_difference(a, b):
    return np.mean(np.abs(a - b))


def count_greater(a, b):
    return np.sum(a > b)


def sum_of_integer_squares(a):
    return np.sum(a * a)


def weighted_total(a, r):
    return np.sum(a * r)          # broadcast operands: two stages


# reductions along an axis of a map over same-shaped matrices: one pass
def row_dots(a, b):
    return np.sum(a * b, axis=1)


def column_variance(x, m):
    return np.mean((x - m) ** 2, axis=0)


def row_mean_abs(a, b, s):
    return np.mean(np.abs(a - b) * s, axis=-1)


def column_counts(a, b):
    return np.sum(a > b, axis=0)


# -- arrays built and sliced inside a compiled function ----------------------
# (numpy/funcs.py:236-310 views and copies, 642-700 arange and eye, 1455-1549
# cov; tril/triu/outer/concatenate/hstack/vstack are registered there too)
def built_arange_steps(a):
    return a[:50] * np.arange(0.5, 25.5, 0.5)


def built_arange_count(a):
    return a + np.arange(5000)


def built_arange_down(a):
    return np.arange(10, 2, -3) + 0 * a[:3]


def built_eye(a):
    return a @ np.eye(200, 100, k=-3)


def built_eye_square(a):
    return a[:200] + np.eye(200)


def built_triangles(a):
    return np.triu(a, 2) - np.tril(a, -1)


def built_outer(a, b):
    return np.outer(a + 1, b * 2).sum(axis=0)


def built_concatenate_columns(a, b):
    return np.concatenate((a, b), axis=1)


def built_concatenate_three(a, b):
    return np.concatenate((a, b, a), axis=-2)


def built_vstack(a, b):
    return np.vstack((a, b))


def built_hstack(a, b):
    return np.hstack((a, b))


def built_cov(a):
    return np.cov(a)


def built_cov_pair(a, b):
    return np.cov(a, b)


def built_cov_columns(a):
    return np.cov(a, rowvar=False, bias=True)


def sliced_sums(a):
    return a[1:-1, ::2].sum() + a[:, 3].sum() + a[5].sum()


def sliced_differences(a):
    return (a[1:] - a[:-1]).sum(axis=0)


def sliced_row(a):
    return a[5] * 2.0


def sliced_row_part(a):
    return a[5, 1:4] * 2.0


def sliced_element(a):
    return a - a[0, 0]


def sliced_element_returned(a):
    return a[2, 3]


def copied_transpose(a):
    return np.copy(a.T)


def copied_method(a):
    return a.copy()


def flattened_transpose(a):
    return a.T.flatten()


def facts_in_a_map(a):
    return a * a.shape[0] + a.size + a.ndim


def facts_after_a_reduction(a):
    return np.sum(a, axis=0) / a.shape[0]


def facts_of_layout(a):
    return a * a.itemsize + a.strides[0] + len(a) + a.shape[1]


def facts_dtype(a):
    return np.zeros(a.shape, a.dtype) + a


def converted(a):
    return (a * 10).astype(np.int32).astype(np.float64) * 0.5


def converted_down(a):
    return a.astype(np.float32)


def built_dstack(a, b):
    return np.dstack((a, b))


def copied_fortran(a):
    return np.asfortranarray(a) * 2.0


def store_slice(a, b):
    a[1:5] = b[:4] * 2.0


def store_column(a, b):
    a[:, 3] = 1.5


def store_block_and_update_row(a, b):
    a[1:-1, 2:5] = b[:-2, :3] * 2.0
    a[0, :] -= 1.0


def update_shifted(a, b):
    a[1:] += b[:-1]


def facts_under_a_branch(a, flag):
    r = a - a.shape[1]
    if flag:
        r = a * a.shape[0] + len(a)
    return r


def facts_of_a_stretched_operand(a, b, flag):
    r = a
    if flag:
        r = a + b.shape[0]
    return r


def update_overlapping(a):
    a[1:] += a[:-1]


def store_overlapping(a):
    a[:-1] = a[1:] * 2


def store_reversed_onto_itself(a):
    a[:] = a[::-1] + 1.0


def inverted(a):
    return ~a


def store_row_and_elements(a, b):
    a[5] = b[7] * 2.0
    a[0, 1] = 3.5
    a[2, 2] += 1.0
    a[-1] -= b[0]


def distances_to_centres(X, C):
    return (X * X).sum(axis=1).reshape(-1, 1) - 2 * X @ C.T + (C * C).sum(axis=1)


def softmax_rows(x):
    e = np.exp(x - x.max(axis=1).reshape(-1, 1))
    return e / e.sum(axis=1).reshape(-1, 1)


def covariance_of_columns(X):
    Xc = X - X.mean(axis=0)
    return Xc.T @ Xc / (X.shape[0] - 1)


def ridge_gradient(X, y, w, lam):
    r = X @ w - y
    return X.T @ r / X.shape[0] + lam * w


def cosine_to_centres(X, C):
    xn = np.sqrt((X * X).sum(axis=1)).reshape(-1, 1)
    cn = np.sqrt((C * C).sum(axis=1)).reshape(1, -1)
    return (X @ C.T) / (xn * cn)
