"""Build-time check of the @kernel translator: one body that touches the
support header's main parts is translated and compiled for gfx950 (hipcc
cross-compiles; no GPU is needed)."""

import math

from . import kernel_compiler as kc
from . import kernel_impl
from .kernel_impl import atomic, barrier, get_global_id, group, local, private


def sample(X1, X2, D, hist):
    i = get_global_id(0)
    j = get_global_id(1)
    tile = local.array((4, 4), "float64")
    acc = private.array(3, "float64")
    d = 0.0
    for k in range(X1.shape[1]):
        acc[k] = X1[i, k] - X2[j, k]
        d += acc[k] * acc[k]
    tile[i % 4, j % 4] = d
    barrier()
    D[i, j] = math.sqrt(d) + group.reduce_max(tile[j % 4, i % 4]) % 3
    atomic.add(hist, (i + j) // 7 % 5, 1)


def compile_sample():
    dense = kc.Array(kc.FLOAT64, 2, layout="C", const_shape=(None, 3))
    types = [dense, dense, kc.Array(kc.FLOAT64, 2), kc.Array(kc.INT64, 1)]
    for boundscheck in (False, True):
        compiled = kc.translate(sample, types, 2, kernel_impl, boundscheck=boundscheck)
        kc.build_code_object(compiled)
