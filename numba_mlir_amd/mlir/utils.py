"""Library discovery and environment helpers.

Mirrors the reference's loader (reference:
numba_mlir/numba_mlir/mlir/utils.py:17-42, 71-82): runtime libraries are
``lib<name>.so`` in the package directory or on ``PYTHONPATH`` and are opened
with ``ctypes.CDLL``.
"""

import ctypes
import os
import sys
import warnings

_PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_lib(name):
    search_paths = [_PACKAGE_DIR]
    try:
        search_paths += os.environ["PYTHONPATH"].split(os.pathsep)
    except KeyError:
        pass

    if not sys.platform.startswith("linux"):
        raise ValueError("the HIP backend is Linux-only")
    lib_name = f"lib{name}.so"

    errors = []
    for path in search_paths:
        lib_path = lib_name if len(path) == 0 else os.path.join(path, lib_name)
        try:
            return ctypes.CDLL(lib_path)
        except OSError as e:
            errors.append(f'CDLL("{lib_path}"): {e}')

    raise ValueError(f'load_lib("{name}") failed:\n' + "\n".join(errors))


def mlir_func_name(name):
    return "_mlir_ciface_" + name


def readenv(name, ctor, default):
    value = os.environ.get(name)
    if value is None:
        return default() if callable(default) else default
    try:
        return ctor(value)
    except Exception:
        warnings.warn(
            "environ %s defined but failed to parse '%s'" % (name, value),
            RuntimeWarning,
        )
        return default
