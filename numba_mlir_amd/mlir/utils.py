"""Finding the runtime libraries, naming their symbols, reading settings.

The conventions are the reference's (reference:
numba_mlir/numba_mlir/mlir/utils.py:17-42, 71-82): a runtime library is the
file ``lib<name>.so``; it is looked for beside the package first and then in
every ``PYTHONPATH`` entry (an empty entry leaves the search to the dynamic
loader); functions the compiled code calls through a C interface wrapper
carry the prefix ``_mlir_ciface_``; a setting comes from the environment,
and a value that does not parse is reported with a warning and replaced by
the default.
"""

import ctypes
import os
import pathlib
import sys
import warnings

PACKAGE_DIR = pathlib.Path(__file__).resolve().parent.parent
CIFACE_PREFIX = "_mlir_ciface_"


class LibraryNotFound(ValueError):
    """No candidate file for a runtime library could be opened."""


def _candidate_files(file_name):
    yield str(PACKAGE_DIR / file_name)
    for entry in os.environ.get("PYTHONPATH", "").split(os.pathsep):
        yield os.path.join(entry, file_name) if entry else file_name


def load_lib(name):
    """Opens ``lib<name>.so``; raises LibraryNotFound listing every attempt."""
    if not sys.platform.startswith("linux"):
        raise LibraryNotFound("the HIP backend is Linux-only")
    attempts = []
    seen = set()
    for candidate in _candidate_files(f"lib{name}.so"):
        if candidate in seen:
            continue
        seen.add(candidate)
        try:
            return ctypes.CDLL(candidate)
        except OSError as err:
            attempts.append(f"  {candidate}: {err}")
    raise LibraryNotFound(
        f'load_lib("{name}") failed, tried:\n' + "\n".join(attempts))


def mlir_func_name(name):
    return CIFACE_PREFIX + name


def readenv(name, ctor, default):
    """``ctor(os.environ[name])``, or the default (called when callable) if
    the variable is unset or does not parse."""
    fallback = default() if callable(default) else default
    raw = os.environ.get(name)
    if raw is None:
        return fallback
    try:
        return ctor(raw)
    except Exception as err:  # noqa: BLE001 - any parser may be passed in
        warnings.warn(f"ignoring {name}={raw!r}: {err}", RuntimeWarning,
                      stacklevel=2)
        return fallback
