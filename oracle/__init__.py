"""TEST INFRASTRUCTURE -- not part of the product.

CPU oracle for the offloaded hot path.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package; nothing under ``numba_mlir_amd/`` does.
"""
