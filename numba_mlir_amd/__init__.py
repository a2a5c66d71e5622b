"""MI355X (gfx950) GPU-offload backend for numba-mlir.

The package holds the HIP implementation of the ``gpux*`` runtime C-ABI, the
device gemm behind ``mkl_gemm_<dtype>_device``, hand-written CDNA4 kernels for
the data-parallel hot path and the host code that drives them.  Native
libraries are built in-tree by ``numba_mlir_amd.build``; importing
``numba_mlir_amd.mlir.lowered`` (or anything that uses the GPU) fails loudly
if they are missing.
"""

__all__ = ["build"]
