/*
 * C-ABI of the HIP math runtime, libnumba-mlir-math-hip-runtime.so: the device
 * gemm the compiler calls for np.dot / @ inside a GPU region.
 *
 * Replaces libnumba-mlir-math-sycl-runtime.so (reference:
 * numba_mlir/numba_mlir/math_runtime/sycl/lib/NumpyLinalg.cpp:67-183), which
 * forwards to oneMKL.  Same entry points, same argument meaning:
 *
 *   c = alpha * op(a) * op(b) + beta * c
 *
 * with a [m, k], b [k, n], c [m, n] described by 2-D memrefs.  Which operand
 * is transposed and whether c is row- or column-major is derived from which
 * stride equals 1 (NumpyLinalg.cpp:87-102); an operand with no unit stride is
 * fatal (73-85).  The call blocks until c is complete (127, 145).
 *
 * `queue` is the pointer returned by gpuxQueueCreate.
 */
#ifndef NUMBA_MLIR_HIP_MATH_RUNTIME_H
#define NUMBA_MLIR_HIP_MATH_RUNTIME_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Layout of Memref<2, T> (reference:
 * numba_mlir/numba_mlir/math_runtime/include/Common.hpp:17-28).  The first
 * element is data[offset]; dims and strides are in elements. */
typedef struct NmhipMemref2F32 {
  void *userData;
  float *data;
  size_t offset;
  size_t dims[2];
  size_t strides[2];
} NmhipMemref2F32;

typedef struct NmhipMemref2F64 {
  void *userData;
  double *data;
  size_t offset;
  size_t dims[2];
  size_t strides[2];
} NmhipMemref2F64;

/* NumpyLinalg.cpp:166-175 (registered for the JIT as
 * _mlir_ciface_mkl_gemm_<dtype>_device, math_runtime.py:21-40). */
void mkl_gemm_float32_device(void *queue, const NmhipMemref2F32 *a,
                             const NmhipMemref2F32 *b, float alpha, float beta,
                             NmhipMemref2F32 *c);
void mkl_gemm_float64_device(void *queue, const NmhipMemref2F64 *a,
                             const NmhipMemref2F64 *b, double alpha,
                             double beta, NmhipMemref2F64 *c);

/* NumpyLinalg.cpp:178-183.  Not thread safe, as in the reference. */
void nmrtMathRuntimeInit(void);
void nmrtMathRuntimeFinalize(void);

/* Name of the device kernel the most recent gemm call on this thread ran
 * ("sgemm_mfma_256x256", "sgemm_mfma_128x128", "dgemm_mfma_128x128",
 * "sgemm_generic", "dgemm_generic"; "<tile kernel>_ragged" for the guarded
 * instance that takes shapes which are not whole tiles, "_splitk" after
 * either when K was cut into slices, "<tile kernel>+edges" when the strided
 * kernel completed what the tiles left); for tests and profiling. */
const char *nmhipMathLastKernel(void);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* NUMBA_MLIR_HIP_MATH_RUNTIME_H */
