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

/*
 * mkl_gemm_float32_device for callers that cannot allocate device memory
 * (tight serving loops, harnesses that forbid hipMalloc).  No counterpart in
 * the reference.  Same arguments as mkl_gemm_float32_device; it calls no
 * hipMalloc / hipFree.  Like that entry point it returns when C is complete
 * (it synchronises the queue's stream), so it cannot be issued on a stream
 * that is being captured into a HIP graph.  Where that
 * entry point takes its workspace from a heap block it grows on demand, this
 * one uses a fixed 16 MiB array that lives in the library's device image on
 * every GPU it runs on, and shares K out over the blocks by split K only
 * (the even shares of K slabs the allocating entry point may take instead
 * need up to 128 MiB): where both run the same kernel the results agree bit
 * for bit, elsewhere to float32's accuracy.  The first
 * call on a device looks the array's address up (no allocation).  Returns 0,
 * or 1 -- with a message on stderr and nothing launched -- when the product
 * would need more split-K workspace than the array holds.  Only shapes with
 * fewer than 128 tiles of 128 x 128 split K, into slices x tiles <= 256
 * partial tiles of 64 KiB: 16 MiB is the most a float32 product asks for
 * (1024 x 1024 with k >= 512 does), so the limit is a guard, not a case a
 * float32 caller meets.  The array is shared by every call on a GPU and
 * keeps the last call's partial products; nothing in it needs clearing,
 * each slice is written before it is read.  Calls from several host
 * threads take turns on it (the library holds a lock while a call's kernels
 * run).
 */
int mkl_gemm_float32_device_noalloc(void *queue, const NmhipMemref2F32 *a,
                                    const NmhipMemref2F32 *b, float alpha,
                                    float beta, NmhipMemref2F32 *c);

/* NumpyLinalg.cpp:178-183.  Not thread safe, as in the reference. */
void nmrtMathRuntimeInit(void);
void nmrtMathRuntimeFinalize(void);

/* Name of the device kernel the most recent gemm call on this thread ran
 * ("sgemm_mfma_256x256", "sgemm_mfma_128x128", "dgemm_mfma_128x128",
 * "sgemm_generic", "dgemm_generic"; "<tile kernel>_ragged" for the guarded
 * instance that takes shapes which are not whole tiles, "_even" after the
 * tile kernel's name when the blocks took even shares of all K slabs, "_splitk" after
 * either when K was cut into slices, "<tile kernel>+edges" when the strided
 * kernel completed what the tiles left, "+packed" when an operand whose rows
 * do not begin and end on 128-bit words was first copied into padded rows);
 * for tests and profiling. */
const char *nmhipMathLastKernel(void);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* NUMBA_MLIR_HIP_MATH_RUNTIME_H */
