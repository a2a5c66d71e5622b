/*
 * Host side of the offloaded hot path: what an @njit / @kernel function is
 * lowered to in the reference, written once by hand in C++.
 *
 * In the reference the compiler turns every GPU region into host code that
 * calls the gpux* C-ABI in a fixed order (reference:
 * mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:228-857) with the queue, module and
 * kernel handles created once and cached in a per-function context
 * (mlir_compiler/lib/pipelines/LowerToGpu.cpp:742-940,
 * numba_mlir_runtime/lib/Context.cpp:25-60):
 *
 *   first call : gpuxQueueCreate -> gpuxModuleLoad -> gpuxKernelGet   (cached)
 *   every call : [gpuxSuggestBlockSize] -> [gpuxAlloc, gpuxWait,
 *                gpuxDestroyEvent] -> gpuxLaunchKernel -> gpuxWait ->
 *                gpuxDestroyEvent
 *   unload     : gpuxKernelDestroy, gpuxModuleDestroy, gpuxQueueDestroy
 *
 * libnumba-mlir-hip-offload.so replays exactly that sequence.  It holds the
 * dispatcher that maps an op descriptor (family, dtype, layout) to one of the
 * hand-written gfx950 kernels, and the code objects themselves.  It reaches
 * the GPU only through function pointers registered with
 * nmhipRegisterSymbol, the counterpart of the reference's symbol registration
 * for JIT'd code (numba_mlir/numba_mlir/mlir/gpu_runtime.py:34-79,
 * mlir_compiler/lib/Lowering.cpp:1554-1561) and makes no HIP call of its own:
 * the library does not link the HIP runtime.
 *
 * Every pointer named `dev` / a / b / out / x ... is a device-accessible
 * pointer obtained from nmhipAlloc (or gpuxAlloc).  Sizes and strides are in
 * ELEMENTS.  Errors follow the gpux convention: message on stdout, abort().
 */
#ifndef NUMBA_MLIR_HIP_OFFLOAD_H
#define NUMBA_MLIR_HIP_OFFLOAD_H

#include <stddef.h>
#include <stdint.h>

#include "numba_mlir_hip/GpuRuntime.h"

#ifdef __cplusplus
extern "C" {
#endif

enum NmhipDType {
  NMHIP_I32 = 0,
  NMHIP_I64 = 1,
  NMHIP_F32 = 2,
  NMHIP_F64 = 3
};

/* NMHIP_DIV: float32 and float64 only (true division). */
enum NmhipBinaryOp { NMHIP_ADD = 0, NMHIP_SUB = 1, NMHIP_MUL = 2, NMHIP_DIV = 3 };

enum NmhipReduceOp {
  NMHIP_SUM = 0,
  NMHIP_PROD = 1,
  NMHIP_MIN = 2,
  NMHIP_MAX = 3
};

/* ---- symbol table ------------------------------------------------------ */

/*
 * Registers the address of a runtime entry point under its C name: the 13
 * gpux* functions and mkl_gemm_float32_device / mkl_gemm_float64_device.
 * Calling an op whose symbol was never registered is fatal.  Returns 0, or
 * -1 when `name` is not a symbol the lowered code uses (the reference binds
 * unknown intrinsic placeholders to a dummy address, gpu_runtime.py:74-79).
 */
int nmhipRegisterSymbol(const char *name, void *address);

/* ---- context (queue + cached module/kernel handles) -------------------- */

void *nmhipContextCreate(const char *deviceName);
void nmhipContextDestroy(void *ctx);

/*
 * async == 0 (default): every launch is followed by gpuxWait +
 * gpuxDestroyEvent, as the reference's synchronous lowering does
 * (GpuRuntimeToLlvm.cpp:619-622).  async != 0: launches are only enqueued;
 * the event of the last one is kept until nmhipContextSynchronize.
 */
void nmhipContextSetAsync(void *ctx, int async);
void nmhipContextSynchronize(void *ctx);

/* The gpux queue handle of the context (a numba::GPUQueueInterface*). */
void *nmhipContextQueue(void *ctx);

/* Name of the kernel chosen by the most recent op on this context. */
const char *nmhipLastKernelName(void *ctx);

/* ---- device memory ----------------------------------------------------- */

/* gpuxAlloc + gpuxWait + gpuxDestroyEvent (GpuRuntimeToLlvm.cpp:630-754). */
void *nmhipAlloc(void *ctx, size_t bytes, int gpuxAllocType);
void nmhipFree(void *ctx, void *dev);
/* Blocking host <-> device copies (counterpart of the USM copies dpctl
 * performs for the reference's device arrays), done without leaving the gpux
 * C-ABI: a pinned staging block from gpuxAlloc(Host) and a byte-copy kernel
 * launched with gpuxLaunchKernel. */
void nmhipMemcpyHtoD(void *ctx, void *dev, const void *host, size_t bytes);
void nmhipMemcpyDtoH(void *ctx, void *host, const void *dev, size_t bytes);

/* Device-to-device copy of a contiguous buffer on the context's queue (what
 * the compiler's force_copy of a contiguous operand lowers to,
 * numpy/funcs.py:759-764); bytes and pointers must be multiples of 16. */
void nmhipCopy(void *ctx, void *dst, const void *src, size_t bytes);

/* ---- elementwise / broadcast maps -------------------------------------- */

/*
 * out[i, j] = a[i, j] (op) b[i, j] over an [n0, n1] iteration space; a
 * broadcast dimension has stride 0 (NtensorToLinalg.cpp:487-557).  Rank-1
 * operands are passed as [1, n].  Replaces the kernel generated for
 * numpy.add/subtract/multiply (numpy/funcs.py:457-462, linalg_builder.py:297-325).
 */
void nmhipMapBinary(void *ctx, int op, int dtype, const void *a,
                    const int64_t aStrides[2], const void *b,
                    const int64_t bStrides[2], void *out,
                    const int64_t outStrides[2], int64_t n0, int64_t n1);

/*
 * Fused Black-Scholes over n options (tests/test_numpy.py:2827-2852).
 * wide != 0: literal-bearing intermediates in float64, the reference's
 * typing; wide == 0: float32 throughout.
 */
void nmhipBlackScholesF32(void *ctx, const float *price, const float *strike,
                          const float *t, float rate, float volatility,
                          float *call, float *put, int64_t n, int wide);

/* ---- reductions -------------------------------------------------------- */

/*
 * Reduces x[n0, n1] (strides s0, s1) with `op`.  axis = 0 or 1 writes n1 or
 * n0 contiguous results; axis = -1 reduces everything to out[0] (x must be
 * C-contiguous).  Integer input accumulates and stores int64; float output
 * has the input dtype (numpy/funcs.py:120-123, 163-229).
 */
void nmhipReduce(void *ctx, int op, int dtype, const void *x, int64_t n0,
                 int64_t n1, int64_t s0, int64_t s1, int axis, void *out);

/* out[r] = sqrt(sum_c x[r, c]^2) for a row-major float32 [n0, n1] array with
 * row stride s0: np.sqrt(np.square(a).sum(axis=1)) fused into one kernel. */
void nmhipNorm2RowsF32(void *ctx, const float *x, int64_t n0, int64_t n1,
                       int64_t s0, float *out);

/* out[0] = sqrt(sum(x * x)) over n contiguous float32. */
void nmhipNorm2F32(void *ctx, const float *x, int64_t n, float *out);

/* ---- matmul ------------------------------------------------------------ */

/*
 * np.dot of 2-D arrays: c = alpha * a @ b + beta * c through the registered
 * mkl_gemm_<dtype>_device (numpy/funcs.py:759-785).  dtype is NMHIP_F32 or
 * NMHIP_F64; shapes [m, k] @ [k, n]; strides in elements, one stride of each
 * operand must be 1.
 */
void nmhipGemm(void *ctx, int dtype, const void *a, const int64_t aStrides[2],
               const void *b, const int64_t bStrides[2], void *c,
               const int64_t cStrides[2], int64_t m, int64_t n, int64_t k,
               double alpha, double beta);

/* ---- @kernel launches -------------------------------------------------- */

/*
 * Block size the runtime suggests for `kernelName` over a global extent
 * (gpuxSuggestBlockSize; used when the user gives no local size,
 * LowerToGpu.cpp:373-471).
 */
void nmhipSuggestBlockSize(void *ctx, const char *kernelName,
                           const uint32_t *globalSize, uint32_t *blockSize,
                           size_t numDims);

/*
 * Launches a kernel of the built-in code objects by name with an explicit
 * grid (in blocks) and a gpux parameter array (terminated as in
 * gpuxLaunchKernel).
 */
void nmhipLaunch(void *ctx, const char *kernelName, const size_t grid[3],
                 const size_t block[3], GpuxParamDesc *params);

/*
 * Pairwise distance @kernel over global size (n1, n2) with the remapped
 * float64 twin (X1 [n1,3], X2 [n2,3], D [n1,n2], all C-contiguous, n2 even).
 */
void nmhipPairwiseF64(void *ctx, const double *X1, const double *X2, double *D,
                      int64_t n1, int64_t n2);

/* ---- code objects and tuning ------------------------------------------- */

/* The embedded gfx950 code object of a family: "maps", "reduce", "twins", or
 * "reduce_release" (the reduction kernels with the release / acquire hand-off
 * of partial results). */
const void *nmhipKernelBlob(const char *family, size_t *size);

/* Overrides a launch-shape knob ("rowbcast_rows", "map_blocks", "bs_blocks",
 * "reduce_blocks", "axis0_rows", "cols_blocks", "pairwise_rows"); 0 restores
 * the default.  "handoff_release" = 1 takes the reduction kernels from the
 * "reduce_release" code object instead of "reduce". */
void nmhipSetTuning(const char *knob, int64_t value);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* NUMBA_MLIR_HIP_OFFLOAD_H */
