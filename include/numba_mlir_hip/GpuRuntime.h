/*
 * C-ABI of the MI355X (HIP) GPU runtime for numba-mlir.
 *
 * libnumba-mlir-gpu-runtime-hip.so exports exactly the thirteen gpux* entry
 * points below and nothing else (see csrc/runtime/export.map).  They are the
 * functions the numba-mlir compiler emits calls to
 * (reference: mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:95-194) and that the
 * SYCL runtime implements (reference:
 * numba_mlir_gpu_runtime_sycl/lib/GpuRuntime.cpp:361-463).  The wire structs
 * have the layout of numba_mlir_gpu_common/GpuCommon.hpp:30-64.
 *
 * Error convention (reference: numba_mlir_gpu_runtime_sycl/lib/Utils.hpp:8-21):
 * no return codes; any failure prints a message to stdout and calls abort().
 *
 * Environment (reference: GpuRuntime.cpp:29-59):
 *   NUMBA_MLIR_LOG_GPU_RUNTIME_CALLS=1  prints "<fn> enter"/"<fn> exit" on stdout
 *   NUMBA_MLIR_DUMP_KERNEL_BLOB=1       writes each loaded blob to
 *                                       ./kernel_dump_<unix-ms>
 */
#ifndef NUMBA_MLIR_HIP_GPU_RUNTIME_H
#define NUMBA_MLIR_HIP_GPU_RUNTIME_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GpuCommon.hpp:30 */
enum GpuxAllocType {
  GPUX_ALLOC_DEVICE = 0, /* hipMalloc: HBM, not host-dereferenceable        */
  GPUX_ALLOC_SHARED = 1, /* host-dereferenceable and device-accessible      */
  GPUX_ALLOC_LOCAL = 2,  /* LDS: returns ptr == NULL, sized at launch       */
  GPUX_ALLOC_HOST = 3    /* pinned host memory, device-accessible           */
};

/* GpuCommon.hpp:32-42 */
enum GpuxParamType {
  GPUX_PARAM_NULL = 0,
  GPUX_PARAM_BOOL = 1,
  GPUX_PARAM_INT8 = 2,
  GPUX_PARAM_INT16 = 3,
  GPUX_PARAM_INT32 = 4,
  GPUX_PARAM_INT64 = 5,
  GPUX_PARAM_FLOAT32 = 6,
  GPUX_PARAM_FLOAT64 = 7,
  GPUX_PARAM_PTR = 8
};

/*
 * GpuCommon.hpp:45-55; the compiler mirrors it as {ptr, i32, i32}
 * (GpuRuntimeToLlvm.cpp:87-89).  `data` points at a host slot holding the
 * VALUE of the argument (for GPUX_PARAM_PTR: a slot holding the device
 * pointer).  A GPUX_PARAM_PTR entry with data == NULL asks for `size` bytes of
 * workgroup (LDS) memory (GpuRuntimeToLlvm.cpp:507-536).
 *
 * HIP convention for LDS entries: the kernel receives, in that argument
 * position, a uint64_t holding the byte offset of the buffer inside the
 * kernel's dynamic LDS block (`extern __shared__`); offsets are 16-byte
 * aligned and the sum becomes the launch's dynamic LDS size.
 */
typedef struct GpuxParamDesc {
  const void *data;
  int32_t size;
  int32_t type; /* enum GpuxParamType */
} GpuxParamDesc;

/* GpuCommon.hpp:61-64 */
typedef struct GpuxAllocResult {
  void *ptr;
  void *event;
} GpuxAllocResult;

/*
 * Queue.  `deviceName` may be NULL.  Accepted: NULL, "", "gpu", "hip",
 * "<backend>:gpu", "<backend>:gpu:<n>", "<backend>:<n>" (SYCL filter-string
 * shapes used by the callers, e.g. "level_zero:gpu:0"); <n> selects the HIP
 * device ordinal.  Anything else is fatal.  The returned pointer is a
 * numba::GPUQueueInterface* (see GpuQueueInterface.hpp).  The queue is
 * reference counted: +1 here, +1 per live event, +1 per live allocation;
 * gpuxQueueDestroy drops the creator's reference only
 * (GpuRuntime.cpp:134-139, 248-251, 287-299).
 */
void *gpuxQueueCreate(const char *deviceName);     /* GpuRuntime.cpp:361-365 */
void gpuxQueueDestroy(void *queue);                /* GpuRuntime.cpp:367-371 */

/*
 * Module / kernel.  `data` is a gfx950 code object (ELF or clang offload
 * bundle) of `size` bytes; one blob may hold many kernels.
 */
void *gpuxModuleLoad(void *queue, const void *data, size_t size); /* :373-377 */
void gpuxModuleDestroy(void *module);                             /* :379-383 */
void *gpuxKernelGet(void *module, const char *name);              /* :385-391 */
void gpuxKernelDestroy(void *kernel);                             /* :393-397 */

/*
 * Launch gridX*gridY*gridZ blocks of blockX*blockY*blockZ threads (X fastest,
 * GpuRuntime.cpp:184-187).  `depEvents` is a NULL-terminated array of events
 * the launch must wait for; `params` is terminated by {NULL, 0,
 * GPUX_PARAM_NULL}.  Returns a pooled event the caller passes to gpuxWait and
 * then gpuxDestroyEvent.  The launch is asynchronous.  A launch with any
 * zero dimension is a no-op that returns a completed event.
 */
void *gpuxLaunchKernel(void *queue, void *kernel, size_t gridX, size_t gridY,
                       size_t gridZ, size_t blockX, size_t blockY,
                       size_t blockZ, void *depEvents,
                       void *params);                       /* :399-410 */
void gpuxWait(void *queue, void *event);                    /* :412-417 */
void gpuxDestroyEvent(void *queue, void *event);            /* :419-425 */

/*
 * Allocation (GpuRuntime.cpp:215-260, 427-443).  Waits for `depEvents` first,
 * then allocates `size` bytes with at least `alignment` alignment (power of
 * two, <= 256 honoured).  `type` is enum GpuxAllocType; an unknown type is
 * fatal.  LOCAL returns ptr == NULL.  The result event is already complete.
 * gpuxDeAlloc(queue, NULL) is legal and balances a LOCAL allocation.  DeAlloc
 * may be called from any thread, after gpuxQueueDestroy.
 */
void gpuxAlloc(void *queue, size_t size, size_t alignment, int type,
               void *depEvents, GpuxAllocResult *result);
void gpuxDeAlloc(void *queue, void *ptr);

/*
 * Block-size suggestion (GpuRuntime.cpp:445-453, GpuModule.cpp:453-509).
 * `gridSize` holds the GLOBAL extent (work-items, not blocks) of each of the
 * numDims (1..3) dimensions; writes the suggested block extent per dimension:
 *   maxWg = largest power of two <= the kernel's preferred workgroup size;
 *   for each dim in order: l = g > 1 ? min(g, maxWg) : 1; maxWg /= upPow2(l).
 * The caller launches ceil(g/l) blocks per dim and guards the tail in-kernel.
 */
void gpuxSuggestBlockSize(void *queue, void *kernel, const uint32_t *gridSize,
                          uint32_t *blockSize, size_t numDims);

/*
 * Duplicates a raw native queue handle (GpuRuntime.cpp:455-463; used by the
 * parfor-replacement glue only).  Here the native handle is a hipStream_t
 * boxed as `hipStream_t*`; the copy shares the stream and is released with
 * free().
 */
void *gpuxDuplicateQueue(void *rawNativeQueue);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* NUMBA_MLIR_HIP_GPU_RUNTIME_H */
