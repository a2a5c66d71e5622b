// Thin table of the HIP driver entry points the gpux runtime uses.
//
// The runtime never calls HIP directly; it goes through hipApi().  The shipped
// library binds the table to libamdhip64 (HipApiReal.cpp).  The host-only unit
// tests link the same runtime sources against a recording table so argument
// marshalling, reference counting and error paths can be checked without a
// GPU (the reference reaches its own backends through dlopen'd loader tables
// in the same way: numba_mlir_gpu_runtime_sycl/lib/GpuModule.cpp:35-132).
#pragma once

#include <hip/hip_runtime_api.h>

namespace nmhip {

struct HipApi {
  hipError_t (*getDeviceCount)(int *);
  hipError_t (*setDevice)(int);
  hipError_t (*streamCreateWithFlags)(hipStream_t *, unsigned);
  hipError_t (*streamDestroy)(hipStream_t);
  hipError_t (*streamWaitEvent)(hipStream_t, hipEvent_t, unsigned);
  hipError_t (*streamSynchronize)(hipStream_t);
  hipError_t (*eventCreateWithFlags)(hipEvent_t *, unsigned);
  hipError_t (*eventDestroy)(hipEvent_t);
  hipError_t (*eventRecord)(hipEvent_t, hipStream_t);
  hipError_t (*eventSynchronize)(hipEvent_t);
  hipError_t (*malloc_)(void **, size_t);
  hipError_t (*mallocManaged)(void **, size_t, unsigned);
  hipError_t (*hostMalloc)(void **, size_t, unsigned);
  hipError_t (*free_)(void *);
  hipError_t (*hostFree)(void *);
  hipError_t (*moduleLoadData)(hipModule_t *, const void *);
  hipError_t (*moduleUnload)(hipModule_t);
  hipError_t (*moduleGetFunction)(hipFunction_t *, hipModule_t, const char *);
  hipError_t (*funcGetAttribute)(int *, hipFunction_attribute, hipFunction_t);
  hipError_t (*moduleLaunchKernel)(hipFunction_t, unsigned, unsigned, unsigned,
                                   unsigned, unsigned, unsigned, unsigned,
                                   hipStream_t, void **, void **);
  const char *(*getErrorString)(hipError_t);
};

/// The table in use.  Defined once per link: HipApiReal.cpp for the product,
/// the recording table for host-only tests.
const HipApi &hipApi();

} // namespace nmhip
