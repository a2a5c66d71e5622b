// Binds the runtime's HIP table to libamdhip64.  There is no other binding in
// the shipped library: without a working HIP installation every entry point
// fails loudly (message on stdout + abort()).
#include "HipApi.hpp"

namespace nmhip {

const HipApi &hipApi() {
  static const HipApi api = {
      &hipGetDeviceCount,
      &hipSetDevice,
      &hipStreamCreateWithFlags,
      &hipStreamDestroy,
      &hipStreamWaitEvent,
      &hipStreamSynchronize,
      &hipEventCreateWithFlags,
      &hipEventDestroy,
      &hipEventRecord,
      &hipEventSynchronize,
      &hipMalloc,
      [](void **p, size_t n, unsigned f) { return hipMallocManaged(p, n, f); },
      [](void **p, size_t n, unsigned f) { return hipHostMalloc(p, n, f); },
      &hipFree,
      &hipHostFree,
      &hipModuleLoadData,
      &hipModuleUnload,
      &hipModuleGetFunction,
      &hipFuncGetAttribute,
      &hipModuleLaunchKernel,
      &hipGetErrorString,
  };
  return api;
}

} // namespace nmhip
