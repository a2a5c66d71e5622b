// The object behind the opaque `queue` pointer of the gpux* C-ABI.
//
// Companion libraries (the math runtime's mkl_gemm_*_device) receive the queue
// as `void*` and cast it to numba::GPUQueueInterface*
// (reference: numba_mlir/numba_mlir/math_runtime/sycl/lib/NumpyLinalg.cpp:71),
// so the first base of the HIP queue keeps the virtual-table layout of
// numba_mlir_gpu_common/GpuCommon.hpp:18-28: destructor, getDeviceName(),
// getQueue().  getQueue() answers nullptr ("queue is not available",
// GpuCommon.hpp:25-27) because there is no SYCL queue; HIP-aware companions
// use the extension slots of numba::HipQueueInterface instead.
#pragma once

#include <cstdint>
#include <string_view>

namespace sycl {
inline namespace _V1 {
class queue;
}
} // namespace sycl

namespace numba {

class GPUQueueInterface {
public:
  virtual ~GPUQueueInterface() = default;

  /// Device string the queue was created with ("" when NULL was passed).
  virtual std::string_view getDeviceName() = 0;

  /// Always nullptr for the HIP runtime.
  virtual sycl::queue *getQueue() = 0;
};

/// Extension implemented by every queue created by
/// libnumba-mlir-gpu-runtime-hip.so.  New slots are only ever appended.
class HipQueueInterface : public GPUQueueInterface {
public:
  static constexpr uint64_t kMagic = 0x4e4d484950513031ull; // "NMHIPQ01"

  /// Returns kMagic; lets a companion library reject a foreign queue object.
  virtual uint64_t hipMagic() = 0;

  /// The hipStream_t every launch of this queue is enqueued on.
  virtual void *hipStream() = 0;

  /// HIP device ordinal of the queue.
  virtual int hipDevice() = 0;

  /// Keeps the queue alive (same counter gpuxQueueCreate/Destroy use).
  virtual void hipRetain() = 0;
  virtual void hipRelease() = 0;
};

} // namespace numba
