// Stopwatch for bench.py: a pair of HIP events recorded on the stream of a
// gpux queue, so that the measured interval is exactly what the kernels
// launched through gpuxLaunchKernel between start and stop took on the GPU.
// Not part of the offloaded path: nothing but the benchmark loads this.
#include "numba_mlir_hip/GpuQueueInterface.hpp"

#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>

namespace {

struct Timer {
  hipStream_t stream;
  int device;
  hipEvent_t start, stop;
};

void check(hipError_t err, const char *what) {
  if (err == hipSuccess)
    return;
  std::fprintf(stdout, "bench timer: %s failed: %s\n", what, hipGetErrorString(err));
  std::fflush(stdout);
  std::abort();
}

} // namespace

#define TIMER_EXPORT extern "C" __attribute__((visibility("default")))

// `queue` is the handle gpuxQueueCreate returned.
TIMER_EXPORT void *benchTimerCreate(void *queue) {
  auto *base = static_cast<numba::GPUQueueInterface *>(queue);
  auto *q = static_cast<numba::HipQueueInterface *>(base);
  if (!q || q->hipMagic() != numba::HipQueueInterface::kMagic) {
    std::fprintf(stdout, "bench timer: not a queue of the HIP GPU runtime\n");
    std::abort();
  }
  auto *t = new Timer{static_cast<hipStream_t>(q->hipStream()), q->hipDevice(),
                      nullptr, nullptr};
  check(hipSetDevice(t->device), "hipSetDevice");
  check(hipEventCreate(&t->start), "hipEventCreate");
  check(hipEventCreate(&t->stop), "hipEventCreate");
  return t;
}

TIMER_EXPORT void benchTimerStart(void *timer) {
  auto *t = static_cast<Timer *>(timer);
  check(hipEventRecord(t->start, t->stream), "hipEventRecord");
}

TIMER_EXPORT void benchTimerStop(void *timer) {
  auto *t = static_cast<Timer *>(timer);
  check(hipEventRecord(t->stop, t->stream), "hipEventRecord");
}

// Waits for the stop event.
TIMER_EXPORT double benchTimerElapsedMs(void *timer) {
  auto *t = static_cast<Timer *>(timer);
  check(hipEventSynchronize(t->stop), "hipEventSynchronize");
  float ms = 0.f;
  check(hipEventElapsedTime(&ms, t->start, t->stop), "hipEventElapsedTime");
  return ms;
}

TIMER_EXPORT void benchTimerDestroy(void *timer) {
  auto *t = static_cast<Timer *>(timer);
  if (!t)
    return;
  (void)hipEventDestroy(t->start);
  (void)hipEventDestroy(t->stop);
  delete t;
}
