// Recording stand-in for the HIP entry points of the gpux runtime, for
// host-only unit tests.  Linked with the runtime's own sources into
// tests/host/_build/libgpux-mock.so; never part of the shipped libraries.
#include "HipApi.hpp"

#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>

namespace {

struct LaunchRecord {
  unsigned grid[3];
  unsigned block[3];
  unsigned sharedBytes;
  void *stream;
  void *function;
  int numParams;
  uint64_t params[32];    // first 8 bytes behind every kernelParams[i]
  void *paramPtrs[32];
};

struct State {
  std::mutex mutex;
  int deviceCount = 2;
  int currentDevice = -1;
  long streamsCreated = 0, streamsDestroyed = 0;
  long eventsCreated = 0, eventsDestroyed = 0;
  long eventRecords = 0, eventSyncs = 0, streamWaits = 0, streamSyncs = 0;
  long launches = 0;
  long modulesLoaded = 0, modulesUnloaded = 0;
  int expectParams = 0;
  LaunchRecord last{};
  std::unordered_map<void *, int> allocs; // ptr -> 0 device, 1 managed, 2 host
  long freesDevice = 0, freesHost = 0, mallocsDevice = 0;
  uintptr_t nextHandle = 0x1000;
  std::unordered_map<void *, std::string> functionNames;
};

State &st() {
  static State s;
  return s;
}

void *newHandle() {
  st().nextHandle += 0x10;
  return reinterpret_cast<void *>(st().nextHandle);
}

hipError_t mGetDeviceCount(int *n) {
  *n = st().deviceCount;
  return hipSuccess;
}
hipError_t mSetDevice(int d) {
  std::lock_guard<std::mutex> l(st().mutex);
  if (d < 0 || d >= st().deviceCount)
    return hipErrorInvalidDevice;
  st().currentDevice = d;
  return hipSuccess;
}
hipError_t mStreamCreate(hipStream_t *s, unsigned) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().streamsCreated;
  *s = static_cast<hipStream_t>(newHandle());
  return hipSuccess;
}
hipError_t mStreamDestroy(hipStream_t) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().streamsDestroyed;
  return hipSuccess;
}
hipError_t mStreamWaitEvent(hipStream_t, hipEvent_t, unsigned) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().streamWaits;
  return hipSuccess;
}
hipError_t mStreamSync(hipStream_t) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().streamSyncs;
  return hipSuccess;
}
hipError_t mEventCreate(hipEvent_t *e, unsigned) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().eventsCreated;
  *e = static_cast<hipEvent_t>(newHandle());
  return hipSuccess;
}
hipError_t mEventDestroy(hipEvent_t) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().eventsDestroyed;
  return hipSuccess;
}
hipError_t mEventRecord(hipEvent_t, hipStream_t) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().eventRecords;
  return hipSuccess;
}
hipError_t mEventSync(hipEvent_t) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().eventSyncs;
  return hipSuccess;
}
hipError_t allocKind(void **p, size_t n, int kind) {
  void *mem = std::aligned_alloc(256, (n + 255) / 256 * 256);
  if (!mem)
    return hipErrorOutOfMemory;
  std::lock_guard<std::mutex> l(st().mutex);
  st().allocs[mem] = kind;
  *p = mem;
  return hipSuccess;
}
hipError_t mMalloc(void **p, size_t n) {
  st().mallocsDevice++;
  return allocKind(p, n, 0);
}
hipError_t mMallocManaged(void **p, size_t n, unsigned) {
  return allocKind(p, n, 1);
}
hipError_t mHostMalloc(void **p, size_t n, unsigned) {
  return allocKind(p, n, 2);
}
hipError_t freeKind(void *p, bool host) {
  std::lock_guard<std::mutex> l(st().mutex);
  auto it = st().allocs.find(p);
  if (it == st().allocs.end() || (it->second == 2) != host)
    return hipErrorInvalidValue;
  st().allocs.erase(it);
  (host ? st().freesHost : st().freesDevice)++;
  std::free(p);
  return hipSuccess;
}
hipError_t mFree(void *p) { return freeKind(p, false); }
hipError_t mHostFree(void *p) { return freeKind(p, true); }
hipError_t mModuleLoadData(hipModule_t *m, const void *) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().modulesLoaded;
  *m = static_cast<hipModule_t>(newHandle());
  return hipSuccess;
}
hipError_t mModuleUnload(hipModule_t) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().modulesUnloaded;
  return hipSuccess;
}
hipError_t mModuleGetFunction(hipFunction_t *f, hipModule_t, const char *name) {
  if (std::strcmp(name, "missing") == 0)
    return hipErrorNotFound;
  std::lock_guard<std::mutex> l(st().mutex);
  void *h = newHandle();
  st().functionNames[h] = name;
  *f = static_cast<hipFunction_t>(h);
  return hipSuccess;
}
hipError_t mFuncGetAttribute(int *v, hipFunction_attribute, hipFunction_t f) {
  std::lock_guard<std::mutex> l(st().mutex);
  const std::string &name = st().functionNames[f];
  // "<anything>_wg<N>" declares a launch bound of N threads.
  auto pos = name.rfind("_wg");
  *v = pos == std::string::npos ? 1024 : std::atoi(name.c_str() + pos + 3);
  return hipSuccess;
}
hipError_t mLaunch(hipFunction_t f, unsigned gx, unsigned gy, unsigned gz,
                   unsigned bx, unsigned by, unsigned bz, unsigned shared,
                   hipStream_t stream, void **params, void **) {
  std::lock_guard<std::mutex> l(st().mutex);
  ++st().launches;
  LaunchRecord &r = st().last;
  r.grid[0] = gx, r.grid[1] = gy, r.grid[2] = gz;
  r.block[0] = bx, r.block[1] = by, r.block[2] = bz;
  r.sharedBytes = shared;
  r.stream = stream;
  r.function = f;
  r.numParams = st().expectParams;
  for (int i = 0; i < r.numParams && i < 32; ++i) {
    r.paramPtrs[i] = params[i];
    std::memcpy(&r.params[i], params[i], 8);
  }
  return hipSuccess;
}
const char *mErrorString(hipError_t e) {
  return e == hipErrorNotFound ? "named symbol not found" : "mock hip error";
}

} // namespace

namespace nmhip {
const HipApi &hipApi() {
  static const HipApi api = {
      mGetDeviceCount, mSetDevice,     mStreamCreate,      mStreamDestroy,
      mStreamWaitEvent, mStreamSync,   mEventCreate,       mEventDestroy,
      mEventRecord,    mEventSync,     mMalloc,            mMallocManaged,
      mHostMalloc,     mFree,          mHostFree,          mModuleLoadData,
      mModuleUnload,   mModuleGetFunction, mFuncGetAttribute, mLaunch,
      mErrorString,
  };
  return api;
}
} // namespace nmhip

#define MOCK_EXPORT extern "C" __attribute__((visibility("default")))

MOCK_EXPORT void mockExpectParams(int n) { st().expectParams = n; }
MOCK_EXPORT long mockCounter(const char *name) {
  std::lock_guard<std::mutex> l(st().mutex);
  const std::string n(name);
  State &s = st();
  if (n == "streams_live") return s.streamsCreated - s.streamsDestroyed;
  if (n == "streams_created") return s.streamsCreated;
  if (n == "events_live") return s.eventsCreated - s.eventsDestroyed;
  if (n == "events_created") return s.eventsCreated;
  if (n == "event_records") return s.eventRecords;
  if (n == "event_syncs") return s.eventSyncs;
  if (n == "stream_waits") return s.streamWaits;
  if (n == "stream_syncs") return s.streamSyncs;
  if (n == "launches") return s.launches;
  if (n == "allocs_live") return long(s.allocs.size());
  if (n == "frees_device") return s.freesDevice;
  if (n == "mallocs_device") return s.mallocsDevice;
  if (n == "frees_host") return s.freesHost;
  if (n == "modules_live") return s.modulesLoaded - s.modulesUnloaded;
  if (n == "current_device") return s.currentDevice;
  return -1;
}
MOCK_EXPORT void mockLastLaunch(unsigned *grid, unsigned *block,
                                unsigned *shared, uint64_t *params,
                                void **paramPtrs, void **stream) {
  std::lock_guard<std::mutex> l(st().mutex);
  const LaunchRecord &r = st().last;
  std::memcpy(grid, r.grid, sizeof(r.grid));
  std::memcpy(block, r.block, sizeof(r.block));
  *shared = r.sharedBytes;
  std::memcpy(params, r.params, sizeof(uint64_t) * r.numParams);
  std::memcpy(paramPtrs, r.paramPtrs, sizeof(void *) * r.numParams);
  *stream = r.stream;
}
