// HIP implementation of the gpux* C-ABI (include/numba_mlir_hip/GpuRuntime.h).
//
// Behavioural contract taken from the SYCL runtime it replaces
// (reference: numba_mlir_gpu_runtime_sycl/lib/GpuRuntime.cpp:121-463,
// GpuModule.cpp:322-509, Utils.hpp:8-21); the implementation is HIP-native:
// one non-blocking hipStream_t per queue, pooled hipEvent_t objects, code
// objects loaded with hipModuleLoadData, launches through
// hipModuleLaunchKernel with the caller's value slots used directly as the
// kernel-parameter array.
#include "HipApi.hpp"

#include "numba_mlir_hip/GpuQueueInterface.hpp"
#include "numba_mlir_hip/GpuRuntime.h"

#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

using nmhip::hipApi;

namespace {

bool envFlag(const char *name) {
  const char *env = std::getenv(name);
  return env && std::atoi(env) != 0;
}

bool isLogFunctionsEnabled() {
  static bool enable = envFlag("NUMBA_MLIR_LOG_GPU_RUNTIME_CALLS");
  return enable;
}

bool isKernelDumpEnabled() {
  static bool enable = envFlag("NUMBA_MLIR_DUMP_KERNEL_BLOB");
  return enable;
}

// "<fn> enter" / "<fn> exit" on stdout, flushed (GpuRuntime.cpp:61-80).
struct CallLog {
  explicit CallLog(const char *fn) : name(fn), on(isLogFunctionsEnabled()) {
    if (on) {
      std::fprintf(stdout, "%s enter\n", name);
      std::fflush(stdout);
    }
  }
  CallLog(const CallLog &) = delete;
  ~CallLog() {
    if (on) {
      std::fprintf(stdout, "%s exit\n", name);
      std::fflush(stdout);
    }
  }
  const char *name;
  bool on;
};

[[noreturn]] void fail(const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  throw std::runtime_error(buf);
}

void check(hipError_t err, const char *what) {
  if (err != hipSuccess)
    fail("%s failed: %s (%d)", what, hipApi().getErrorString(err),
         static_cast<int>(err));
}

// Any failure: message on stdout, then abort() (Utils.hpp:8-21).
template <typename F> auto guarded(F &&body) noexcept {
  try {
    return body();
  } catch (const std::exception &e) {
    std::fprintf(stdout, "An exception was thrown: %s\n", e.what());
    std::fflush(stdout);
    std::abort();
  } catch (...) {
    std::fprintf(stdout, "An unknown exception was thrown\n");
    std::fflush(stdout);
    std::abort();
  }
}

void dumpKernelBlob(const void *data, size_t size) {
  if (!isKernelDumpEnabled())
    return;
  using namespace std::chrono;
  auto ms = duration_cast<milliseconds>(system_clock::now().time_since_epoch())
                .count();
  std::ofstream file("kernel_dump_" + std::to_string(ms),
                     std::ios::binary | std::ios::trunc);
  file.write(static_cast<const char *>(data),
             static_cast<std::streamsize>(size));
}

uint32_t downPow2(uint32_t x) {
  uint32_t r = 1;
  while ((r << 1) != 0 && (r << 1) <= x)
    r <<= 1;
  return r;
}

uint32_t upPow2(uint32_t x) {
  uint32_t r = 1;
  while (r < x && (r << 1) != 0)
    r <<= 1;
  return r;
}

bool isNumber(const std::string &s) {
  if (s.empty())
    return false;
  for (char c : s)
    if (c < '0' || c > '9')
      return false;
  return true;
}

// Device strings are SYCL filter strings, "backend:device_type:device_num"
// with every part optional (callers use "level_zero:gpu:0", "opencl:gpu:0",
// "gpu", ""; reference: numba_mlir/numba_mlir/mlir/dpctl_interop.py:293-306).
// Only the ordinal matters here; a non-GPU device type or an unknown token
// is an error.
int parseDeviceOrdinal(const std::string &name) {
  static const char *const backends[] = {"hip",    "level_zero", "opencl",
                                         "cuda",   "ext_oneapi_level_zero",
                                         "ext_oneapi_hip", "*"};
  int ordinal = 0;
  bool haveOrdinal = false;
  size_t pos = 0;
  int index = 0;
  while (pos <= name.size() && !name.empty()) {
    size_t end = name.find(':', pos);
    if (end == std::string::npos)
      end = name.size();
    std::string tok = name.substr(pos, end - pos);
    bool known = false;
    if (isNumber(tok)) {
      if (haveOrdinal)
        fail("Invalid device name '%s': two device numbers", name.c_str());
      ordinal = std::atoi(tok.c_str());
      haveOrdinal = true;
      known = true;
    } else if (tok == "gpu" || tok == "*") {
      known = true;
    } else if (tok == "cpu" || tok == "acc" || tok == "accelerator" ||
               tok == "host") {
      fail("Failed to find device matching name '%s': the HIP runtime only "
           "drives GPU devices",
           name.c_str());
    } else if (index == 0) {
      for (const char *b : backends)
        known = known || tok == b;
    }
    if (!known)
      fail("Failed to find device matching name '%s': unknown token '%s'",
           name.c_str(), tok.c_str());
    ++index;
    if (end == name.size())
      break;
    pos = end + 1;
  }
  return ordinal;
}

class Queue;

// What gpuxLaunchKernel / gpuxAlloc hand out.  A queue is one in-order
// stream, so an event is just a position in that stream: the ticket of the
// launch it follows.  Nothing is recorded on the device for it -- a marker
// packet after every kernel costs several microseconds of idle GPU between
// back-to-back launches -- until another queue has to wait for it, which
// records a real hipEvent_t at the stream's current tail (a later, hence
// sufficient, position).
struct Event {
  Queue *owner = nullptr;
  uint64_t ticket = 0;          // launches enqueued on owner up to this one
  hipEvent_t event = nullptr;   // created on first cross-queue use, then kept
  bool recorded = false;        // event holds a record covering `ticket`
  Event *next = nullptr;
};

// Kind, size and device of every live pointer handed out by gpuxAlloc, so
// gpuxDeAlloc can pick hipFree or hipHostFree.  DeAlloc may arrive from any
// thread.
struct AllocInfo {
  int kind = -1;
  size_t bytes = 0;
  int device = 0;
};

struct AllocRegistry {
  std::mutex mutex;
  std::unordered_map<void *, AllocInfo> live;

  void add(void *ptr, AllocInfo info) {
    std::lock_guard<std::mutex> lock(mutex);
    live[ptr] = info;
  }
  AllocInfo take(void *ptr) {
    std::lock_guard<std::mutex> lock(mutex);
    auto it = live.find(ptr);
    if (it == live.end())
      return AllocInfo();
    AllocInfo info = it->second;
    live.erase(it);
    return info;
  }
};

AllocRegistry &allocRegistry() {
  static AllocRegistry *reg = new AllocRegistry; // outlives late DeAllocs
  return *reg;
}

// Device blocks given back by gpuxDeAlloc are kept for the next gpuxAlloc of
// the same size on the same device: hipMalloc / hipFree of the arrays a
// compiled function returns cost several kernel times each (hipFree also
// synchronises the device, which the cache does not).  A kept block therefore
// goes back only to the queue that released it -- work of that queue which
// may still touch the block is ahead of any new use on the same in-order
// stream -- or to any queue once the releasing queue's stream has been
// drained and destroyed.  Blocks below 64 KiB are not worth keeping; the
// total kept is capped (NUMBA_MLIR_GPU_ALLOC_CACHE_MB, default 16384, 0 =
// off) and everything is released when an allocation fails.
class DeviceBlockCache {
public:
  static constexpr size_t kMinBytes = 64 * 1024;

  // A block of `bytes` on `device` that `stream` may use at once.
  void *take(int device, size_t bytes, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(mutex);
    auto it = blocks.find(key(device, bytes));
    if (it == blocks.end())
      return nullptr;
    std::vector<Block> &kept_ = it->second;
    for (size_t k = kept_.size(); k-- > 0;) {
      if (kept_[k].stream != stream && kept_[k].stream != nullptr)
        continue;
      void *ptr = kept_[k].ptr;
      kept_.erase(kept_.begin() + long(k));
      kept -= bytes;
      return ptr;
    }
    return nullptr;
  }

  // False when the block should be freed for real.
  bool put(int device, void *ptr, size_t bytes, hipStream_t stream) {
    if (bytes < kMinBytes)
      return false;
    std::lock_guard<std::mutex> lock(mutex);
    if (kept + bytes > limit())
      return false;
    blocks[key(device, bytes)].push_back(Block{ptr, stream});
    kept += bytes;
    return true;
  }

  // `stream` has finished all its work and is gone: what it released is
  // anybody's.
  void streamRetired(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(mutex);
    for (auto &entry : blocks)
      for (Block &b : entry.second)
        if (b.stream == stream)
          b.stream = nullptr;
  }

  // Hands every kept block of `device` to `release`.
  template <typename F> void flush(int device, F release) {
    std::vector<void *> all;
    {
      std::lock_guard<std::mutex> lock(mutex);
      for (auto &entry : blocks) {
        if (int(entry.first >> 48) != device)
          continue;
        kept -= (entry.first & ((uint64_t(1) << 48) - 1)) * entry.second.size();
        for (const Block &b : entry.second)
          all.push_back(b.ptr);
        entry.second.clear();
      }
    }
    for (void *ptr : all)
      release(ptr);
  }

private:
  struct Block {
    void *ptr;
    hipStream_t stream; // the releasing queue's; nullptr: idle for everybody
  };
  static uint64_t key(int device, size_t bytes) {
    return (uint64_t(device) << 48) | uint64_t(bytes);
  }
  static size_t limit() {
    static size_t value = [] {
      const char *env = std::getenv("NUMBA_MLIR_GPU_ALLOC_CACHE_MB");
      const long long mb = env ? std::atoll(env) : 16384;
      return size_t(mb > 0 ? mb : 0) << 20;
    }();
    return value;
  }
  std::mutex mutex;
  std::unordered_map<uint64_t, std::vector<Block>> blocks;
  size_t kept = 0;
};

DeviceBlockCache &deviceBlockCache() {
  static DeviceBlockCache *cache = new DeviceBlockCache; // never destroyed
  return *cache;
}

struct Kernel {
  hipFunction_t function = nullptr;
  int device = 0;
  uint32_t maxThreads = 0; // launch bound of the kernel
};

struct Module {
  hipModule_t module = nullptr;
  int device = 0;
};

class Queue final : public numba::HipQueueInterface {
public:
  explicit Queue(const char *devName) : deviceName(devName ? devName : "") {
    CallLog log("Queue");
    device = parseDeviceOrdinal(deviceName);
    int count = 0;
    check(hipApi().getDeviceCount(&count), "hipGetDeviceCount");
    if (device >= count)
      fail("Failed to find device matching name '%s': %d HIP device(s) present",
           deviceName.c_str(), count);
    makeCurrent();
    check(hipApi().streamCreateWithFlags(&stream, hipStreamNonBlocking),
          "hipStreamCreateWithFlags");
  }
  Queue(const Queue &) = delete;

  ~Queue() override {
    CallLog log("~Queue");
    // No exceptions from a destructor: report and continue.
    (void)hipApi().setDevice(device);
    while (freeList) {
      Event *ev = freeList;
      freeList = ev->next;
      if (ev->event)
        (void)hipApi().eventDestroy(ev->event);
      delete ev;
    }
    if (stream) {
      // Drained first: the blocks this queue released become anybody's.
      (void)hipApi().streamSynchronize(stream);
      (void)hipApi().streamDestroy(stream);
      deviceBlockCache().streamRetired(stream);
    }
  }

  std::string_view getDeviceName() override { return deviceName; }
  sycl::queue *getQueue() override { return nullptr; }
  uint64_t hipMagic() override { return kMagic; }
  void *hipStream() override { return stream; }
  int hipDevice() override { return device; }
  void hipRetain() override { retain(); }
  void hipRelease() override { release(); }

  void retain() { refs.fetch_add(1, std::memory_order_relaxed); }
  void release() {
    if (refs.fetch_sub(1, std::memory_order_acq_rel) == 1)
      delete this;
  }

  void makeCurrent() { check(hipApi().setDevice(device), "hipSetDevice"); }

  Module *loadModule(const void *data, size_t size) {
    if (!data)
      fail("Invalid module: null blob");
    dumpKernelBlob(data, size);
    static const char elfMagic[4] = {0x7f, 'E', 'L', 'F'};
    static const char bundleMagic[] = "__CLANG_OFFLOAD_BUNDLE__";
    const bool isElf = size >= 64 && std::memcmp(data, elfMagic, 4) == 0;
    const bool isBundle = size >= sizeof(bundleMagic) - 1 &&
                          std::memcmp(data, bundleMagic,
                                      sizeof(bundleMagic) - 1) == 0;
    if (!isElf && !isBundle)
      fail("Invalid module: %zu-byte blob is neither a gfx950 ELF code object "
           "nor a clang offload bundle",
           size);
    makeCurrent();
    auto mod = new Module;
    mod->device = device;
    hipError_t err = hipApi().moduleLoadData(&mod->module, data);
    if (err != hipSuccess) {
      delete mod;
      check(err, "hipModuleLoadData");
    }
    return mod;
  }

  Event *launch(Kernel *kernel, size_t gridX, size_t gridY, size_t gridZ,
                size_t blockX, size_t blockY, size_t blockZ, Event **deps,
                GpuxParamDesc *params) {
    if (!kernel)
      fail("Invalid kernel");
    if (!deps || !params)
      fail("gpuxLaunchKernel: deps and params must be terminated arrays");
    makeCurrent();
    waitOnStream(deps);

    size_t count = 0;
    while (!(params[count].data == nullptr && params[count].size == 0 &&
             params[count].type == GPUX_PARAM_NULL))
      ++count;

    std::vector<void *> args(count);
    std::vector<uint64_t> ldsOffsets(count);
    size_t ldsBytes = 0;
    for (size_t i = 0; i < count; ++i) {
      const GpuxParamDesc &p = params[i];
      size_t expect = 0;
      switch (p.type) {
      case GPUX_PARAM_BOOL:
      case GPUX_PARAM_INT8:
        expect = 1;
        break;
      case GPUX_PARAM_INT16:
        expect = 2;
        break;
      case GPUX_PARAM_INT32:
      case GPUX_PARAM_FLOAT32:
        expect = 4;
        break;
      case GPUX_PARAM_INT64:
      case GPUX_PARAM_FLOAT64:
        expect = 8;
        break;
      case GPUX_PARAM_PTR:
        break;
      default:
        std::fprintf(stdout, "Unhandled param type: %d\n", p.type);
        std::fflush(stdout);
        std::abort();
      }
      if (p.type == GPUX_PARAM_PTR) {
        if (p.data) {
          args[i] = const_cast<void *>(p.data);
        } else {
          if (p.size < 0)
            fail("Kernel param %zu: negative workgroup-memory size", i);
          ldsBytes = (ldsBytes + 15) & ~size_t(15);
          ldsOffsets[i] = ldsBytes;
          ldsBytes += static_cast<size_t>(p.size);
          args[i] = &ldsOffsets[i];
        }
      } else {
        if (!p.data || static_cast<size_t>(p.size) != expect)
          fail("Kernel param %zu: type %d needs a %zu-byte value, got %d", i,
               p.type, expect, p.size);
        args[i] = const_cast<void *>(p.data);
      }
    }

    Event *ev = getEvent();
    const bool empty = gridX == 0 || gridY == 0 || gridZ == 0 || blockX == 0 ||
                       blockY == 0 || blockZ == 0;
    if (!empty) {
      // HIP limits: x <= 2^31-1 blocks, y/z <= 65535 blocks, 1024 threads.
      if (gridX > 0x7fffffffull || gridY > 65535 || gridZ > 65535)
        fail("Launch grid (%zu, %zu, %zu) exceeds the HIP limits "
             "(2147483647, 65535, 65535)",
             gridX, gridY, gridZ);
      if (blockX * blockY * blockZ > 1024)
        fail("Launch block (%zu, %zu, %zu) exceeds 1024 threads", blockX,
             blockY, blockZ);
      // The dispatch packet counts the work-items of a dimension in 32 bits;
      // a larger product would wrap without an error from the launch call.
      if (gridX * blockX > 0xffffffffull || gridY * blockY > 0xffffffffull ||
          gridZ * blockZ > 0xffffffffull)
        fail("Launch of (%zu, %zu, %zu) blocks of (%zu, %zu, %zu) exceeds "
             "4294967295 work-items along a dimension",
             gridX, gridY, gridZ, blockX, blockY, blockZ);
      if (ldsBytes > 160 * 1024)
        fail("Launch needs %zu bytes of workgroup memory; gfx950 has 163840",
             ldsBytes);
      check(hipApi().moduleLaunchKernel(
                kernel->function, static_cast<unsigned>(gridX),
                static_cast<unsigned>(gridY), static_cast<unsigned>(gridZ),
                static_cast<unsigned>(blockX), static_cast<unsigned>(blockY),
                static_cast<unsigned>(blockZ), static_cast<unsigned>(ldsBytes),
                stream, args.data(), nullptr),
            "hipModuleLaunchKernel");
    }
    ev->ticket = enqueued.fetch_add(1, std::memory_order_acq_rel) + 1;
    return ev;
  }

  // Host wait.  Events of this queue are stream positions: if the position
  // is not known to be complete yet, drain the stream (which also completes
  // everything enqueued before the call) and remember how far that got.
  void waitHost(Event *ev) {
    if (!ev)
      fail("Invalid event");
    if (ev->owner != this) {
      ev->owner->waitHost(ev);
      return;
    }
    if (completed.load(std::memory_order_acquire) >= ev->ticket)
      return;
    const uint64_t upTo = enqueued.load(std::memory_order_acquire);
    makeCurrent();
    check(hipApi().streamSynchronize(stream), "hipStreamSynchronize");
    uint64_t seen = completed.load(std::memory_order_relaxed);
    while (seen < upTo && !completed.compare_exchange_weak(
                              seen, upTo, std::memory_order_release)) {
    }
  }

  void wait(Event *ev) { waitHost(ev); }

  void destroyEvent(Event *ev) {
    if (!ev)
      fail("Invalid event");
    {
      std::lock_guard<std::mutex> lock(poolMutex);
      ev->next = freeList;
      freeList = ev;
    }
    release(); // taken in getEvent()
  }

  std::pair<void *, Event *> alloc(size_t size, size_t alignment, int type,
                                   Event **deps) {
    if (!deps)
      fail("gpuxAlloc: deps must be a NULL-terminated array");
    // Allocation is synchronous: wait for the dependencies on the host
    // (GpuRuntime.cpp:218-224).
    for (Event **d = deps; *d; ++d)
      waitHost(*d);
    if (alignment > 256 && type != GPUX_ALLOC_LOCAL)
      fail("gpuxAlloc: alignment %zu above the 256 bytes HIP guarantees",
           alignment);

    makeCurrent();
    void *ptr = nullptr;
    // device blocks come in multiples of 256 bytes, so equal requests match
    const size_t bytes =
        type == GPUX_ALLOC_DEVICE ? ((size ? size : 1) + 255) / 256 * 256
                                  : (size ? size : 1);
    switch (type) {
    case GPUX_ALLOC_DEVICE:
      ptr = deviceBlockCache().take(device, bytes, stream);
      if (!ptr && (hipApi().malloc_(&ptr, bytes) != hipSuccess || !ptr)) {
        // give back what is kept and try once more
        ptr = nullptr;
        deviceBlockCache().flush(device, [](void *p) { (void)hipApi().free_(p); });
        if (hipApi().malloc_(&ptr, bytes) != hipSuccess || !ptr)
          fail("Failed to allocate device memory");
      }
      break;
    case GPUX_ALLOC_SHARED:
      if (hipApi().mallocManaged(&ptr, bytes, hipMemAttachGlobal) !=
              hipSuccess ||
          !ptr)
        fail("Failed to allocate shared memory");
      break;
    case GPUX_ALLOC_LOCAL:
      break; // sized at launch; no host-side pointer (GpuRuntime.cpp:236-238)
    case GPUX_ALLOC_HOST:
      if (hipApi().hostMalloc(&ptr, bytes, hipHostMallocDefault) !=
              hipSuccess ||
          !ptr)
        fail("Failed to allocate host memory");
      break;
    default:
      fail("Invalid allocation type");
    }
    if (ptr)
      allocRegistry().add(ptr, AllocInfo{type, bytes, device});

    // The allocation is synchronous, so its event is complete already
    // (position 0), as the reference's default-constructed event is
    // (GpuRuntime.cpp:226, 251).
    Event *ev = getEvent();
    ev->ticket = 0;
    retain(); // until gpuxDeAlloc (GpuRuntime.cpp:248-251)
    return {ptr, ev};
  }

  void dealloc(void *ptr) {
    if (ptr) {
      const AllocInfo info = allocRegistry().take(ptr);
      if (info.kind < 0)
        fail("gpuxDeAlloc: pointer %p was not allocated by gpuxAlloc", ptr);
      makeCurrent();
      if (info.kind == GPUX_ALLOC_HOST)
        check(hipApi().hostFree(ptr), "hipHostFree");
      else if (info.kind != GPUX_ALLOC_DEVICE ||
               !deviceBlockCache().put(info.device, ptr, info.bytes, stream))
        check(hipApi().free_(ptr), "hipFree");
    }
    release(); // taken in alloc()
  }

  static void suggestBlockSize(Kernel *kernel, const uint32_t *global,
                               uint32_t *block, size_t numDims) {
    if (!kernel)
      fail("Invalid kernel");
    if (numDims < 1 || numDims > 3 || !global || !block)
      fail("gpuxSuggestBlockSize: numDims must be 1..3");
    // 256 threads (4 wave64) is the preferred CDNA workgroup for
    // one-item-per-thread kernels; a tighter launch bound wins.
    uint32_t maxWg = kernel->maxThreads ? kernel->maxThreads : 256;
    if (maxWg > 256)
      maxWg = 256;
    maxWg = downPow2(maxWg);
    for (size_t i = 0; i < numDims; ++i) {
      uint32_t g = global[i];
      if (g > 1) {
        uint32_t l = g < maxWg ? g : maxWg;
        block[i] = l;
        maxWg /= upPow2(l);
        if (maxWg == 0)
          maxWg = 1;
      } else {
        block[i] = 1;
      }
    }
  }

private:
  std::atomic<unsigned> refs{1};
  std::string deviceName;
  int device = 0;
  hipStream_t stream = nullptr;
  std::mutex poolMutex;
  Event *freeList = nullptr;
  std::atomic<uint64_t> enqueued{0};  // launches put on the stream so far
  std::atomic<uint64_t> completed{0}; // launches known to have finished

  // Makes this queue's stream wait for the dependencies.  Events of this
  // queue are earlier positions of the same in-order stream: nothing to do.
  void waitOnStream(Event **deps) {
    for (Event **d = deps; *d; ++d) {
      Event *dep = *d;
      if (dep->owner == this)
        continue;
      dep->owner->recordForOthers(dep);
      check(hipApi().streamWaitEvent(stream, dep->event, 0),
            "hipStreamWaitEvent");
    }
  }

  // Gives `ev` a real device event other streams can wait on.
  void recordForOthers(Event *ev) {
    std::lock_guard<std::mutex> lock(poolMutex);
    if (ev->recorded)
      return;
    check(hipApi().setDevice(device), "hipSetDevice");
    if (!ev->event)
      check(hipApi().eventCreateWithFlags(&ev->event, hipEventDisableTiming),
            "hipEventCreateWithFlags");
    check(hipApi().eventRecord(ev->event, stream), "hipEventRecord");
    ev->recorded = true;
  }

  Event *getEvent() {
    Event *ev = nullptr;
    {
      std::lock_guard<std::mutex> lock(poolMutex);
      if (freeList) {
        ev = freeList;
        freeList = ev->next;
        ev->next = nullptr;
      }
    }
    if (!ev)
      ev = new Event;
    ev->owner = this;
    ev->recorded = false;
    retain(); // until gpuxDestroyEvent (GpuRuntime.cpp:287-299)
    return ev;
  }
};

Queue *toQueue(void *queue) {
  if (!queue)
    fail("Invalid queue");
  return static_cast<Queue *>(static_cast<numba::HipQueueInterface *>(queue));
}

} // namespace

#define GPUX_EXPORT extern "C" __attribute__((visibility("default")))

GPUX_EXPORT void *gpuxQueueCreate(const char *deviceName) {
  CallLog log(__func__);
  return guarded([&]() -> void * {
    return static_cast<numba::HipQueueInterface *>(new Queue(deviceName));
  });
}

GPUX_EXPORT void gpuxQueueDestroy(void *queue) {
  CallLog log(__func__);
  guarded([&]() { toQueue(queue)->release(); });
}

GPUX_EXPORT void *gpuxModuleLoad(void *queue, const void *data, size_t size) {
  CallLog log(__func__);
  return guarded(
      [&]() -> void * { return toQueue(queue)->loadModule(data, size); });
}

GPUX_EXPORT void gpuxModuleDestroy(void *module) {
  CallLog log(__func__);
  guarded([&]() {
    auto *mod = static_cast<Module *>(module);
    if (!mod)
      fail("Invalid module");
    check(hipApi().setDevice(mod->device), "hipSetDevice");
    check(hipApi().moduleUnload(mod->module), "hipModuleUnload");
    delete mod;
  });
}

GPUX_EXPORT void *gpuxKernelGet(void *module, const char *name) {
  CallLog log(__func__);
  return guarded([&]() -> void * {
    auto *mod = static_cast<Module *>(module);
    if (!mod)
      fail("Invalid module");
    if (!name)
      fail("Invalid kernel name");
    check(hipApi().setDevice(mod->device), "hipSetDevice");
    auto kernel = new Kernel;
    kernel->device = mod->device;
    hipError_t err =
        hipApi().moduleGetFunction(&kernel->function, mod->module, name);
    if (err != hipSuccess) {
      delete kernel;
      fail("Kernel '%s' not found in module: %s (%d)", name,
           hipApi().getErrorString(err), static_cast<int>(err));
    }
    int maxThreads = 0;
    if (hipApi().funcGetAttribute(&maxThreads,
                                  HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK,
                                  kernel->function) == hipSuccess &&
        maxThreads > 0)
      kernel->maxThreads = static_cast<uint32_t>(maxThreads);
    return kernel;
  });
}

GPUX_EXPORT void gpuxKernelDestroy(void *kernel) {
  CallLog log(__func__);
  guarded([&]() {
    if (!kernel)
      fail("Invalid kernel");
    delete static_cast<Kernel *>(kernel);
  });
}

GPUX_EXPORT void *gpuxLaunchKernel(void *queue, void *kernel, size_t gridX,
                                   size_t gridY, size_t gridZ, size_t blockX,
                                   size_t blockY, size_t blockZ,
                                   void *depEvents, void *params) {
  CallLog log(__func__);
  return guarded([&]() -> void * {
    return toQueue(queue)->launch(
        static_cast<Kernel *>(kernel), gridX, gridY, gridZ, blockX, blockY,
        blockZ, static_cast<Event **>(depEvents),
        static_cast<GpuxParamDesc *>(params));
  });
}

GPUX_EXPORT void gpuxWait(void *queue, void *event) {
  CallLog log(__func__);
  guarded([&]() { toQueue(queue)->wait(static_cast<Event *>(event)); });
}

GPUX_EXPORT void gpuxDestroyEvent(void *queue, void *event) {
  CallLog log(__func__);
  guarded([&]() {
    // The event goes back to the pool of the queue that handed it out (and
    // drops that queue's reference), whichever queue the caller names.
    Queue *named = toQueue(queue);
    Event *ev = static_cast<Event *>(event);
    (ev && ev->owner ? ev->owner : named)->destroyEvent(ev);
  });
}

GPUX_EXPORT void gpuxAlloc(void *queue, size_t size, size_t alignment, int type,
                           void *depEvents, GpuxAllocResult *result) {
  CallLog log(__func__);
  guarded([&]() {
    if (!result)
      fail("gpuxAlloc: null result");
    auto res = toQueue(queue)->alloc(size, alignment, type,
                                     static_cast<Event **>(depEvents));
    result->ptr = res.first;
    result->event = res.second;
  });
}

GPUX_EXPORT void gpuxDeAlloc(void *queue, void *ptr) {
  CallLog log(__func__);
  guarded([&]() { toQueue(queue)->dealloc(ptr); });
}

GPUX_EXPORT void gpuxSuggestBlockSize(void *queue, void *kernel,
                                      const uint32_t *gridSize,
                                      uint32_t *blockSize, size_t numDims) {
  CallLog log(__func__);
  guarded([&]() {
    (void)toQueue(queue);
    Queue::suggestBlockSize(static_cast<Kernel *>(kernel), gridSize, blockSize,
                            numDims);
  });
}

GPUX_EXPORT void *gpuxDuplicateQueue(void *rawNativeQueue) {
  CallLog log(__func__);
  return guarded([&]() -> void * {
    if (!rawNativeQueue)
      fail("Invalid native queue");
    auto *copy = static_cast<hipStream_t *>(std::malloc(sizeof(hipStream_t)));
    if (!copy)
      fail("Failed to allocate host memory");
    *copy = *static_cast<hipStream_t *>(rawNativeQueue);
    return copy;
  });
}
