// Lowered host code + kernel dispatcher (include/numba_mlir_hip/Offload.h).
//
// Every device action goes through the registered gpux* pointers in the order
// the reference's generated host code uses (reference:
// mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:228-857; handle caching
// mlir_compiler/lib/pipelines/LowerToGpu.cpp:742-940 and
// numba_mlir_runtime/lib/Context.cpp:25-60).
#include "numba_mlir_hip/Offload.h"

#include "numba_mlir_hip/GpuQueueInterface.hpp"
#include "numba_mlir_hip/MathRuntime.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <initializer_list>
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

// Code objects, embedded by Blobs.S.
extern "C" const unsigned char nmhip_blob_maps[], nmhip_blob_maps_end[];
extern "C" const unsigned char nmhip_blob_reduce[], nmhip_blob_reduce_end[];
extern "C" const unsigned char nmhip_blob_reduce_release[],
    nmhip_blob_reduce_release_end[];
extern "C" const unsigned char nmhip_blob_twins[], nmhip_blob_twins_end[];

namespace {

[[noreturn]] void fail(const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  throw std::runtime_error(buf);
}

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

// ---- the symbol table the lowered code calls through ----------------------

struct Symbols {
  void *(*QueueCreate)(const char *) = nullptr;
  void (*QueueDestroy)(void *) = nullptr;
  void *(*ModuleLoad)(void *, const void *, size_t) = nullptr;
  void (*ModuleDestroy)(void *) = nullptr;
  void *(*KernelGet)(void *, const char *) = nullptr;
  void (*KernelDestroy)(void *) = nullptr;
  void *(*LaunchKernel)(void *, void *, size_t, size_t, size_t, size_t, size_t,
                        size_t, void *, void *) = nullptr;
  void (*Wait)(void *, void *) = nullptr;
  void (*DestroyEvent)(void *, void *) = nullptr;
  void (*Alloc)(void *, size_t, size_t, int, void *, GpuxAllocResult *) =
      nullptr;
  void (*DeAlloc)(void *, void *) = nullptr;
  void (*SuggestBlockSize)(void *, void *, const uint32_t *, uint32_t *,
                           size_t) = nullptr;
  void *(*DuplicateQueue)(void *) = nullptr;
  void (*GemmF32)(void *, const NmhipMemref2F32 *, const NmhipMemref2F32 *,
                  float, float, NmhipMemref2F32 *) = nullptr;
  void (*GemmF64)(void *, const NmhipMemref2F64 *, const NmhipMemref2F64 *,
                  double, double, NmhipMemref2F64 *) = nullptr;
};

Symbols &symbols() {
  static Symbols s;
  return s;
}

template <typename T> T need(T fn, const char *name) {
  if (!fn)
    fail("Runtime symbol '%s' is not registered (load the HIP GPU runtime "
         "first)",
         name);
  return fn;
}
#define SYM(field, cname) need(symbols().field, cname)

// ---- tuning knobs ----------------------------------------------------------

struct Tuning {
  int64_t rowbcastRows = 0;
  int64_t mapBlocks = 0;
  int64_t reduceBlocks = 0;
  int64_t axis0Rows = 0;
  int64_t pairwiseRows = 0;
  int64_t bsBlocks = 0;
  int64_t colsBlocks = 0;
  // Non-zero: reduction kernels come from the code object whose hand-off of
  // partial results uses release / acquire (slower; for checking the default
  // hand-off against).
  int64_t handoffRelease = 0;
};

Tuning &tuning() {
  static Tuning t;
  return t;
}

// Which of the block-per-row kernels of float32 rows (`stem`_wide[_w4|_w3]_f32;
// reduce.hip) suits rows of n1 elements read as 128-bit words: a row is read
// in batches of 16 KiB (1024 words), the rest word by word a lane.  Rows of
// exactly one batch run fastest at four waves a SIMD, rows of two or three
// whole batches at three when there are thousands of them, anything else
// uncapped.
std::string wideRowKernel(const char *stem, int64_t n0, int64_t n1, bool words) {
  const int64_t nvec = n1 / 4;
  const char *cap = "";
  if (words && nvec % 1024 == 0) {
    const int64_t batches = nvec / 1024;
    if (batches == 1)
      cap = "_w4";
    else if (batches <= 3 && n0 >= 4096)
      cap = "_w3";
  }
  return std::string(stem) + "_wide" + cap + "_f32";
}

// Blocks of the float32 full sums (nmk_sum_all_f32, nmk_norm2_f32), each with
// 16 KiB of loads in flight: 6 MiB over the device.  Measured on MI355X over
// 512 MiB: 256 blocks 88.9 us, 320 80.5, 384 76.5, 448 77.1, 512 78.2, 768 79.4.
constexpr int64_t kFullSumBlocks = 384;

int64_t ceilDiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// ---- kernel argument packing ----------------------------------------------

struct Arg {
  union {
    int64_t i64;
    int32_t i32;
    double f64;
    float f32;
    const void *ptr;
  } v;
  int32_t size;
  int32_t type;

  static Arg I64(int64_t x) {
    Arg a;
    a.v.i64 = x;
    a.size = 8;
    a.type = GPUX_PARAM_INT64;
    return a;
  }
  static Arg I32(int32_t x) {
    Arg a;
    a.v.i64 = 0;
    a.v.i32 = x;
    a.size = 4;
    a.type = GPUX_PARAM_INT32;
    return a;
  }
  static Arg F32(float x) {
    Arg a;
    a.v.i64 = 0;
    a.v.f32 = x;
    a.size = 4;
    a.type = GPUX_PARAM_FLOAT32;
    return a;
  }
  static Arg F64(double x) {
    Arg a;
    a.v.f64 = x;
    a.size = 8;
    a.type = GPUX_PARAM_FLOAT64;
    return a;
  }
  static Arg Ptr(const void *p) {
    Arg a;
    a.v.ptr = p;
    a.size = 8;
    a.type = GPUX_PARAM_PTR;
    return a;
  }
};

struct Blob {
  const char *family;
  const unsigned char *begin;
  const unsigned char *end;
};

const Blob *findBlob(const char *family) {
  static const Blob blobs[] = {
      {"maps", nmhip_blob_maps, nmhip_blob_maps_end},
      {"reduce", nmhip_blob_reduce, nmhip_blob_reduce_end},
      // reduce.hip built with NMK_HANDOFF_RELEASE=1 (csrc/kernels/common.h)
      {"reduce_release", nmhip_blob_reduce_release, nmhip_blob_reduce_release_end},
      {"twins", nmhip_blob_twins, nmhip_blob_twins_end},
  };
  for (const Blob &b : blobs)
    if (std::strcmp(b.family, family) == 0)
      return &b;
  return nullptr;
}

// Kernel name -> family.  Names are prefixed by family:
//   nmk_map2_*, nmk_black_scholes_*, nmk_fill_* : maps
//   nmk_sum_*, nmk_norm2_*, nmk_reduce*         : reduce
//   nmk_twin_*                                  : twins
const char *familyOf(const std::string &kernel) {
  auto starts = [&](const char *p) { return kernel.rfind(p, 0) == 0; };
  if (starts("nmk_map2_") || starts("nmk_black_scholes_") ||
      starts("nmk_fill_") || starts("nmk_copy_"))
    return "maps";
  if (starts("nmk_sum_") || starts("nmk_norm2_") || starts("nmk_reduce"))
    return "reduce";
  if (starts("nmk_twin_"))
    return "twins";
  fail("Kernel '%s' does not belong to a built-in code object", kernel.c_str());
}

constexpr size_t kMaxTickets = 4096;

class Context {
public:
  explicit Context(const char *device) {
    queue = SYM(QueueCreate, "gpuxQueueCreate")(device);
  }

  ~Context() {
    // Outlined deinit: kernels, modules, then the queue
    // (LowerToGpu.cpp:698-715, 832-858).
    if (lastEvent)
      retireEvent(lastEvent, true);
    if (staging)
      symbols().DeAlloc(queue, staging);
    if (scratch)
      symbols().DeAlloc(queue, scratch);
    if (tickets)
      symbols().DeAlloc(queue, tickets);
    for (auto &kv : kernels)
      symbols().KernelDestroy(kv.second);
    for (auto &kv : modules)
      symbols().ModuleDestroy(kv.second);
    symbols().QueueDestroy(queue);
  }

  void *queue = nullptr;
  bool async = false;
  std::string lastKernel;
  std::mutex mutex;

  void *kernel(const std::string &name) {
    const char *family = familyOf(name);
    if (tuning().handoffRelease && std::strcmp(family, "reduce") == 0)
      family = "reduce_release";
    const std::string key = std::string(family) + ":" + name;
    auto it = kernels.find(key);
    if (it != kernels.end())
      return it->second;
    void *&mod = modules[family];
    if (!mod) {
      const Blob *blob = findBlob(family);
      mod = SYM(ModuleLoad, "gpuxModuleLoad")(
          queue, blob->begin, static_cast<size_t>(blob->end - blob->begin));
    }
    void *k = SYM(KernelGet, "gpuxKernelGet")(mod, name.c_str());
    kernels.emplace(key, k);
    return k;
  }

  void launchDesc(const std::string &name, const size_t grid[3],
                  const size_t block[3], GpuxParamDesc *params) {
    void *k = kernel(name);
    lastKernel = name;
    void *deps[1] = {nullptr};
    void *ev = SYM(LaunchKernel, "gpuxLaunchKernel")(
        queue, k, grid[0], grid[1], grid[2], block[0], block[1], block[2], deps,
        params);
    if (async) {
      if (lastEvent)
        retireEvent(lastEvent, false);
      lastEvent = ev;
    } else {
      retireEvent(ev, true);
    }
  }

  void launch(const std::string &name, size_t gx, size_t gy, size_t gz,
              size_t bx, size_t by, size_t bz, std::initializer_list<Arg> args) {
    std::vector<Arg> slots(args);
    std::vector<GpuxParamDesc> descs(slots.size() + 1);
    for (size_t i = 0; i < slots.size(); ++i) {
      descs[i].data = &slots[i].v;
      descs[i].size = slots[i].size;
      descs[i].type = slots[i].type;
    }
    descs[slots.size()] = GpuxParamDesc{nullptr, 0, GPUX_PARAM_NULL};
    const size_t grid[3] = {gx, gy, gz};
    const size_t block[3] = {bx, by, bz};
    launchDesc(name, grid, block, descs.data());
  }

  // A launch of `blocks` blocks of 256 lanes whose kernel counts its blocks
  // along x, then y (blockLinearXY): a dimension of a launch holds at most
  // 2^32 - 1 work-items, 2^24 - 1 such blocks.
  void launchBlocksXY(const std::string &name, int64_t blocks,
                      std::initializer_list<Arg> args) {
    const int64_t most = int64_t(1) << 23;
    const int64_t gx = blocks < most ? blocks : most;
    const int64_t gy = ceilDiv(blocks, gx);
    if (gy > 65535)
      fail("%s: %lld blocks are more than one launch holds", name.c_str(), (long long)blocks);
    launch(name, size_t(gx), size_t(gy), 1, 256, 1, 1, args);
  }

  void synchronize() {
    if (lastEvent) {
      retireEvent(lastEvent, true);
      lastEvent = nullptr;
    }
  }

  void *alloc(size_t bytes, int type) {
    void *deps[1] = {nullptr};
    GpuxAllocResult res = {nullptr, nullptr};
    // 64-byte alignment request, then wait + destroy of the alloc event
    // (GpuRuntimeToLlvm.cpp:670, 741-744).
    SYM(Alloc, "gpuxAlloc")(queue, bytes, 64, type, deps, &res);
    retireEvent(res.event, true);
    return res.ptr;
  }

  void free(void *ptr) { SYM(DeAlloc, "gpuxDeAlloc")(queue, ptr); }

  // Device scratch for single-launch reductions: `bytes` of partials plus
  // kMaxTickets zeroed ticket counters.  Kernels leave the tickets at zero.
  void *scratchFor(size_t bytes) {
    if (!tickets) {
      tickets = static_cast<uint32_t *>(
          alloc(kMaxTickets * sizeof(uint32_t), GPUX_ALLOC_DEVICE));
      launch("nmk_fill_u32", 16, 1, 1, 256, 1, 1,
             {Arg::Ptr(tickets), Arg::I32(0), Arg::I64(kMaxTickets)});
    }
    if (bytes > scratchBytes) {
      if (scratch) {
        synchronize();
        free(scratch);
      }
      scratchBytes = bytes < (size_t(1) << 20) ? (size_t(1) << 20) : bytes;
      scratch = alloc(scratchBytes, GPUX_ALLOC_DEVICE);
    }
    return scratch;
  }

  uint32_t *tickets = nullptr;

  // Host <-> device transfers without leaving the C-ABI: a pinned, device-
  // visible staging block from gpuxAlloc(Host), filled or drained by memcpy
  // on the host side and by the byte-copy kernel (launched and waited for
  // through gpuxLaunchKernel / gpuxWait) on the device side.  Two halves
  // alternate, so the host copies one while the kernel moves the other.
  static constexpr size_t kStagingHalf = size_t(16) << 20;

  // Each half has 16 spare bytes: a transfer is staged at the offset within a
  // 128-bit word that its device address has (`skew`, the same for every
  // chunk: the chunks are whole words apart), so that the copy kernel moves
  // words whatever the view's first byte.
  char *stagingHalf(int which, size_t skew = 0) {
    if (!staging)
      staging = static_cast<char *>(alloc(2 * (kStagingHalf + 16), GPUX_ALLOC_HOST));
    return staging + size_t(which) * (kStagingHalf + 16) + skew;
  }

  void *copyBytesAsync(const void *src, void *dst, size_t bytes) {
    Arg slots[3] = {Arg::Ptr(src), Arg::Ptr(dst), Arg::I64(int64_t(bytes))};
    GpuxParamDesc descs[4];
    for (int i = 0; i < 3; ++i) {
      descs[i].data = &slots[i].v;
      descs[i].size = slots[i].size;
      descs[i].type = slots[i].type;
    }
    descs[3] = GpuxParamDesc{nullptr, 0, GPUX_PARAM_NULL};
    size_t blocks = (bytes / 16 + 255) / 256;
    if (blocks < 1)
      blocks = 1;
    if (blocks > 4096)
      blocks = 4096;
    void *deps[1] = {nullptr};
    return SYM(LaunchKernel, "gpuxLaunchKernel")(
        queue, kernel("nmk_copy_bytes"), blocks, 1, 1, 256, 1, 1, deps, descs);
  }

  void hostToDevice(void *dev, const void *host, size_t bytes) {
    synchronize();
    void *pending[2] = {nullptr, nullptr};
    int half = 0;
    const size_t skew = reinterpret_cast<uintptr_t>(dev) & 15u;
    for (size_t off = 0; off < bytes; off += kStagingHalf, half ^= 1) {
      const size_t n = bytes - off < kStagingHalf ? bytes - off : kStagingHalf;
      if (pending[half]) { // the kernel that last read this half
        retireEvent(pending[half], true);
        pending[half] = nullptr;
      }
      char *stage = stagingHalf(half, skew);
      std::memcpy(stage, static_cast<const char *>(host) + off, n);
      pending[half] = copyBytesAsync(stage, static_cast<char *>(dev) + off, n);
    }
    for (void *ev : pending)
      if (ev)
        retireEvent(ev, true);
  }

  void deviceToHost(void *host, const void *dev, size_t bytes) {
    synchronize();
    void *pending[2] = {nullptr, nullptr};
    size_t pendingOff[2] = {0, 0}, pendingBytes[2] = {0, 0};
    const size_t skew = reinterpret_cast<uintptr_t>(dev) & 15u;
    auto drain = [&](int half) {
      if (!pending[half])
        return;
      retireEvent(pending[half], true);
      pending[half] = nullptr;
      std::memcpy(static_cast<char *>(host) + pendingOff[half], stagingHalf(half, skew),
                  pendingBytes[half]);
    };
    int half = 0;
    for (size_t off = 0; off < bytes; off += kStagingHalf, half ^= 1) {
      const size_t n = bytes - off < kStagingHalf ? bytes - off : kStagingHalf;
      drain(half);
      pending[half] = copyBytesAsync(static_cast<const char *>(dev) + off,
                                     stagingHalf(half, skew), n);
      pendingOff[half] = off;
      pendingBytes[half] = n;
      drain(half ^ 1); // the other half's kernel ran while this one was queued
    }
    drain(0);
    drain(1);
  }

private:
  std::unordered_map<std::string, void *> modules;
  std::unordered_map<std::string, void *> kernels;
  void *lastEvent = nullptr;
  void *scratch = nullptr;
  size_t scratchBytes = 0;
  char *staging = nullptr;

  void retireEvent(void *ev, bool wait) {
    if (wait)
      SYM(Wait, "gpuxWait")(queue, ev);
    SYM(DestroyEvent, "gpuxDestroyEvent")(queue, ev);
  }
};

Context *toCtx(void *ctx) {
  if (!ctx)
    fail("Invalid context");
  return static_cast<Context *>(ctx);
}

const char *dtypeName(int dtype) {
  switch (dtype) {
  case NMHIP_I32:
    return "i32";
  case NMHIP_I64:
    return "i64";
  case NMHIP_F32:
    return "f32";
  case NMHIP_F64:
    return "f64";
  }
  fail("Unsupported dtype %d", dtype);
}

size_t dtypeSize(int dtype) {
  return (dtype == NMHIP_I32 || dtype == NMHIP_F32) ? 4 : 8;
}

} // namespace

#define NMHIP_EXPORT extern "C" __attribute__((visibility("default")))

NMHIP_EXPORT int nmhipRegisterSymbol(const char *name, void *address) {
  return guarded([&]() -> int {
    if (!name)
      fail("nmhipRegisterSymbol: null name");
    Symbols &s = symbols();
    struct Entry {
      const char *name;
      void **slot;
    };
    const Entry table[] = {
        {"gpuxQueueCreate", reinterpret_cast<void **>(&s.QueueCreate)},
        {"gpuxQueueDestroy", reinterpret_cast<void **>(&s.QueueDestroy)},
        {"gpuxModuleLoad", reinterpret_cast<void **>(&s.ModuleLoad)},
        {"gpuxModuleDestroy", reinterpret_cast<void **>(&s.ModuleDestroy)},
        {"gpuxKernelGet", reinterpret_cast<void **>(&s.KernelGet)},
        {"gpuxKernelDestroy", reinterpret_cast<void **>(&s.KernelDestroy)},
        {"gpuxLaunchKernel", reinterpret_cast<void **>(&s.LaunchKernel)},
        {"gpuxWait", reinterpret_cast<void **>(&s.Wait)},
        {"gpuxDestroyEvent", reinterpret_cast<void **>(&s.DestroyEvent)},
        {"gpuxAlloc", reinterpret_cast<void **>(&s.Alloc)},
        {"gpuxDeAlloc", reinterpret_cast<void **>(&s.DeAlloc)},
        {"gpuxSuggestBlockSize",
         reinterpret_cast<void **>(&s.SuggestBlockSize)},
        {"gpuxDuplicateQueue", reinterpret_cast<void **>(&s.DuplicateQueue)},
        {"mkl_gemm_float32_device", reinterpret_cast<void **>(&s.GemmF32)},
        {"mkl_gemm_float64_device", reinterpret_cast<void **>(&s.GemmF64)},
    };
    // The JIT sees the gemm entry points under the _mlir_ciface_ prefix
    // (math_runtime.py:21-40).
    static const char prefix[] = "_mlir_ciface_";
    if (std::strncmp(name, prefix, sizeof(prefix) - 1) == 0)
      name += sizeof(prefix) - 1;
    for (const Entry &e : table) {
      if (std::strcmp(e.name, name) == 0) {
        *e.slot = address;
        return 0;
      }
    }
    return -1;
  });
}

NMHIP_EXPORT void *nmhipContextCreate(const char *deviceName) {
  return guarded([&]() -> void * { return new Context(deviceName); });
}

NMHIP_EXPORT void nmhipContextDestroy(void *ctx) {
  guarded([&]() { delete toCtx(ctx); });
}

NMHIP_EXPORT void nmhipContextSetAsync(void *ctx, int async) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (!async)
      c->synchronize();
    c->async = async != 0;
  });
}

NMHIP_EXPORT void nmhipContextSynchronize(void *ctx) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    c->synchronize();
  });
}

NMHIP_EXPORT void *nmhipContextQueue(void *ctx) {
  return guarded([&]() -> void * { return toCtx(ctx)->queue; });
}

NMHIP_EXPORT const char *nmhipLastKernelName(void *ctx) {
  return guarded([&]() -> const char * { return toCtx(ctx)->lastKernel.c_str(); });
}

NMHIP_EXPORT void *nmhipAlloc(void *ctx, size_t bytes, int type) {
  return guarded([&]() -> void * { return toCtx(ctx)->alloc(bytes, type); });
}

NMHIP_EXPORT void nmhipFree(void *ctx, void *dev) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    {
      std::lock_guard<std::mutex> lock(c->mutex);
      c->synchronize();
    }
    c->free(dev);
  });
}

NMHIP_EXPORT void nmhipMemcpyHtoD(void *ctx, void *dev, const void *host,
                                  size_t bytes) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (bytes != 0)
      c->hostToDevice(dev, host, bytes);
  });
}

NMHIP_EXPORT void nmhipMemcpyDtoH(void *ctx, void *host, const void *dev,
                                  size_t bytes) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (bytes != 0)
      c->deviceToHost(host, dev, bytes);
  });
}

NMHIP_EXPORT void nmhipCopy(void *ctx, void *dst, const void *src,
                            size_t bytes) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (bytes == 0)
      return;
    if (bytes % 16 != 0 || !aligned16(dst) || !aligned16(src))
      fail("nmhipCopy: needs 16-byte aligned pointers and size");
    const int64_t nvec = int64_t(bytes / 16);
    int64_t blocks = ceilDiv(nvec, 256);
    if (blocks > (int64_t(1) << 20))
      blocks = int64_t(1) << 20;
    c->launch("nmk_copy_b128", size_t(blocks), 1, 1, 256, 1, 1,
              {Arg::Ptr(src), Arg::Ptr(dst), Arg::I64(nvec)});
  });
}

NMHIP_EXPORT void nmhipMapBinary(void *ctx, int op, int dtype, const void *a,
                                 const int64_t aS[2], const void *b,
                                 const int64_t bS[2], void *out,
                                 const int64_t oS[2], int64_t n0, int64_t n1) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (n0 < 0 || n1 < 0)
      fail("nmhipMapBinary: negative extent");
    if (n0 == 0 || n1 == 0)
      return;
    static const char *const opNames[] = {"add", "sub", "mul", "div"};
    if (op < 0 || op > NMHIP_DIV)
      fail("Unsupported binary op %d", op);
    if (op == NMHIP_DIV && dtype != NMHIP_F32 && dtype != NMHIP_F64)
      fail("nmhipMapBinary: division is implemented for float32 and float64");
    const std::string suffix =
        std::string(opNames[op]) + "_" + dtypeName(dtype);
    const bool isFloat = dtype == NMHIP_F32 || dtype == NMHIP_F64;
    const int64_t lanesElems = 16 / static_cast<int64_t>(dtypeSize(dtype));
    auto dense = [&](const int64_t s[2]) {
      return s[1] == 1 && (n0 == 1 || s[0] == n1);
    };
    auto rowBroadcast = [&](const int64_t s[2]) {
      return s[1] == 1 && s[0] == 0 && n0 > 1;
    };
    const bool alignedAll = aligned16(a) && aligned16(b) && aligned16(out);

    if (isFloat && alignedAll && dense(oS) && dense(aS) && dense(bS) &&
        (n0 * n1) % lanesElems == 0) {
      const int64_t nvec = n0 * n1 / lanesElems;
      int64_t blocks = tuning().mapBlocks ? tuning().mapBlocks : 256 * 16;
      const int64_t need = ceilDiv(nvec, 2 * 256);
      if (blocks > need)
        blocks = need;
      c->launch("nmk_map2_contig_" + suffix, size_t(blocks), 1, 1, 256, 1, 1,
                {Arg::Ptr(a), Arg::Ptr(b), Arg::Ptr(out), Arg::I64(n0 * n1)});
      return;
    }
    // Row-broadcast operand on either side (commutative ops may swap).
    const void *full = a;
    const void *row = b;
    bool rowCase = dense(aS) && rowBroadcast(bS);
    if (!rowCase && op != NMHIP_SUB && op != NMHIP_DIV && dense(bS) &&
        rowBroadcast(aS)) {
      full = b;
      row = a;
      rowCase = true;
    }
    if (isFloat && alignedAll && rowCase && dense(oS) && n1 % lanesElems == 0) {
      const int64_t gx = ceilDiv(n1, 256 * lanesElems);
      int64_t rowsPerBlock = tuning().rowbcastRows;
      if (!rowsPerBlock) {
        // Two rows per block: many short-lived blocks stream best; more
        // only when grid.y would overflow.
        rowsPerBlock = 2;
        if (ceilDiv(n0, rowsPerBlock) > 65535)
          rowsPerBlock = ceilDiv(n0, 65535);
      }
      const int64_t gy = ceilDiv(n0, rowsPerBlock);
      if (gy <= 65535) {
        c->launch("nmk_map2_rowbcast_" + suffix, size_t(gx), size_t(gy), 1, 256,
                  1, 1,
                  {Arg::Ptr(full), Arg::Ptr(row), Arg::Ptr(out), Arg::I64(n0),
                   Arg::I64(n1), Arg::I64(rowsPerBlock)});
        return;
      }
    }
    // General case: one element per work-item, x <-> last dimension, block
    // from the runtime's suggestion, tail guarded in the kernel
    // (GpuToGpuRuntime.cpp:1395-1584).
    const std::string name = "nmk_map2_strided_" + suffix;
    if (n0 > 0xffffffffll || n1 > 0xffffffffll)
      fail("nmhipMapBinary: extent above 2^32");
    const uint32_t global[2] = {static_cast<uint32_t>(n1),
                                static_cast<uint32_t>(n0)};
    uint32_t block[2] = {1, 1};
    SYM(SuggestBlockSize, "gpuxSuggestBlockSize")(c->queue, c->kernel(name),
                                                  global, block, 2);
    int64_t gy = ceilDiv(n0, block[1]), gz = 1;
    if (gy > 65535) {
      gz = ceilDiv(gy, 65535);
      gy = 65535;
      if (gz > 65535)
        fail("nmhipMapBinary: %lld rows are more than one launch holds", (long long)n0);
    }
    c->launch(name, size_t(ceilDiv(n1, block[0])), size_t(gy), size_t(gz), block[0],
              block[1], 1,
              {Arg::Ptr(a), Arg::I64(aS[0]), Arg::I64(aS[1]), Arg::Ptr(b),
               Arg::I64(bS[0]), Arg::I64(bS[1]), Arg::Ptr(out), Arg::I64(oS[0]),
               Arg::I64(oS[1]), Arg::I64(n0), Arg::I64(n1)});
  });
}

NMHIP_EXPORT void nmhipBlackScholesF32(void *ctx, const float *price,
                                       const float *strike, const float *t,
                                       float rate, float volatility,
                                       float *call, float *put, int64_t n,
                                       int wide) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (n < 0)
      fail("nmhipBlackScholesF32: negative extent");
    if (n == 0)
      return;
    if (!(aligned16(price) && aligned16(strike) && aligned16(t) &&
          aligned16(call) && aligned16(put)))
      fail("nmhipBlackScholesF32: arrays must be 16-byte aligned");
    // Four options per lane and trip.  Both kernels stream best from many
    // short blocks, two trips a lane (8192 blocks at 2^24 options: 2.5 us
    // faster than 4096 blocks and than 16384, where staging the erf table
    // once per block weighs more), the two trips 128 pieces of 256 words
    // (512 KiB of each array) apart (maps.hip, BsTrips: 1 to 1.6 us faster
    // than a grid apart); small inputs and a block count set by hand walk by
    // whole grids.
    const int64_t need = ceilDiv(ceilDiv(n, 4), 256);
    int64_t blocks, distance, trips;
    if (!tuning().bsBlocks && need >= 4 * 128) {
      distance = 128;
      trips = 2;
      blocks = ceilDiv(need, distance * trips) * distance;
    } else {
      blocks = tuning().bsBlocks ? tuning().bsBlocks : ceilDiv(need, 2);
      if (blocks > need)
        blocks = need;
      if (blocks > 0x7fffffff)
        blocks = 0x7fffffff;
      distance = blocks;
      trips = ceilDiv(need, blocks);
    }
    if (blocks > 0x7fffffff || trips > 0x7fffffff)
      fail("nmhipBlackScholesF32: %lld options are more than one launch holds", (long long)n);
    c->launch(wide ? "nmk_black_scholes_f32_w64" : "nmk_black_scholes_f32_w32",
              size_t(blocks), 1, 1, 256, 1, 1,
              {Arg::Ptr(price), Arg::Ptr(strike), Arg::Ptr(t), Arg::F32(rate),
               Arg::F32(volatility), Arg::Ptr(call), Arg::Ptr(put),
               Arg::I64(n), Arg::I32(int32_t(distance)), Arg::I32(int32_t(trips))});
  });
}

NMHIP_EXPORT void nmhipReduce(void *ctx, int op, int dtype, const void *x,
                              int64_t n0, int64_t n1, int64_t s0, int64_t s1,
                              int axis, void *out) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (n0 < 0 || n1 < 0)
      fail("nmhipReduce: negative extent");
    if (axis < -1 || axis > 1)
      fail("nmhipReduce: axis must be -1, 0 or 1");
    static const char *const opNames[] = {"sum", "prod", "min", "max"};
    if (op < 0 || op > NMHIP_MAX)
      fail("Unsupported reduce op %d", op);
    const bool rowMajor = s1 == 1 && (n0 <= 1 || s0 >= n1);
    const bool contiguous = s1 == 1 && (n0 <= 1 || s0 == n1);

    // float32 row sums: a wave per row.
    if (op == NMHIP_SUM && dtype == NMHIP_F32 && axis == 1 && rowMajor &&
        n0 > 0 && n1 > 0) {
      const int vec = (aligned16(x) && s0 % 4 == 0 && n1 % 4 == 0) ? 1 : 0;
      // a block per row for long rows, a wave per row otherwise
      const bool wide = n1 >= 4096;
      c->launchBlocksXY(wide ? wideRowKernel("nmk_sum_axis1", n0, n1, vec != 0)
                             : std::string("nmk_sum_axis1_f32"),
                        wide ? n0 : ceilDiv(n0, 4),
                        {Arg::Ptr(x), Arg::Ptr(out), Arg::I64(n0), Arg::I64(n1),
                         Arg::I64(s0), Arg::I32(vec)});
      return;
    }
    // int32 column sums into int64: column strips x row chunks, device finish.
    if (op == NMHIP_SUM && dtype == NMHIP_I32 && axis == 0 && rowMajor &&
        aligned16(x) && s0 % 4 == 0 && n1 % 4 == 0 && n0 >= 64 && n1 > 0) {
      const int64_t strips = ceilDiv(n1, 256);
      int64_t rowsPerBlock = tuning().axis0Rows;
      if (!rowsPerBlock) {
        // One block per CU (256) measured fastest: few, long-lived blocks
        // keep the finish short.  Chunks of whole 64 rows: at [16384, 8192]
        // they start 64 MiB apart, which measured 2 us faster than chunks of
        // whole 24-row groups (6 loads x 4 waves) that do not.
        rowsPerBlock = ceilDiv(n0 * strips, 256);
        rowsPerBlock = ceilDiv(rowsPerBlock, 64) * 64;
      }
      const int64_t chunks = ceilDiv(n0, rowsPerBlock);
      if (strips <= int64_t(kMaxTickets) && chunks <= 65535) {
        void *partial = c->scratchFor(size_t(chunks) * size_t(n1) * 8);
        c->launch("nmk_sum_axis0_i32_i64", size_t(strips), size_t(chunks), 1,
                  256, 1, 1,
                  {Arg::Ptr(x), Arg::Ptr(out), Arg::I64(n0), Arg::I64(n1),
                   Arg::I64(s0), Arg::I64(rowsPerBlock), Arg::Ptr(partial),
                   Arg::Ptr(c->tickets)});
        return;
      }
    }
    // float32 full sum: grid-stride, device finish.
    if (op == NMHIP_SUM && dtype == NMHIP_F32 && axis == -1 && contiguous &&
        n0 * n1 >= 4096) {
      const int64_t n = n0 * n1;
      int64_t blocks = tuning().reduceBlocks ? tuning().reduceBlocks : kFullSumBlocks;
      const int64_t need = ceilDiv(n, 256 * 16);
      if (blocks > need)
        blocks = need;
      void *partial = c->scratchFor(size_t(blocks) * 4);
      c->launch("nmk_sum_all_f32", size_t(blocks), 1, 1, 256, 1, 1,
                {Arg::Ptr(x), Arg::Ptr(out), Arg::I64(n),
                 Arg::I32(aligned16(x) ? 1 : 0), Arg::Ptr(partial),
                 Arg::Ptr(c->tickets)});
      return;
    }
    // Generic strided fallback: a wave per kept index.
    int64_t nKeep, nRed, sk, sr;
    if (axis == 1) {
      nKeep = n0;
      nRed = n1;
      sk = s0;
      sr = s1;
    } else if (axis == 0) {
      nKeep = n1;
      nRed = n0;
      sk = s1;
      sr = s0;
    } else {
      if (!contiguous)
        fail("nmhipReduce: a full reduction needs a C-contiguous array");
      nKeep = 1;
      nRed = n0 * n1;
      sk = 0;
      sr = 1;
    }
    if (nKeep == 0)
      return;
    const std::string opAndType = std::string(opNames[op]) + "_" + dtypeName(dtype);
    // the accumulator type's own kernels fold partial results
    const bool isInt = dtype == NMHIP_I32 || dtype == NMHIP_I64;
    const std::string opAndAcc =
        std::string(opNames[op]) + "_" + (isInt ? "i64" : dtypeName(dtype));
    const size_t accSize = dtype == NMHIP_F32 ? 4 : 8;
    // elements of the input in a 128-bit word
    const int64_t word = (dtype == NMHIP_F32 || dtype == NMHIP_I32) ? 4 : 2;
    // The kept index has unit stride (column sums of a row-major matrix):
    // lanes along the kept index, row chunks over grid.y, partial results
    // folded by the same kernel.
    if (sk == 1 && nKeep > 1 && nRed >= 64 && sr >= nKeep) {
      // a 128-bit word of adjacent kept indices a lane where every row of
      // the matrix begins and ends on one
      const int vec = (aligned16(x) && sr % word == 0 && nKeep % word == 0) ? 1 : 0;
      const int64_t strips = ceilDiv(nKeep, vec ? 64 * word : 256);
      // (few long blocks stream best on words -- 256 blocks: 79 us for
      // [16384, 8192] float32, 2048 blocks: 92 us -- many short ones on
      // single elements)
      int64_t chunks =
          ceilDiv(tuning().colsBlocks ? tuning().colsBlocks : vec ? 256 : 2048, strips);
      if (chunks > nRed / 32)
        chunks = nRed / 32;
      if (chunks < 1)
        chunks = 1;
      if (chunks > 65535)
        chunks = 65535;
      const int64_t rowsPerChunk = ceilDiv(nRed, chunks);
      chunks = ceilDiv(nRed, rowsPerChunk);
      if (chunks == 1) {
        c->launch("nmk_reducecols_" + opAndType, size_t(strips), 1, 1, 256, 1, 1,
                  {Arg::Ptr(x), Arg::Ptr(out), Arg::I64(nRed), Arg::I64(nKeep),
                   Arg::I64(sr), Arg::I64(nRed), Arg::I32(vec)});
      } else {
        void *partial = c->scratchFor(size_t(chunks) * size_t(nKeep) * accSize);
        c->launch("nmk_reducecols_" + opAndType, size_t(strips), size_t(chunks), 1,
                  256, 1, 1,
                  {Arg::Ptr(x), Arg::Ptr(partial), Arg::I64(nRed), Arg::I64(nKeep),
                   Arg::I64(sr), Arg::I64(rowsPerChunk), Arg::I32(vec)});
        c->launch("nmk_reducecols_" + opAndAcc, size_t(ceilDiv(nKeep, 256)), 1, 1, 256, 1,
                  1,
                  {Arg::Ptr(partial), Arg::Ptr(out), Arg::I64(chunks),
                   Arg::I64(nKeep), Arg::I64(nKeep), Arg::I64(chunks), Arg::I32(0)});
      }
      return;
    }
    // A long contiguous run reduced to one value: a wave per chunk, then the
    // chunks' results by one wave.
    if (nKeep == 1 && sr == 1 && nRed >= 65536) {
      // one block a chunk: as many as stream well at once, 16 KiB or more each
      int64_t nChunks = ceilDiv(nRed * int64_t(16 / word), 16384);
      const int64_t most = tuning().reduceBlocks ? tuning().reduceBlocks : 512;
      if (nChunks > most)
        nChunks = most;
      // (chunks of whole 128-bit words, so that every chunk of an aligned
      // array starts on one)
      const int64_t chunk = ceilDiv(ceilDiv(nRed, nChunks), word) * word;
      nChunks = ceilDiv(nRed, chunk);
      void *partial = c->scratchFor(size_t(nChunks) * accSize);
      c->launch("nmk_reducechunks_" + opAndType, size_t(nChunks), 1, 1, 256, 1, 1,
                {Arg::Ptr(x), Arg::Ptr(partial), Arg::I64(nRed), Arg::I64(chunk),
                 Arg::I64(nChunks), Arg::I32(aligned16(x) ? 1 : 0)});
      c->launch("nmk_reduce_" + opAndAcc, 1, 1, 1, 256, 1, 1,
                {Arg::Ptr(partial), Arg::Ptr(out), Arg::I64(1), Arg::I64(nChunks),
                 Arg::I64(0), Arg::I64(1), Arg::I64(1), Arg::I32(0)});
      return;
    }
    // Many short runs (the rows of a tall matrix of a few columns): a group
    // of 1 to 32 lanes a kept index, two elements or so a lane.
    if (nRed >= 1 && nRed <= 64 && nKeep >= 4096) {
      int gShift = 0;
      while (sr == 1 && (int64_t(2) << gShift) < nRed && gShift < 5)
        ++gShift; // (a lane a kept index where the run is strided: the lanes then
                  // follow the kept index, which has the shorter stride)
      const int mode = 4 | (gShift << 8);
      c->launchBlocksXY(std::string("nmk_reduce_") + opNames[op] + "_" + dtypeName(dtype),
                        ceilDiv(nKeep << gShift, 256),
                        {Arg::Ptr(x), Arg::Ptr(out), Arg::I64(nKeep), Arg::I64(nRed),
                         Arg::I64(sk), Arg::I64(sr), Arg::I64(1), Arg::I32(mode)});
      return;
    }
    // (a block per kept index where the reduced run is long, a wave per
    // kept index otherwise)
    const bool wide = nRed >= 4096;
    const int mode = ((sr == 1 && aligned16(x) && (nKeep == 1 || sk % word == 0)) ? 1 : 0) |
                     (wide ? 2 : 0);
    c->launchBlocksXY(std::string("nmk_reduce_") + opNames[op] + "_" + dtypeName(dtype),
                      wide ? nKeep : ceilDiv(nKeep, 4),
                      {Arg::Ptr(x), Arg::Ptr(out), Arg::I64(nKeep), Arg::I64(nRed),
                       Arg::I64(sk), Arg::I64(sr), Arg::I64(1), Arg::I32(mode)});
  });
}

NMHIP_EXPORT void nmhipNorm2RowsF32(void *ctx, const float *x, int64_t n0,
                                    int64_t n1, int64_t s0, float *out) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (n0 < 0 || n1 < 0 || (n0 > 1 && s0 < n1))
      fail("nmhipNorm2RowsF32: needs a row-major array");
    if (n0 == 0)
      return;
    const int vec = (aligned16(x) && s0 % 4 == 0 && n1 % 4 == 0) ? 1 : 0;
    const bool wide = n1 >= 4096;
    c->launchBlocksXY(wide ? wideRowKernel("nmk_norm2_axis1", n0, n1, vec != 0)
                           : std::string("nmk_norm2_axis1_f32"),
                      wide ? n0 : ceilDiv(n0, 4),
                      {Arg::Ptr(x), Arg::Ptr(out), Arg::I64(n0), Arg::I64(n1),
                       Arg::I64(s0), Arg::I32(vec)});
  });
}

NMHIP_EXPORT void nmhipNorm2F32(void *ctx, const float *x, int64_t n,
                                float *out) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (n < 0)
      fail("nmhipNorm2F32: negative extent");
    int64_t blocks = tuning().reduceBlocks ? tuning().reduceBlocks : kFullSumBlocks;
    int64_t need = ceilDiv(n, 256 * 16);
    if (need < 1)
      need = 1;
    if (blocks > need)
      blocks = need;
    void *partial = c->scratchFor(size_t(blocks) * 4);
    c->launch("nmk_norm2_f32", size_t(blocks), 1, 1, 256, 1, 1,
              {Arg::Ptr(x), Arg::Ptr(out), Arg::I64(n),
               Arg::I32(aligned16(x) ? 1 : 0), Arg::Ptr(partial),
               Arg::Ptr(c->tickets)});
  });
}

NMHIP_EXPORT void nmhipGemm(void *ctx, int dtype, const void *a,
                            const int64_t aS[2], const void *b,
                            const int64_t bS[2], void *cPtr,
                            const int64_t cS[2], int64_t m, int64_t n,
                            int64_t k, double alpha, double beta) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (m < 0 || n < 0 || k < 0)
      fail("nmhipGemm: negative extent");
    // The gemm entry point blocks on the queue's stream; drain our own
    // pending event first so async mode keeps its ordering guarantees.
    c->synchronize();
    c->lastKernel = "mkl_gemm";
    auto fill = [&](auto &ref, const void *data, const int64_t s[2], int64_t d0,
                    int64_t d1) {
      ref.userData = nullptr;
      ref.data = static_cast<decltype(ref.data)>(const_cast<void *>(data));
      ref.offset = 0;
      ref.dims[0] = size_t(d0);
      ref.dims[1] = size_t(d1);
      ref.strides[0] = size_t(s[0]);
      ref.strides[1] = size_t(s[1]);
    };
    if (dtype == NMHIP_F32) {
      NmhipMemref2F32 ra, rb, rc;
      fill(ra, a, aS, m, k);
      fill(rb, b, bS, k, n);
      fill(rc, cPtr, cS, m, n);
      SYM(GemmF32, "mkl_gemm_float32_device")(c->queue, &ra, &rb, float(alpha),
                                              float(beta), &rc);
    } else if (dtype == NMHIP_F64) {
      NmhipMemref2F64 ra, rb, rc;
      fill(ra, a, aS, m, k);
      fill(rb, b, bS, k, n);
      fill(rc, cPtr, cS, m, n);
      SYM(GemmF64, "mkl_gemm_float64_device")(c->queue, &ra, &rb, alpha, beta,
                                              &rc);
    } else {
      fail("nmhipGemm: dtype must be float32 or float64");
    }
  });
}

NMHIP_EXPORT void nmhipSuggestBlockSize(void *ctx, const char *kernelName,
                                        const uint32_t *globalSize,
                                        uint32_t *blockSize, size_t numDims) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    SYM(SuggestBlockSize, "gpuxSuggestBlockSize")(
        c->queue, c->kernel(kernelName), globalSize, blockSize, numDims);
  });
}

NMHIP_EXPORT void nmhipLaunch(void *ctx, const char *kernelName,
                              const size_t grid[3], const size_t block[3],
                              GpuxParamDesc *params) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (!kernelName || !grid || !block || !params)
      fail("nmhipLaunch: null argument");
    c->launchDesc(kernelName, grid, block, params);
  });
}

NMHIP_EXPORT void nmhipPairwiseF64(void *ctx, const double *X1,
                                   const double *X2, double *D, int64_t n1,
                                   int64_t n2) {
  guarded([&]() {
    Context *c = toCtx(ctx);
    std::lock_guard<std::mutex> lock(c->mutex);
    if (n1 <= 0 || n2 <= 0)
      return;
    if (n2 % 2 != 0 || !aligned16(D))
      fail("nmhipPairwiseF64: needs an even n2 and a 16-byte aligned D");
    const int64_t gx = ceilDiv(n2, 512);
    int64_t rows = tuning().pairwiseRows;
    if (!rows) {
      // Two rows (8 KiB of D) per block: as for the row-broadcast map, many
      // short blocks stream stores best (78-81 us against 89 with four rows;
      // a store-only kernel of the same size takes 79).
      rows = 2;
      if (ceilDiv(n1, rows) > 65535)
        rows = ceilDiv(n1, 65535);
    }
    const int64_t gy = ceilDiv(n1, rows);
    if (gy > 65535)
      fail("nmhipPairwiseF64: too many row chunks");
    c->launch("nmk_twin_pairwise_f64_rows", size_t(gx), size_t(gy), 1, 256, 1, 1,
              {Arg::Ptr(X1), Arg::Ptr(X2), Arg::Ptr(D), Arg::I64(n1),
               Arg::I64(n2), Arg::I64(rows)});
  });
}

NMHIP_EXPORT const void *nmhipKernelBlob(const char *family, size_t *size) {
  return guarded([&]() -> const void * {
    const Blob *b = family ? findBlob(family) : nullptr;
    if (!b)
      fail("Unknown kernel family '%s'", family ? family : "(null)");
    if (size)
      *size = static_cast<size_t>(b->end - b->begin);
    return b->begin;
  });
}

NMHIP_EXPORT void nmhipSetTuning(const char *knob, int64_t value) {
  guarded([&]() {
    if (!knob)
      fail("nmhipSetTuning: null knob");
    Tuning &t = tuning();
    const std::string k(knob);
    if (k == "rowbcast_rows")
      t.rowbcastRows = value;
    else if (k == "map_blocks")
      t.mapBlocks = value;
    else if (k == "reduce_blocks")
      t.reduceBlocks = value;
    else if (k == "axis0_rows")
      t.axis0Rows = value;
    else if (k == "pairwise_rows")
      t.pairwiseRows = value;
    else if (k == "bs_blocks")
      t.bsBlocks = value;
    else if (k == "cols_blocks")
      t.colsBlocks = value;
    else if (k == "handoff_release")
      t.handoffRelease = value;
    else
      fail("Unknown tuning knob '%s'", knob);
  });
}
