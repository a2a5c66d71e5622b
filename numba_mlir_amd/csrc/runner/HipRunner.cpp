// hip-runner: runs the reference's end-to-end runner cases against a gpux*
// runtime, with no Python and no compiler in the process.
//
// The reference's runner (mlir/tools/level_zero_runner/LevelZeroRunner.cpp:
// 39-135) JIT-compiles an .mlir file through its GPU pipeline and executes
// `main` against the runtime libraries named by -shared-libs; the files under
// mlir/test/L0_RUNNER pipe its output into FileCheck.  There is no MLIR here,
// so this runner carries each of those programs already lowered: the host
// side below is the call sequence the lowering emits (stream and module
// created once, per kernel launch -> wait -> destroy event,
// mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:444-628), the device side is
// runner_kernels.hip.  Everything else is the reference runner's contract:
//
//   hip-runner <case | path/to/<case>.mlir> -e main -entry-point-result=void
//              -shared-libs=<lib>[,<lib>...] [-shared-libs=...]
//
// The runtime is reached only through the thirteen gpux* symbols resolved
// from the -shared-libs libraries (a library without them is an error), and
// the result is printed the way the MLIR runner utilities' printMemrefF32 /
// printMemrefF64 print a memref, so the CHECK lines of the reference's files
// apply to the output unchanged.  `hip-runner --list` names the cases.
#include "numba_mlir_hip/GpuRuntime.h"

#include <dlfcn.h>

#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <iostream>
#include <map>
#include <string>
#include <vector>

extern "C" const unsigned char hip_runner_blob[];
extern "C" const unsigned char hip_runner_blob_end[];

namespace {

[[noreturn]] void die(const std::string &msg) {
  std::fprintf(stderr, "hip-runner: %s\n", msg.c_str());
  std::exit(1);
}

// ---- the runtime, by name -------------------------------------------------
struct Runtime {
  decltype(&gpuxQueueCreate) queueCreate;
  decltype(&gpuxQueueDestroy) queueDestroy;
  decltype(&gpuxModuleLoad) moduleLoad;
  decltype(&gpuxModuleDestroy) moduleDestroy;
  decltype(&gpuxKernelGet) kernelGet;
  decltype(&gpuxKernelDestroy) kernelDestroy;
  decltype(&gpuxLaunchKernel) launchKernel;
  decltype(&gpuxWait) wait;
  decltype(&gpuxDestroyEvent) destroyEvent;
  decltype(&gpuxAlloc) alloc;
  decltype(&gpuxDeAlloc) deAlloc;
  decltype(&gpuxSuggestBlockSize) suggestBlockSize;
  decltype(&gpuxDuplicateQueue) duplicateQueue;
};

void *findSymbol(const std::vector<void *> &libs, const char *name) {
  for (void *lib : libs)
    if (void *sym = dlsym(lib, name))
      return sym;
  return nullptr;
}

Runtime bindRuntime(const std::vector<void *> &libs) {
  Runtime rt{};
  std::string missing;
  auto bind = [&](auto &slot, const char *name) {
    void *sym = findSymbol(libs, name);
    if (!sym)
      missing += std::string(missing.empty() ? "" : ", ") + name;
    slot = reinterpret_cast<std::remove_reference_t<decltype(slot)>>(sym);
  };
  bind(rt.queueCreate, "gpuxQueueCreate");
  bind(rt.queueDestroy, "gpuxQueueDestroy");
  bind(rt.moduleLoad, "gpuxModuleLoad");
  bind(rt.moduleDestroy, "gpuxModuleDestroy");
  bind(rt.kernelGet, "gpuxKernelGet");
  bind(rt.kernelDestroy, "gpuxKernelDestroy");
  bind(rt.launchKernel, "gpuxLaunchKernel");
  bind(rt.wait, "gpuxWait");
  bind(rt.destroyEvent, "gpuxDestroyEvent");
  bind(rt.alloc, "gpuxAlloc");
  bind(rt.deAlloc, "gpuxDeAlloc");
  bind(rt.suggestBlockSize, "gpuxSuggestBlockSize");
  bind(rt.duplicateQueue, "gpuxDuplicateQueue");
  if (!missing.empty())
    die("the -shared-libs libraries do not export " + missing);
  return rt;
}

// ---- a lowered program's view of the runtime --------------------------------
struct Arg {
  enum Kind { Ptr, I32, I64 } kind;
  union {
    void *p;
    int32_t i32;
    int64_t i64;
  };
  static Arg ptr(const void *v) {
    Arg a;
    a.kind = Ptr;
    a.p = const_cast<void *>(v);
    return a;
  }
  static Arg i(int32_t v) {
    Arg a;
    a.kind = I32;
    a.i32 = v;
    return a;
  }
  static Arg l(int64_t v) {
    Arg a;
    a.kind = I64;
    a.i64 = v;
    return a;
  }
};

class Program {
public:
  explicit Program(const Runtime &runtime) : rt(runtime) {
    const char *device = std::getenv("HIP_RUNNER_DEVICE"); // NULL: the default
    queue = rt.queueCreate(device);
    module = rt.moduleLoad(queue, hip_runner_blob,
                           size_t(hip_runner_blob_end - hip_runner_blob));
  }
  ~Program() {
    for (void *p : buffers)
      rt.deAlloc(queue, p);
    for (auto &k : kernels)
      rt.kernelDestroy(k.second);
    rt.moduleDestroy(module);
    rt.queueDestroy(queue);
  }

  // memref.alloc of a buffer the kernels touch: host-dereferenceable and
  // device-accessible, 64-byte aligned (GpuRuntimeToLlvm.cpp:670); the
  // allocation's event is waited for and destroyed at once (741-744).
  template <typename T> T *alloc(size_t count) {
    void *noDeps[1] = {nullptr};
    GpuxAllocResult res{};
    rt.alloc(queue, count * sizeof(T), 64, GPUX_ALLOC_SHARED, noDeps, &res);
    rt.wait(queue, res.event);
    rt.destroyEvent(queue, res.event);
    if (!res.ptr && count)
      die("gpuxAlloc returned no memory");
    buffers.push_back(res.ptr);
    return static_cast<T *>(res.ptr);
  }

  // gpu.launch_func without an async token: launch, wait, destroy event.
  void launch(const char *name, size_t gx, size_t gy, size_t gz,
              const std::vector<Arg> &args) {
    void *&kernel = kernels[name];
    if (!kernel)
      kernel = rt.kernelGet(module, name);
    std::vector<GpuxParamDesc> params(args.size() + 1);
    for (size_t k = 0; k < args.size(); ++k) {
      const Arg &a = args[k];
      params[k].data = &a.p; // (the union's members share their address)
      params[k].size = a.kind == Arg::I32 ? 4 : 8;
      params[k].type = a.kind == Arg::Ptr   ? GPUX_PARAM_PTR
                       : a.kind == Arg::I32 ? GPUX_PARAM_INT32
                                            : GPUX_PARAM_INT64;
    }
    params[args.size()] = GpuxParamDesc{nullptr, 0, GPUX_PARAM_NULL};
    void *noDeps[1] = {nullptr};
    void *event = rt.launchKernel(queue, kernel, gx, gy, gz, 1, 1, 1, noDeps,
                                  params.data());
    rt.wait(queue, event);
    rt.destroyEvent(queue, event);
  }

private:
  const Runtime &rt;
  void *queue = nullptr;
  void *module = nullptr;
  std::map<std::string, void *> kernels;
  std::vector<void *> buffers;
};

// ---- printMemrefF32 / printMemrefF64 ----------------------------------------
// The format of the MLIR runner utilities: a line of metadata, then the
// elements as nested bracketed lists, one innermost row per line, numbers
// through a default-formatted ostream (six significant digits).
template <typename T>
void printData(std::ostream &os, const T *base, int64_t dim, int64_t rank,
               int64_t offset, const int64_t *sizes, const int64_t *strides) {
  if (dim == 0) {
    os << base[offset];
    return;
  }
  auto spaces = [&](int64_t n) {
    for (int64_t k = 0; k < n; ++k)
      os << " ";
  };
  os << "[";
  printData(os, base, dim - 1, rank, offset, sizes + 1, strides + 1);
  if (sizes[0] <= 1) {
    os << "]";
    return;
  }
  os << ", ";
  if (dim > 1)
    os << "\n";
  for (int64_t i = 1; i + 1 < sizes[0]; ++i) {
    spaces(rank - dim + 1);
    printData(os, base, dim - 1, rank, offset + i * strides[0], sizes + 1,
              strides + 1);
    os << ", ";
    if (dim > 1)
      os << "\n";
  }
  spaces(rank - dim + 1);
  printData(os, base, dim - 1, rank, offset + (sizes[0] - 1) * strides[0],
            sizes + 1, strides + 1);
  os << "]";
}

template <typename T>
void printMemref(const T *data, const std::vector<int64_t> &sizes) {
  const int64_t rank = int64_t(sizes.size());
  std::vector<int64_t> strides(sizes.size(), 1);
  for (int64_t k = rank - 2; k >= 0; --k)
    strides[k] = strides[k + 1] * sizes[k + 1];
  char base[32];
  std::snprintf(base, sizeof(base), "0x%" PRIxPTR, reinterpret_cast<uintptr_t>(data));
  std::ostream &os = std::cout;
  os << "Unranked Memref base@ = " << base << " rank = " << rank << " offset = 0";
  auto list = [&](const std::vector<int64_t> &v) {
    for (size_t k = 0; k < v.size(); ++k)
      os << (k ? ", " : "") << v[k];
  };
  os << " sizes = [";
  list(sizes);
  os << "] strides = [";
  list(strides);
  os << "] data = " << std::endl;
  if (rank == 0)
    os << "[";
  printData(os, data, rank, rank, 0, sizes.data(), strides.data());
  if (rank == 0)
    os << "]";
  os << std::endl;
}

// ---- the cases ---------------------------------------------------------------
enum { ADD = 0, SUB = 1, MUL = 2, DIV = 3 }; // runner_kernels.hip
enum { YIELD = 0, NEG = 1, EXP = 2 };

// mlir/test/L0_RUNNER/addf.mlir: three memref<8xf32>, filled with 1.1, 2.2
// and 0; gpu.launch over 8 blocks of one thread adds them.
void caseAddf(Program &p) {
  float *a = p.alloc<float>(8), *b = p.alloc<float>(8), *c = p.alloc<float>(8);
  for (int k = 0; k < 8; ++k) {
    a[k] = 1.1f;
    b[k] = 2.2f;
    c[k] = 0.0f;
  }
  p.launch("rk_addf_blocks_f32", 8, 1, 1, {Arg::ptr(a), Arg::ptr(b), Arg::ptr(c)});
  printMemref(c, {8});
}

// linalg_addf.mlir: one all-parallel linalg.generic over tensor<2x5xf32>.
void caseLinalgAddf(Program &p) {
  const float av[10] = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10};
  const float bv[10] = {10, 9, 8, 7, 6, 5, 4, 3, 2, 1};
  float *a = p.alloc<float>(10), *b = p.alloc<float>(10), *out = p.alloc<float>(10);
  std::memcpy(a, av, sizeof(av));
  std::memcpy(b, bv, sizeof(bv));
  p.launch("rk_map2_f32", 2, 5, 1,
           {Arg::i(ADD), Arg::ptr(a), Arg::l(5), Arg::l(1), Arg::ptr(b), Arg::l(5),
            Arg::l(1), Arg::ptr(out), Arg::l(5), Arg::l(1)});
  printMemref(out, {2, 5});
}

// linalg_gemvf.mlir: y[i] += A[i, j] x[j], the result buffer starts as y.
void caseLinalgGemvf(Program &p) {
  const float av[9] = {1.0f, 0.5f, 1.0f, 1.0f, 1.0f, 1.0f, 1.0f, 0.6f, 1.0f};
  float *a = p.alloc<float>(9), *x = p.alloc<float>(3), *y = p.alloc<float>(3);
  std::memcpy(a, av, sizeof(av));
  for (int k = 0; k < 3; ++k)
    x[k] = y[k] = 1.0f;
  p.launch("rk_gemv_f32", 3, 1, 1,
           {Arg::ptr(a), Arg::l(3), Arg::ptr(x), Arg::ptr(y), Arg::l(3)});
  printMemref(y, {3});
}

// linalg_gemmf.mlir: C[i, j] += A[i, k] B[k, j] on 3x3 operands, C starts as ones.
void caseLinalgGemmf(Program &p) {
  const float av[9] = {0.5f, 0.2f, 4.0f, 1.0f, 1.0f, 2.0f, 3.0f, 3.0f, 0.3f};
  const float bv[9] = {1.0f, 2.0f, 3.0f, 3.0f, 4.0f, 0.5f, 3.0f, 3.0f, 3.0f};
  float *a = p.alloc<float>(9), *b = p.alloc<float>(9), *c = p.alloc<float>(9);
  std::memcpy(a, av, sizeof(av));
  std::memcpy(b, bv, sizeof(bv));
  for (int k = 0; k < 9; ++k)
    c[k] = 1.0f;
  p.launch("rk_gemm_f32", 3, 3, 1,
           {Arg::ptr(a), Arg::l(3), Arg::ptr(b), Arg::l(3), Arg::ptr(c), Arg::l(3),
            Arg::l(3)});
  printMemref(c, {3, 3});
}

// OpTest.ExplicitPadding.mlir: a 2x3 tensor written into a zero-filled 6x5
// one at offset (2, 1).
void caseExplicitPadding(Program &p) {
  float *in = p.alloc<float>(6), *out = p.alloc<float>(30);
  for (int k = 0; k < 6; ++k)
    in[k] = float(k + 1);
  for (int k = 0; k < 30; ++k)
    out[k] = 0.0f; // linalg.fill
  p.launch("rk_explicit_padding_f32", 2, 3, 1,
           {Arg::ptr(in), Arg::l(3), Arg::ptr(out), Arg::l(5)});
  printMemref(out, {6, 5});
}

// linalg_test_f32.mlir / linalg_test_f64.mlir: @foo(ones(500), [5, 4, 3, 2, 1]),
// nineteen linalg.generic ops.  The rank-0 ones have no parallel dimension
// and stay on the host; every rank-1 one is a launch of its own over 500
// iterations with a freshly allocated result (tensor.empty).
template <typename T> void caseLinalgTest(Program &p, const char *suffix) {
  const int64_t n = 500;
  const std::string map1 = std::string("rk_map1_") + suffix;
  const std::string map2 = std::string("rk_map2_") + suffix;
  T *arg0 = p.alloc<T>(n), *arg1 = p.alloc<T>(5);
  for (int64_t k = 0; k < n; ++k)
    arg0[k] = T(1);
  for (int k = 0; k < 5; ++k)
    arg1[k] = T(5 - k);
  T *scalars = p.alloc<T>(3);
  T *v11 = scalars, *v13 = scalars + 1, *v15 = scalars + 2;
  *v11 = arg1[0] + arg1[1]; // %11
  *v13 = arg1[4] - arg1[3]; // %13
  *v15 = -arg1[2];          // %15
  auto broadcast = [&](const T *scalar) { // (d0) -> () into (d0) -> (d0)
    T *out = p.alloc<T>(n);
    p.launch(map1.c_str(), n, 1, 1,
             {Arg::i(YIELD), Arg::ptr(scalar), Arg::l(0), Arg::l(0), Arg::ptr(out),
              Arg::l(1), Arg::l(0)});
    return out;
  };
  auto unary = [&](int op, const T *a) {
    T *out = p.alloc<T>(n);
    p.launch(map1.c_str(), n, 1, 1,
             {Arg::i(op), Arg::ptr(a), Arg::l(1), Arg::l(0), Arg::ptr(out), Arg::l(1),
              Arg::l(0)});
    return out;
  };
  auto binary = [&](int op, const T *a, const T *b) {
    T *out = p.alloc<T>(n);
    p.launch(map2.c_str(), n, 1, 1,
             {Arg::i(op), Arg::ptr(a), Arg::l(1), Arg::l(0), Arg::ptr(b), Arg::l(1),
              Arg::l(0), Arg::ptr(out), Arg::l(1), Arg::l(0)});
    return out;
  };
  T *t17 = broadcast(arg1 + 0);
  T *t19 = binary(SUB, arg0, t17);
  T *t21 = broadcast(v15);
  T *t23 = binary(MUL, t21, t19);
  T *t25 = unary(EXP, t23);
  T *t27 = binary(ADD, t25, arg0);
  T *t29 = broadcast(v13);
  T *t31 = binary(DIV, t29, t27);
  T *t33 = broadcast(arg1 + 3);
  T *t35 = binary(ADD, t33, t31);
  T *t37 = broadcast(arg1 + 0);
  T *t39 = binary(SUB, arg0, t37);
  T *t41 = binary(MUL, t35, t39);
  T *t43 = broadcast(v11);
  T *t45 = binary(ADD, t43, t41);
  printMemref(t45, {n});
}

struct Case {
  const char *name;
  const char *source; // the reference file it restates
  std::function<void(Program &)> run;
};

const std::vector<Case> &cases() {
  static const std::vector<Case> table = {
      {"addf", "mlir/test/L0_RUNNER/addf.mlir", caseAddf},
      {"linalg_addf", "mlir/test/L0_RUNNER/linalg_addf.mlir", caseLinalgAddf},
      {"linalg_gemvf", "mlir/test/L0_RUNNER/linalg_gemvf.mlir", caseLinalgGemvf},
      {"linalg_gemmf", "mlir/test/L0_RUNNER/linalg_gemmf.mlir", caseLinalgGemmf},
      {"linalg_test_f32", "mlir/test/L0_RUNNER/linalg_test_f32.mlir",
       [](Program &p) { caseLinalgTest<float>(p, "f32"); }},
      {"linalg_test_f64", "mlir/test/L0_RUNNER/linalg_test_f64.mlir",
       [](Program &p) { caseLinalgTest<double>(p, "f64"); }},
      {"OpTest.ExplicitPadding", "mlir/test/L0_RUNNER/OpTest.ExplicitPadding.mlir",
       caseExplicitPadding},
  };
  return table;
}

// "dir/linalg_addf.mlir" -> "linalg_addf"
std::string caseName(std::string arg) {
  const size_t slash = arg.find_last_of('/');
  if (slash != std::string::npos)
    arg = arg.substr(slash + 1);
  const std::string ext = ".mlir";
  if (arg.size() > ext.size() && arg.compare(arg.size() - ext.size(), ext.size(), ext) == 0)
    arg.resize(arg.size() - ext.size());
  return arg;
}

} // namespace

int main(int argc, char **argv) {
  std::string which, entry = "main", result = "void";
  std::vector<std::string> libPaths;
  for (int k = 1; k < argc; ++k) {
    std::string a = argv[k];
    while (a.size() > 2 && a[0] == '-' && a[1] == '-')
      a.erase(0, 1); // --flag and -flag are the same flag
    auto value = [&](const char *flag, std::string &out) {
      const std::string f(flag);
      if (a == f) {
        if (++k >= argc)
          die("missing value after " + f);
        out = argv[k];
        return true;
      }
      if (a.compare(0, f.size() + 1, f + "=") == 0) {
        out = a.substr(f.size() + 1);
        return true;
      }
      return false;
    };
    std::string v;
    if (a == "-list") {
      for (const Case &c : cases())
        std::printf("%s\t%s\n", c.name, c.source);
      return 0;
    } else if (value("-e", entry) || value("-entry-point-result", result)) {
    } else if (value("-shared-libs", v)) {
      size_t start = 0;
      while (start <= v.size()) {
        const size_t comma = v.find(',', start);
        const std::string one = v.substr(start, comma == std::string::npos ? comma : comma - start);
        if (!one.empty())
          libPaths.push_back(one);
        if (comma == std::string::npos)
          break;
        start = comma + 1;
      }
    } else if (!a.empty() && a[0] == '-') {
      die("unknown option " + std::string(argv[k]));
    } else if (which.empty()) {
      which = caseName(a);
    } else {
      die("more than one input: " + which + ", " + a);
    }
  }
  if (which.empty())
    die("no input (a case name or the path of the reference's .mlir file; --list "
        "names the cases)");
  if (entry != "main")
    die("entry point '" + entry + "' not found (the cases define main)");
  if (result != "void")
    die("-entry-point-result=" + result + ": main returns void");
  const Case *chosen = nullptr;
  for (const Case &c : cases())
    if (which == c.name)
      chosen = &c;
  if (!chosen)
    die("unknown case '" + which + "' (--list names the cases)");
  if (libPaths.empty())
    die("no -shared-libs: name the gpux* runtime library");
  std::vector<void *> libs;
  for (const std::string &path : libPaths) {
    void *lib = dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL);
    if (!lib)
      die(std::string("cannot load ") + path + ": " + dlerror());
    libs.push_back(lib);
  }
  const Runtime rt = bindRuntime(libs);
  {
    Program program(rt);
    chosen->run(program);
  }
  std::cout.flush();
  return 0;
}
