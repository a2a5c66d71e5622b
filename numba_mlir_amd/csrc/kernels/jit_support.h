// Device-side support for kernels generated from Python @kernel bodies
// (numba_mlir_amd/mlir/kernel_compiler.py).  The generated source includes
// this header and nothing else; it is compiled for gfx950 on its own.
//
// What the reference's lowering provides as GPU-dialect ops and SPIR-V
// builtins (reference: numba_mlir/mlir_compiler/lib/pipelines/LowerToGpu.cpp:
// ids 1195-1265, atomics 1404-1465, barriers 1515-1553, group reductions
// 1564-1780, local/private arrays 1296-1386) are plain device functions here.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "erf_table.inc"
#include "erf_taylor.inc"
#include "fast_math.h"

namespace nmkjit {

// ---- array views ----------------------------------------------------------
// An N-d strided view: what a memref argument is unpacked into.  Strides are
// in elements.
template <typename T, int N> struct View {
  T *p;
  int64_t shape[N];
  int64_t stride[N];
};

// Compile-time switches handed to a generic lambda.
struct Yes {
  static constexpr bool value = true;
};
struct No {
  static constexpr bool value = false;
};

// Python index normalisation: a negative index counts from the end.
__device__ __forceinline__ int64_t wrap(int64_t i, int64_t n) {
  return i < 0 ? i + n : i;
}

// Bounds-checked builds: an index outside [0, n) raises the flag and is
// redirected to element 0, so the kernel finishes and the host can report it.
__device__ __forceinline__ int64_t checked(int64_t i, int64_t n, int *flag) {
  if (i < 0 || i >= n) {
    *flag = 1;
    return 0;
  }
  return i;
}

// v[i] on the leading dimension: the view of rank N - 1.
template <typename T, int N>
__device__ __forceinline__ View<T, N - 1> sub(const View<T, N> &v, int64_t i) {
  View<T, N - 1> r;
  r.p = v.p + i * v.stride[0];
#pragma unroll
  for (int k = 1; k < N; ++k) {
    r.shape[k - 1] = v.shape[k];
    r.stride[k - 1] = v.stride[k];
  }
  return r;
}

// The same on dimension `dim`.
template <typename T, int N>
__device__ __forceinline__ View<T, N - 1> subAt(const View<T, N> &v, int dim,
                                                int64_t i) {
  View<T, N - 1> r;
  r.p = v.p + i * v.stride[dim];
#pragma unroll
  for (int k = 0; k < N - 1; ++k) {
    r.shape[k] = v.shape[k < dim ? k : k + 1];
    r.stride[k] = v.stride[k < dim ? k : k + 1];
  }
  return r;
}

// v[..., start:stop:step, ...] on dimension `dim`, Python slice semantics;
// kNone marks an omitted bound.
constexpr int64_t kNone = INT64_MIN;

template <typename T, int N>
__device__ __forceinline__ View<T, N> slice(const View<T, N> &v, int dim,
                                            int64_t start, int64_t stop,
                                            int64_t step) {
  const int64_t n = v.shape[dim];
  if (step == kNone)
    step = 1;
  int64_t lo, hi;
  if (step > 0) {
    lo = start == kNone ? 0 : (start < 0 ? (start + n < 0 ? 0 : start + n) : (start > n ? n : start));
    hi = stop == kNone ? n : (stop < 0 ? (stop + n < 0 ? 0 : stop + n) : (stop > n ? n : stop));
  } else {
    lo = start == kNone ? n - 1 : (start < 0 ? (start + n < 0 ? -1 : start + n) : (start >= n ? n - 1 : start));
    hi = stop == kNone ? -1 : (stop < 0 ? (stop + n < 0 ? -1 : stop + n) : (stop >= n ? n - 1 : stop));
  }
  int64_t count = 0;
  if (step > 0 && hi > lo)
    count = (hi - lo + step - 1) / step;
  else if (step < 0 && hi < lo)
    count = (lo - hi - step - 1) / (-step);
  View<T, N> r = v;
  r.p = v.p + lo * v.stride[dim];
  r.shape[dim] = count;
  r.stride[dim] = v.stride[dim] * step;
  return r;
}

// ---- Python arithmetic ----------------------------------------------------
template <typename T> __device__ __forceinline__ T floordivInt(T a, T b) {
  if (b == 0)
    return 0;
  const T q = a / b;
  return ((a % b != 0) && ((a < 0) != (b < 0))) ? q - 1 : q;
}
template <typename T> __device__ __forceinline__ T modInt(T a, T b) {
  if (b == 0)
    return 0;
  const T r = a % b;
  return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r;
}
// CPython's float_divmod.
template <typename T> __device__ __forceinline__ T modFloat(T a, T b) {
  T m = fmod(a, b);
  if (m != T(0)) {
    if ((b < T(0)) != (m < T(0)))
      m += b;
  } else {
    m = copysign(T(0), b);
  }
  return m;
}
template <typename T> __device__ __forceinline__ T floordivFloat(T a, T b) {
  T m = fmod(a, b);
  T d = (a - m) / b;
  if (m != T(0) && ((b < T(0)) != (m < T(0))))
    d -= T(1);
  if (d != T(0)) {
    T f = floor(d);
    if (d - f > T(0.5))
      f += T(1);
    return f;
  }
  return copysign(T(0), a / b);
}
template <typename T> __device__ __forceinline__ T powInt(T base, T e) {
  if (e < 0)
    return base == 1 ? 1 : (base == -1 ? ((e & 1) ? -1 : 1) : 0);
  T r = 1;
  while (e > 0) {
    if (e & 1)
      r *= base;
    base *= base;
    e >>= 1;
  }
  return r;
}

// ---- atomics (return the old value) ---------------------------------------
__device__ __forceinline__ int32_t atomicAddT(int32_t *p, int32_t v) {
  return atomicAdd(p, v);
}
__device__ __forceinline__ int64_t atomicAddT(int64_t *p, int64_t v) {
  return int64_t(atomicAdd(reinterpret_cast<unsigned long long *>(p),
                           static_cast<unsigned long long>(v)));
}
__device__ __forceinline__ float atomicAddT(float *p, float v) {
  return atomicAdd(p, v);
}
__device__ __forceinline__ double atomicAddT(double *p, double v) {
  return atomicAdd(p, v);
}

// ---- work-group helpers ---------------------------------------------------
__device__ __forceinline__ int linearLocalId() {
  return threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z);
}
__device__ __forceinline__ int localCount() {
  return blockDim.x * blockDim.y * blockDim.z;
}

struct AddOp {
  template <typename T> __device__ T operator()(T a, T b) const { return a + b; }
};
struct MulOp {
  template <typename T> __device__ T operator()(T a, T b) const { return a * b; }
};
// (a NaN on either side loses, as in the group minimum / maximum of the
// reference's target, which skip NaNs)
struct MinOp {
  template <typename T> __device__ T operator()(T a, T b) const {
    return (b < a || a != a) ? b : a;
  }
};
struct MaxOp {
  template <typename T> __device__ T operator()(T a, T b) const {
    return (a < b || a != a) ? b : a;
  }
};

constexpr int kMaxGroup = 1024;

// Work-group reduction.  Work-items outside the global size never run the
// kernel body, so they cannot take part: before the body, every lane of the
// block (in or out) parks the neutral element in its slot (groupInit), and
// the block learns whether it is clipped.  A full block reduces by an LDS
// tree; a clipped block, whose members need not be a prefix of the linear
// ids, has every member fold all slots in order.
template <typename T>
__device__ __forceinline__ void groupInit(T *slots, T neutral) {
  slots[linearLocalId()] = neutral;
}

template <typename T, typename Op>
__device__ __forceinline__ T groupReduce(T *slots, T v, bool clipped, Op op) {
  const int tid = linearLocalId();
  const int n = localCount();
  __syncthreads(); // a previous call may still be reading the slots
  slots[tid] = v;
  __syncthreads();
  if (!clipped) {
    int s = 1;
    while (s < n)
      s <<= 1;
    for (s >>= 1; s > 0; s >>= 1) {
      if (tid < s && tid + s < n)
        slots[tid] = op(slots[tid], slots[tid + s]);
      __syncthreads();
    }
    return slots[0];
  }
  T r = slots[0];
  for (int i = 1; i < n; ++i)
    r = op(r, slots[i]);
  return r;
}

// Reduction of one value per lane over the whole block (every lane calls it,
// lanes outside the global size with the neutral element): lane 0 gets the
// block's result.  The tree is fixed by the block shape, so repeated launches
// give the same bits.
template <typename T, typename Op>
__device__ __forceinline__ T blockReduce(T v, Op op) {
  __shared__ T slots[kMaxGroup];
  const int tid = linearLocalId();
  const int n = localCount();
  __syncthreads(); // the slots may serve several reductions in a row
  slots[tid] = v;
  __syncthreads();
  int s = 1;
  while (s < n)
    s <<= 1;
  for (s >>= 1; s > 0; s >>= 1) {
    if (tid < s && tid + s < n)
      slots[tid] = op(slots[tid], slots[tid + s]);
    __syncthreads();
  }
  return slots[0];
}

// A launch's reduction variables finish on the device (the reference stores
// per-workgroup partial results to host-shared memory and adds them in a host
// loop, mlir/lib/Conversion/GpuToGpuRuntime.cpp:2161-2277).  Every block
// leaves its partial result at partial[block index] with a store that is
// visible device-wide once acknowledged; the block that draws the last ticket
// reads all of them back past its own caches, folds them -- a fixed tree over
// the block index, so repeated launches give the same bits -- and leaves the
// total at partial[number of blocks].  No value is accumulated with an
// atomic: the ticket only orders the blocks.
__device__ __forceinline__ int64_t blockCount() {
  return int64_t(gridDim.x) * gridDim.y * gridDim.z;
}

template <typename T, typename Op>
__device__ __forceinline__ void blockReduceStore(T v, Op op, T *partial) {
  const T total = blockReduce(v, op);
  if (linearLocalId() == 0)
    __hip_atomic_store(
        partial + (blockIdx.x + gridDim.x * (blockIdx.y + int64_t(gridDim.y) * blockIdx.z)),
        total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// After the blockReduceStore calls of a kernel: true in every lane of the
// block that arrived last (all partial results are then visible to it).
// Device-wide atomics on one 256-byte line of memory are served one after
// the other, about 7 ns each, and the blocks of a streaming kernel all end
// together: 2048 tickets from one counter, or from sixteen counters next to
// each other, add 16 us to a launch of 79 us.  So the tickets are drawn in
// two steps from counters 256 bytes apart: a block draws from one of
// kTicketGroups counters (its index modulo their number), and only the last
// of each group draws from the counter behind them (with that, 2 us).
// `ticket`: (kTicketGroups + 1) * kTicketStride counters, zero between
// launches (the block that empties a counter puts it back).
constexpr int kTicketGroups = 16;
constexpr int kTicketStride = 64; // counters 256 bytes apart

__device__ __forceinline__ bool drewLastTicket(uint32_t *ticket) {
  __shared__ uint32_t last;
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0); // the partial results are acknowledged
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __syncthreads();
  if (linearLocalId() == 0) {
    const int64_t blocks = blockCount();
    const int64_t me = blockIdx.x + gridDim.x * (blockIdx.y + int64_t(gridDim.y) * blockIdx.z);
    const int64_t group = me % kTicketGroups;
    const int64_t inGroup = (blocks - group + kTicketGroups - 1) / kTicketGroups;
    const int64_t groups = blocks < kTicketGroups ? blocks : kTicketGroups;
    uint32_t mine = __hip_atomic_fetch_add(ticket + group * kTicketStride, 1u, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
    last = 0u;
    if (mine == uint32_t(inGroup - 1)) {
      __hip_atomic_store(ticket + group * kTicketStride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      mine = __hip_atomic_fetch_add(ticket + kTicketGroups * kTicketStride, 1u, __ATOMIC_RELAXED,
                                    __HIP_MEMORY_SCOPE_AGENT);
      if (mine == uint32_t(groups - 1)) {
        __hip_atomic_store(ticket + kTicketGroups * kTicketStride, 0u, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        last = 1u;
      }
    }
  }
  __syncthreads();
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  return last != 0;
}

// In the last block: partial[number of blocks] = fold of partial[0 ..).
template <typename T, typename Op>
__device__ __forceinline__ void foldPartials(T *partial, Op op, T neutral) {
  const int64_t blocks = blockCount();
  const int64_t n = localCount();
  T acc = neutral;
  // (eight loads in flight a lane: each comes from beyond the caches)
  for (int64_t base = linearLocalId(); base < blocks; base += 8 * n) {
    T v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int64_t i = base + u * n;
      v[u] = i < blocks ? __hip_atomic_load(partial + i, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT)
                        : neutral;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      acc = op(acc, v[u]);
  }
  const T total = blockReduce(acc, op);
  if (linearLocalId() == 0)
    partial[blocks] = total;
}

// A store of a value that no work-item of the launch reads back.  `unit`:
// adjacent lanes write adjacent elements, so a wave completes whole lines in
// one instruction and they can stream past the caches; any other pattern is
// left to L2 to combine.  `unit` is uniform over the launch.
template <typename T>
__device__ __forceinline__ void streamStore(T *p, T v, bool unit) {
  if (unit)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}
__device__ __forceinline__ void streamStore(bool *p, bool v, bool) { *p = v; }

// ---- erf of a double ------------------------------------------------------
// Piecewise Taylor polynomials on a grid of 97 nodes 1/16 apart, coefficients
// in workgroup memory (erfTableLoad at kernel entry), |x| < 3/32 from the
// series of erf(x) / x: within 2 units in the last place (1 above |x| = 1/4),
// at a fifth of the device library's instructions, which pays for three
// ranges under divergence.  NaN stays NaN, |x| >= 6 gives +-1.
__shared__ double erfLds[NMK_ERFT_NODES * NMK_ERFT_COEFFS];

__device__ __forceinline__ void erfTableLoad() {
  for (int k = linearLocalId(); k < NMK_ERFT_NODES * NMK_ERFT_COEFFS; k += localCount())
    erfLds[k] = kErfTaylor[k];
  __syncthreads();
}

__device__ __forceinline__ double erfF64(double x) {
  const double ax = __builtin_fmin(__builtin_fabs(x), 6.0);
  double r;
  if (ax < 3.0 / 32) {
    const double small[NMK_ERFT_SMALL_TERMS] = {NMK_ERFT_SMALL_LIST};
    const double s = x * x;
    double q = small[NMK_ERFT_SMALL_TERMS - 1];
#pragma unroll
    for (int j = NMK_ERFT_SMALL_TERMS - 2; j >= 0; --j)
      q = __builtin_fma(q, s, small[j]);
    r = x * q;
  } else {
    // one unit in the last place of ax + 1.5 * 2^48 is 1/16: the low word
    // of the sum is the nearest node, the rest of the sum its position
    const double t = ax + 0x1.8p48;
    const int node = __double2loint(t);
    const double u = ax - (t - 0x1.8p48);
    const double *c = erfLds + node * NMK_ERFT_COEFFS;
    double p = c[NMK_ERFT_COEFFS - 1];
#pragma unroll
    for (int j = NMK_ERFT_COEFFS - 2; j >= 0; --j)
      p = __builtin_fma(p, u, c[j]);
    r = __builtin_copysign(p, x);
  }
  return x != x ? x : r;
}

// ---- 0.5 + 0.5 * erf(x) of a double ----------------------------------------
// The normal distribution's cdf term as one operation: a degree-5 polynomial
// for erf / 2 around the nearest of 97 nodes 1/16 apart (absolute error of
// erf 1.5e-12), the node's 48-byte row read from workgroup memory in three
// 128-bit words (cdfTableLoad at kernel entry).  Halving is exact, so the sum
// rounds as 0.5 + 0.5 * erf(x) would.  NaN stays NaN.
typedef double cdf_word __attribute__((ext_vector_type(2)));
__shared__ __attribute__((aligned(16))) cdf_word cdfLds[NMK_ERF_NODES * 3];

__device__ __forceinline__ void cdfTableLoad() {
  static_assert(NMK_ERF_COEFFS == 6 && NMK_ERF_ROW == 6, "three 128-bit words a row");
  const cdf_word *src = reinterpret_cast<const cdf_word *>(kHalfErfTable);
  for (int k = linearLocalId(); k < NMK_ERF_NODES * 3; k += localCount())
    cdfLds[k] = src[k];
  __syncthreads();
}

__device__ __forceinline__ double cdfTermF64(double x) {
  const double ax = __builtin_fmin(__builtin_fabs(x), 6.0);
  const double t = ax + 0x1.8p48; // low word: the nearest sixteenth, 0..96
  const int node = __double2loint(t);
  const double u = ax - (t - 0x1.8p48);
  const cdf_word *row = cdfLds + __mul24(node, 3);
  const cdf_word c01 = row[0], c23 = row[1], c45 = row[2];
  double p = c45[1];
  p = __builtin_fma(p, u, c45[0]);
  p = __builtin_fma(p, u, c23[1]);
  p = __builtin_fma(p, u, c23[0]);
  p = __builtin_fma(p, u, c01[1]);
  p = __builtin_fma(p, u, c01[0]);
  const double r = 0.5 + __builtin_copysign(p, x);
  return x != x ? x : r;
}

// ---- speculation on everyday operands ---------------------------------------
// A fused map that gives a lane four adjacent elements computes them first
// with the routines' plain forms -- the library's own arithmetic without its
// range handling, bit-identical wherever the operand is in range -- while
// each such call clears `ok` if its operand is out of range.  The stores come
// last, so a wave in which any lane saw such an operand simply computes its
// elements again with the general routines (CAREFUL) before anything is
// written.  One wave-uniform branch per four elements replaces a divergent
// branch per call.
// Whether a double is positive with an exponent in [-900, 900): one unsigned
// comparison of its high word (negative numbers, NaNs, infinities, zero and
// denormals all fall outside).
__device__ __forceinline__ bool midRangeF64(double z) {
  return (uint32_t(__double2hiint(z)) - (123u << 20)) < (1800u << 20);
}

// (The tests are combined with & so that the plain form stays one basic
// block.)
template <bool CAREFUL> __device__ __forceinline__ float logF32m(float q, bool &ok) {
  if (CAREFUL)
    return logf(q);
  ok = ok & ((__float_as_uint(q) - 0x03800000u) < 0x78000000u); // normal, positive
  return nmk::logNormalF32(q);
}
template <bool CAREFUL> __device__ __forceinline__ float expF32m(float b, bool &ok) {
  if (CAREFUL)
    return expf(b);
  ok = ok & (__builtin_fabsf(b) <= 80.0f);
  return nmk::expNormalF32(b);
}
template <bool CAREFUL>
__device__ __forceinline__ float logQuotientF32m(float a, float b, bool &ok) {
  if (CAREFUL)
    return logf(a / b);
  ok = ok & nmk::quotientIsPlainF32(a, b);
  return nmk::logNormalF32(nmk::divNormalF32(a, b));
}
template <bool CAREFUL> __device__ __forceinline__ double rsqrtF64m(double z, bool &ok) {
  if (CAREFUL)
    return nmk::rsqrtF64(z);
  ok = ok & midRangeF64(z);
  const double y = __builtin_amdgcn_rsq(z);
  const double e = __builtin_fma(-z, y * y, 1.0); // 1 - z y^2
  return __builtin_fma(y * e, __builtin_fma(0.375, e, 0.5), y);
}
// (plain form: the polynomial of a NaN is some number, so a NaN sends the
// wave to the careful form instead of being put back by a select)
template <bool CAREFUL> __device__ __forceinline__ double cdfTermF64m(double x, bool &ok) {
  if (CAREFUL)
    return cdfTermF64(x);
  ok = ok & (x == x);
  const double ax = __builtin_fmin(__builtin_fabs(x), 6.0);
  const double t = ax + 0x1.8p48;
  const int node = __double2loint(t);
  const double u = ax - (t - 0x1.8p48);
  const cdf_word *row = cdfLds + __mul24(node, 3);
  const cdf_word c01 = row[0], c23 = row[1], c45 = row[2];
  double p = c45[1];
  p = __builtin_fma(p, u, c45[0]);
  p = __builtin_fma(p, u, c23[1]);
  p = __builtin_fma(p, u, c23[0]);
  p = __builtin_fma(p, u, c01[1]);
  p = __builtin_fma(p, u, c01[0]);
  return 0.5 + __builtin_copysign(p, x);
}
template <bool CAREFUL> __device__ __forceinline__ double sqrtF64m(double d, bool &ok) {
  if (CAREFUL)
    return sqrt(d);
  ok = ok & midRangeF64(d);
  const double y = __builtin_amdgcn_rsq(d);
  double g = d * y;
  double h = 0.5 * y;
  const double r = __builtin_fma(-h, g, 0.5);
  g = __builtin_fma(g, r, g);
  h = __builtin_fma(h, r, h);
  const double e = __builtin_fma(-g, g, d);
  return __builtin_fma(e, h, g);
}

} // namespace nmkjit
