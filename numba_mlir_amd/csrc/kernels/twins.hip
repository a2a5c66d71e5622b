// Hand-written gfx950 twins of user @kernel functions.
//
// In the reference a @kernel body is compiled to a GPU kernel whose launch
// covers the global size with ceil(global/local) blocks per dimension, the
// tail guarded in-kernel, dimension 0 mapped to x
// (reference: numba_mlir/numba_mlir/mlir/kernel_impl.py:97-196,
// mlir_compiler/lib/pipelines/LowerToGpu.cpp:1113-1137).  A twin is the same
// body written in HIP.
//
// Twin argument convention (positional, as the launcher flattens them):
//   for every array argument: pointer, shape[0..rank), strides[0..rank)
//     (int64 element counts);
//   for every scalar argument: its value (int64 / float64 / float32 ...);
//   then the global size of the launch: gs0, gs1, gs2 (int64, 1 if unused).
// get_global_id(k) = blockIdx.k * blockDim.k + threadIdx.k.
#include "common.h"

using namespace nmk;

namespace {

struct Ids {
  int64_t g[3]; // get_global_id
  int64_t l[3]; // get_local_id
  int64_t b[3]; // get_group_id
  int64_t ls[3]; // get_local_size
  bool inside;
};

__device__ __forceinline__ Ids ids(int64_t gs0, int64_t gs1, int64_t gs2) {
  Ids r;
  r.l[0] = threadIdx.x;
  r.l[1] = threadIdx.y;
  r.l[2] = threadIdx.z;
  r.b[0] = blockIdx.x;
  r.b[1] = blockIdx.y;
  r.b[2] = blockIdx.z;
  r.ls[0] = blockDim.x;
  r.ls[1] = blockDim.y;
  r.ls[2] = blockDim.z;
  for (int k = 0; k < 3; ++k)
    r.g[k] = r.b[k] * r.ls[k] + r.l[k];
  r.inside = r.g[0] < gs0 && r.g[1] < gs1 && r.g[2] < gs2;
  return r;
}

} // namespace

// ---------------------------------------------------------------------------
// Index builtins (bodies: reference numba_mlir/numba_mlir/mlir/tests/test_gpu.py:580-803).
//   rank 1: c[i]       = v0
//   rank 2: c[i, j]    = v0 + v1 * 100
//   rank 3: c[i, j, k] = v0 + v1 * 100 + v2 * 10000
// where v is the global id, local id, group id, global size or local size.
#define NMK_TWIN_ID(NAME, V0, V1, V2)                                          \
  NMK_KERNEL(256)                                                              \
  nmk_twin_##NAME##_1(int32_t *c, int64_t n0, int64_t s0, int64_t gs0,         \
                      int64_t gs1, int64_t gs2) {                              \
    Ids t = ids(gs0, gs1, gs2);                                                \
    if (t.inside)                                                              \
      c[t.g[0] * s0] = int32_t(V0);                                            \
  }                                                                            \
  NMK_KERNEL(256)                                                              \
  nmk_twin_##NAME##_2(int32_t *c, int64_t n0, int64_t n1, int64_t s0,          \
                      int64_t s1, int64_t gs0, int64_t gs1, int64_t gs2) {     \
    Ids t = ids(gs0, gs1, gs2);                                                \
    if (t.inside)                                                              \
      c[t.g[0] * s0 + t.g[1] * s1] = int32_t(V0 + V1 * 100);                   \
  }                                                                            \
  NMK_KERNEL(256)                                                              \
  nmk_twin_##NAME##_3(int32_t *c, int64_t n0, int64_t n1, int64_t n2,          \
                      int64_t s0, int64_t s1, int64_t s2, int64_t gs0,         \
                      int64_t gs1, int64_t gs2) {                              \
    Ids t = ids(gs0, gs1, gs2);                                                \
    if (t.inside)                                                              \
      c[t.g[0] * s0 + t.g[1] * s1 + t.g[2] * s2] =                             \
          int32_t(V0 + V1 * 100 + V2 * 10000);                                 \
  }

NMK_TWIN_ID(get_global_id, t.g[0], t.g[1], t.g[2])
NMK_TWIN_ID(get_local_id, t.l[0], t.l[1], t.l[2])
NMK_TWIN_ID(get_group_id, t.b[0], t.b[1], t.b[2])
NMK_TWIN_ID(get_global_size, gs0, gs1, gs2)
NMK_TWIN_ID(get_local_size, t.ls[0], t.ls[1], t.ls[2])

// ---------------------------------------------------------------------------
// b[i] = f(a[i]), i = get_global_id(0)  (test_gpu.py:524-548).
#define NMK_TWIN_UNARY(OP, TNAME, T, EXPR)                                     \
  NMK_KERNEL(256)                                                              \
  nmk_twin_unary_##OP##_##TNAME(const T *a, int64_t an, int64_t as, T *b,      \
                                int64_t bn, int64_t bs, int64_t gs0,           \
                                int64_t gs1, int64_t gs2) {                    \
    Ids t = ids(gs0, gs1, gs2);                                                \
    if (t.inside) {                                                            \
      const T x = a[t.g[0] * as];                                              \
      b[t.g[0] * bs] = EXPR;                                                   \
    }                                                                          \
  }

NMK_TWIN_UNARY(sqrt, f32, float, sqrtf(x))
NMK_TWIN_UNARY(log, f32, float, logf(x))
NMK_TWIN_UNARY(exp, f32, float, expf(x))
NMK_TWIN_UNARY(sin, f32, float, sinf(x))
NMK_TWIN_UNARY(cos, f32, float, cosf(x))
NMK_TWIN_UNARY(erf, f32, float, erff(x))
NMK_TWIN_UNARY(tanh, f32, float, tanhf(x))
NMK_TWIN_UNARY(floor, f32, float, floorf(x))
NMK_TWIN_UNARY(ceil, f32, float, ceilf(x))
NMK_TWIN_UNARY(acos, f32, float, acosf(x))
NMK_TWIN_UNARY(sqrt, f64, double, sqrt(x))
NMK_TWIN_UNARY(log, f64, double, log(x))
NMK_TWIN_UNARY(exp, f64, double, exp(x))
NMK_TWIN_UNARY(sin, f64, double, sin(x))
NMK_TWIN_UNARY(cos, f64, double, cos(x))
NMK_TWIN_UNARY(erf, f64, double, erf(x))
NMK_TWIN_UNARY(tanh, f64, double, tanh(x))
NMK_TWIN_UNARY(floor, f64, double, floor(x))
NMK_TWIN_UNARY(ceil, f64, double, ceil(x))
NMK_TWIN_UNARY(acos, f64, double, acos(x))

// ---------------------------------------------------------------------------
// Pairwise Euclidean distance (body: test_gpu.py:1397-1408):
//   i = get_global_id(0); j = get_global_id(1)
//   d = 0.0
//   for k in range(X1.shape[1]): tmp = X1[i, k] - X2[j, k]; d += tmp * tmp
//   D[i, j] = sqrt(d)
// `d` is float64 whatever the array dtype; `tmp` has the array dtype.

// Faithful mapping: one work-item per (i, j), x <-> i.  Adjacent lanes write
// D with a stride of one row; kept as the literal twin of the user's mapping.
template <typename T>
__device__ __forceinline__ void
pairwiseFaithful(const T *X1, int64_t x1r, int64_t x1c, int64_t x1s0,
                 int64_t x1s1, const T *X2, int64_t x2r, int64_t x2c,
                 int64_t x2s0, int64_t x2s1, T *D, int64_t dr, int64_t dc,
                 int64_t ds0, int64_t ds1, int64_t gs0, int64_t gs1,
                 int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  if (!t.inside)
    return;
  const int64_t i = t.g[0], j = t.g[1];
  double d = 0.0;
  for (int64_t k = 0; k < x1c; ++k) {
    T tmp = X1[i * x1s0 + k * x1s1] - X2[j * x2s0 + k * x2s1];
    d += double(tmp * tmp);
  }
  D[i * ds0 + j * ds1] = T(sqrtF64(d));
}

NMK_KERNEL(256)
nmk_twin_pairwise_f64(const double *X1, int64_t x1r, int64_t x1c, int64_t x1s0,
                      int64_t x1s1, const double *X2, int64_t x2r, int64_t x2c,
                      int64_t x2s0, int64_t x2s1, double *D, int64_t dr,
                      int64_t dc, int64_t ds0, int64_t ds1, int64_t gs0,
                      int64_t gs1, int64_t gs2) {
  pairwiseFaithful<double>(X1, x1r, x1c, x1s0, x1s1, X2, x2r, x2c, x2s0, x2s1,
                           D, dr, dc, ds0, ds1, gs0, gs1, gs2);
}

NMK_KERNEL(256)
nmk_twin_pairwise_f32(const float *X1, int64_t x1r, int64_t x1c, int64_t x1s0,
                      int64_t x1s1, const float *X2, int64_t x2r, int64_t x2c,
                      int64_t x2s0, int64_t x2s1, float *D, int64_t dr,
                      int64_t dc, int64_t ds0, int64_t ds1, int64_t gs0,
                      int64_t gs1, int64_t gs2) {
  pairwiseFaithful<float>(X1, x1r, x1c, x1s0, x1s1, X2, x2r, x2c, x2s0, x2s1, D,
                          dr, dc, ds0, ds1, gs0, gs1, gs2);
}

// Remapped float64 twin for 3-column inputs and C-contiguous D with an even
// number of columns.  Work-items do not communicate, so any bijection between
// lanes and (i, j) pairs computes the same D; this one gives every lane two
// adjacent j (one 128-bit store, a wave writes 1 KiB of a row of D) and a
// chunk of rowsPerBlock rows i.  The two X2 rows live in registers for the
// whole chunk; X1 rows are wave-uniform.  Arithmetic per element is the body
// above, k = 0, 1, 2 in order, so results are bit-identical to the faithful
// twin.  Launch: block (256,1,1), grid (ceil(n2/512), ceil(n1/rowsPerBlock)).
NMK_KERNEL(256)
nmk_twin_pairwise_f64_rows(const double *__restrict__ X1,
                           const double *__restrict__ X2,
                           double *__restrict__ D, int64_t n1, int64_t n2,
                           int64_t rowsPerBlock) {
  const int64_t j = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) * 2;
  if (j >= n2)
    return;
  const double y00 = X2[j * 3 + 0], y01 = X2[j * 3 + 1], y02 = X2[j * 3 + 2];
  const double y10 = X2[j * 3 + 3], y11 = X2[j * 3 + 4], y12 = X2[j * 3 + 5];
  int64_t i = int64_t(blockIdx.y) * rowsPerBlock;
  int64_t iEnd = i + rowsPerBlock;
  if (iEnd > n1)
    iEnd = n1;
  for (; i < iEnd; ++i) {
    const double x0 = X1[i * 3 + 0], x1 = X1[i * 3 + 1], x2 = X1[i * 3 + 2];
    double t, d0 = 0.0, d1 = 0.0;
    t = x0 - y00;
    d0 += t * t;
    t = x1 - y01;
    d0 += t * t;
    t = x2 - y02;
    d0 += t * t;
    t = x0 - y10;
    d1 += t * t;
    t = x1 - y11;
    d1 += t * t;
    t = x2 - y12;
    d1 += t * t;
    double2_t r = {sqrtF64(d0), sqrtF64(d1)};
    streamStore(r, reinterpret_cast<double2_t *>(D + i * n2 + j));
  }
}

// ---------------------------------------------------------------------------
// Workgroup-memory kernel: every work-group reverses its slice of `a` through
// a local array and a barrier,
//   tmp = local.array(group_size); tmp[lid] = a[gid]; barrier();
//   b[gid] = tmp[group_size - 1 - lid]
// (local arrays and barriers: reference
// mlir_compiler/lib/pipelines/LowerToGpu.cpp:1296-1386, 1515-1553).
// The local array arrives the way the runtime passes workgroup memory: a
// uint64 byte offset into the launch's dynamic LDS block.  Requires the
// global size to be a multiple of the local size (uniform barrier).
NMK_KERNEL(256)
nmk_twin_group_reverse_i32(const int32_t *a, int64_t an, int64_t as, int32_t *b,
                           int64_t bn, int64_t bs, uint64_t tmpOffset,
                           int64_t gs0, int64_t gs1, int64_t gs2) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ldsBase[];
  int32_t *tmp = reinterpret_cast<int32_t *>(ldsBase + tmpOffset);
  Ids t = ids(gs0, gs1, gs2);
  if (t.inside)
    tmp[t.l[0]] = a[t.g[0] * as];
  __syncthreads();
  if (t.inside)
    b[t.g[0] * bs] = tmp[t.ls[0] - 1 - t.l[0]];
}

// ===========================================================================
// Kernel builtins beyond ids: atomics, barriers / fences, local and private
// arrays, group reductions.  Each twin is the body of a reference test
// (numba_mlir/numba_mlir/mlir/tests/test_gpu.py, cited per kernel); together
// they are the HIP device-side forms of what the reference lowers in
// mlir_compiler/lib/pipelines/LowerToGpu.cpp:1296-1780.
//
//  * atomic.add / atomic.sub (1404-1465): agent-scope atomicAdd; sub adds the
//    negated value, as the reference does (kernel_impl.py:263-322).
//  * barrier(flags) (1515-1553): __syncthreads(), preceded by a device-scope
//    fence for GLOBAL_MEM_FENCE; mem_fence(flags) is the fence alone.
//    Barriers sit outside the bounds guard so every lane reaches them (the
//    reference's MakeBarriersUniform transform does the same hoisting).
//  * local.array (1296-1386): workgroup memory passed by the runtime as a
//    byte offset into dynamic LDS.
//  * private.array: a per-lane array (registers / scratch).
//  * group.reduce_* (1564-1780): an LDS tree over the work-group (any local
//    size up to 256; the reference reduces subgroups of a hard-coded 8 lanes
//    first, 1683-1688); lanes past the global size contribute the neutral
//    element.
// ===========================================================================

namespace {

__device__ __forceinline__ int linearLocalId() {
  return threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z);
}

__device__ __forceinline__ int localCount() {
  return blockDim.x * blockDim.y * blockDim.z;
}

// Workgroup-wide reduction for any block shape up to 256 lanes (full and
// partial waves alike): an LDS tree.  Lanes outside the global size pass the
// neutral element.  Every lane of the block must call it.
template <typename T, typename Op>
__device__ __forceinline__ T groupReduce(T v, T neutral, bool active, Op op) {
  __shared__ T scratch[256];
  const int tid = linearLocalId();
  const int n = localCount();
  __syncthreads(); // scratch may still be read by a previous call
  scratch[tid] = active ? v : neutral;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s && tid + s < n)
      scratch[tid] = op(scratch[tid], scratch[tid + s]);
    __syncthreads();
  }
  return scratch[0];
}

template <typename T> __device__ __forceinline__ void atomicAddT(T *p, T v) {
  atomicAdd(p, v);
}
template <>
__device__ __forceinline__ void atomicAddT<int64_t>(int64_t *p, int64_t v) {
  atomicAdd(reinterpret_cast<unsigned long long *>(p),
            static_cast<unsigned long long>(v));
}

} // namespace

// c[i, j, k] = a[i, j, k] + b[i, j, k]   (test_simple1/2, test_gpu.py:178-232)
NMK_KERNEL(256)
nmk_twin_add3_f32(const float *a, int64_t a0, int64_t a1, int64_t a2,
                  int64_t as0, int64_t as1, int64_t as2, const float *b,
                  int64_t b0, int64_t b1, int64_t b2, int64_t bs0, int64_t bs1,
                  int64_t bs2, float *c, int64_t c0, int64_t c1, int64_t c2,
                  int64_t cs0, int64_t cs1, int64_t cs2, int64_t gs0,
                  int64_t gs1, int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  if (t.inside)
    c[t.g[0] * cs0 + t.g[1] * cs1 + t.g[2] * cs2] =
        a[t.g[0] * as0 + t.g[1] * as1 + t.g[2] * as2] +
        b[t.g[0] * bs0 + t.g[1] * bs1 + t.g[2] * bs2];
}

// b[i, 0] = a[i, 0]; b[i, 1] = a[i, 1]   (test_simple3, 235-259)
NMK_KERNEL(256)
nmk_twin_copy_cols2_f32(const float *a, int64_t a0, int64_t a1, int64_t as0,
                        int64_t as1, float *b, int64_t b0, int64_t b1,
                        int64_t bs0, int64_t bs1, int64_t gs0, int64_t gs1,
                        int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  if (t.inside) {
    b[t.g[0] * bs0] = a[t.g[0] * as0];
    b[t.g[0] * bs0 + bs1] = a[t.g[0] * as0 + as1];
  }
}

// res[i] = a[i] * b[i] + c[i] with two roundings (test_fastmath, 981-1008:
// no fma unless fastmath=True; this file is built with -ffp-contract=off).
NMK_KERNEL(256)
nmk_twin_mul_add_f32(const float *a, int64_t an, int64_t as, const float *b,
                     int64_t bn, int64_t bs, const float *c, int64_t cn,
                     int64_t cs, float *res, int64_t rn, int64_t rs,
                     int64_t gs0, int64_t gs1, int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  if (t.inside)
    res[t.g[0] * rs] = a[t.g[0] * as] * b[t.g[0] * bs] + c[t.g[0] * cs];
}

// Atomics (test_atomics*, 806-955).  MODE selects the body:
//   0: op(b, 0, a[i])          1: op(b, i % 2, a[i])
//   2: op(b, 0, a[i] + 1)      3: op(b, 0, 1)
// SIGN is +1 for atomic.add, -1 for atomic.sub.
template <typename T, int MODE, int SIGN>
__device__ __forceinline__ void atomicBody(const T *a, int64_t as, T *b,
                                           int64_t bs, int64_t gs0,
                                           int64_t gs1, int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  if (!t.inside)
    return;
  const int64_t i = t.g[0];
  T v = MODE == 3 ? T(1) : (MODE == 2 ? T(a[i * as] + T(1)) : a[i * as]);
  if (SIGN < 0)
    v = -v;
  atomicAddT(b + (MODE == 1 ? (i % 2) * bs : 0), v);
}

#define NMK_TWIN_ATOMIC(OPNAME, SIGN, TNAME, T, MODE)                          \
  NMK_KERNEL(256)                                                              \
  nmk_twin_atomic_##OPNAME##_m##MODE##_##TNAME(                                \
      const T *a, int64_t an, int64_t as, T *b, int64_t bn, int64_t bs,        \
      int64_t gs0, int64_t gs1, int64_t gs2) {                                 \
    atomicBody<T, MODE, SIGN>(a, as, b, bs, gs0, gs1, gs2);                    \
  }
#define NMK_TWIN_ATOMIC_ALL(TNAME, T)                                          \
  NMK_TWIN_ATOMIC(add, 1, TNAME, T, 0)                                         \
  NMK_TWIN_ATOMIC(sub, -1, TNAME, T, 0)                                        \
  NMK_TWIN_ATOMIC(add, 1, TNAME, T, 1)                                         \
  NMK_TWIN_ATOMIC(sub, -1, TNAME, T, 1)
NMK_TWIN_ATOMIC_ALL(i32, int32_t)
NMK_TWIN_ATOMIC_ALL(i64, int64_t)
NMK_TWIN_ATOMIC_ALL(f32, float)
NMK_TWIN_ATOMIC(add, 1, i32, int32_t, 2)
NMK_TWIN_ATOMIC(sub, -1, i32, int32_t, 2)
NMK_TWIN_ATOMIC(add, 1, i32, int32_t, 3)
NMK_TWIN_ATOMIC(sub, -1, i32, int32_t, 3)

// atomic.add(b, (i % 2, 0), a[i, j]) / (i % 2, j % 2)   (test_atomics_multidim)
template <int FUNC>
__device__ __forceinline__ void
atomicMultidim(const int32_t *a, int64_t as0, int64_t as1, int32_t *b,
               int64_t bs0, int64_t bs1, int64_t gs0, int64_t gs1,
               int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  if (!t.inside)
    return;
  const int64_t i = t.g[0], j = t.g[1];
  atomicAdd(b + (i % 2) * bs0 + (FUNC == 2 ? (j % 2) * bs1 : 0),
            a[i * as0 + j * as1]);
}
NMK_KERNEL(256)
nmk_twin_atomic_multidim1_i32(const int32_t *a, int64_t a0, int64_t a1,
                              int64_t as0, int64_t as1, int32_t *b, int64_t b0,
                              int64_t b1, int64_t bs0, int64_t bs1,
                              int64_t gs0, int64_t gs1, int64_t gs2) {
  atomicMultidim<1>(a, as0, as1, b, bs0, bs1, gs0, gs1, gs2);
}
NMK_KERNEL(256)
nmk_twin_atomic_multidim2_i32(const int32_t *a, int64_t a0, int64_t a1,
                              int64_t as0, int64_t as1, int32_t *b, int64_t b0,
                              int64_t b1, int64_t bs0, int64_t bs1,
                              int64_t gs0, int64_t gs1, int64_t gs2) {
  atomicMultidim<2>(a, as0, as1, b, bs0, bs1, gs0, gs1, gs2);
}

// atomic.add(a, (i, j), c[i, j]); atomic.add(b, (i), c[i, j])
// (test_atomics_different_dims, 928-955)
NMK_KERNEL(256)
nmk_twin_atomic_dims_i32(int32_t *a, int64_t a0, int64_t a1, int64_t as0,
                         int64_t as1, int32_t *b, int64_t b0, int64_t bs0,
                         const int32_t *c, int64_t c0, int64_t c1, int64_t cs0,
                         int64_t cs1, int64_t gs0, int64_t gs1, int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  if (!t.inside)
    return;
  const int64_t i = t.g[0], j = t.g[1];
  const int32_t v = c[i * cs0 + j * cs1];
  atomicAdd(a + i * as0 + j * as1, v);
  atomicAdd(b + i * bs0, v);
}

// v = a[i]; op(flags); b[i] = a[i]   (test_barrier_ops, 1074-1102)
// isBarrier: barrier(flags) or mem_fence(flags); flags: 1 local, 2 global.
NMK_KERNEL(256)
nmk_twin_barrier_ops_i64(const int64_t *a, int64_t an, int64_t as, int64_t *b,
                         int64_t bn, int64_t bs, int64_t isBarrier,
                         int64_t flags, int64_t gs0, int64_t gs1, int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  int64_t v = 0;
  if (t.inside)
    v = a[t.g[0] * as];
  if (flags & 2)
    __threadfence();
  else
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  if (isBarrier)
    __syncthreads();
  if (t.inside)
    b[t.g[0] * bs] = v;
}

// off = i // local_size; atomic.add(a, off, i); barrier(GLOBAL_MEM_FENCE);
// b[i] = a[off]   (test_barrier1, 1105-1133)
NMK_KERNEL(256)
nmk_twin_barrier1_i64(int64_t *a, int64_t an, int64_t as, int64_t *b,
                      int64_t bn, int64_t bs, int64_t localSize, int64_t gs0,
                      int64_t gs1, int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  const int64_t i = t.g[0];
  const int64_t off = i / localSize;
  if (t.inside)
    atomicAddT(a + off * as, i);
  __threadfence();
  __syncthreads();
  if (t.inside)
    b[i * bs] = __hip_atomic_load(a + off * as, __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_AGENT);
}

// lm = local.array(blocksize, float32); lm[i] = A[i]; barrier(LOCAL);
// A[i] += lm[blocksize - 1 - i]   (test_local_memory1/2, 1136-1198; one
// work-group).  lmOffset: byte offset of lm in dynamic LDS.
NMK_KERNEL(256)
nmk_twin_local_memory_f32(float *A, int64_t an, int64_t as, int64_t blocksize,
                          uint64_t lmOffset, int64_t gs0, int64_t gs1,
                          int64_t gs2) {
  extern __shared__ __attribute__((aligned(16))) unsigned char ldsBase[];
  float *lm = reinterpret_cast<float *>(ldsBase + lmOffset);
  Ids t = ids(gs0, gs1, gs2);
  const int64_t i = t.g[0];
  if (t.inside)
    lm[i] = A[i * as];
  __syncthreads();
  if (t.inside)
    A[i * as] += lm[blocksize - 1 - i];
}

// Private arrays (test_private_memory1-4, 1202-1326).  VARIANT:
//   1/2: p[0] = i; barrier; A[i] = p[0] * 2
//   3  : p[j] = j + i for j < n; res = sum_j p[(j + i) % n]; A[i] = res
//   4  : p[j][k] = i (10 x 10); barrier; A[i] = p[i % 10][i % 10] * 2
NMK_KERNEL(256)
nmk_twin_private_memory_f32(float *A, int64_t an, int64_t as, int64_t variant,
                            int64_t privSize, int64_t gs0, int64_t gs1,
                            int64_t gs2) {
  Ids t = ids(gs0, gs1, gs2);
  const int64_t i = t.g[0];
  float p[100];
  float res = 0.f;
  if (variant == 3) {
    for (int64_t j = 0; j < privSize; ++j)
      p[j] = float(j + i);
    // `res` starts as the integer 0 and becomes float32 on the first add
    for (int64_t j = 0; j < privSize; ++j)
      res += p[(j + i) % privSize];
  } else if (variant == 4) {
    for (int j = 0; j < 100; ++j)
      p[j] = float(i);
    __syncthreads();
    res = p[(i % 10) * 10 + (i % 10)] * 2.f;
  } else {
    p[0] = float(i);
    __syncthreads();
    res = p[0] * 2.f;
  }
  if (t.inside)
    A[i * as] = res;
}

// v = group.reduce_<op>(a[i]); b[i] = v   (test_group_func, 1360-1393)
#define NMK_TWIN_GROUP(OPNAME, OP, TNAME, T, NEUTRAL)                          \
  NMK_KERNEL(256)                                                              \
  nmk_twin_group_reduce_##OPNAME##_##TNAME(const T *a, int64_t an, int64_t as, \
                                           T *b, int64_t bn, int64_t bs,       \
                                           int64_t gs0, int64_t gs1,           \
                                           int64_t gs2) {                      \
    Ids t = ids(gs0, gs1, gs2);                                                \
    T v = t.inside ? a[t.g[0] * as] : T(NEUTRAL);                              \
    v = groupReduce<T>(v, T(NEUTRAL), t.inside, OP());                         \
    if (t.inside)                                                              \
      b[t.g[0] * bs] = v;                                                      \
  }
#define NMK_TWIN_GROUP_ALL(TNAME, T, TMIN, TMAX)                               \
  NMK_TWIN_GROUP(add, AddOp, TNAME, T, 0)                                      \
  NMK_TWIN_GROUP(mul, MulOp, TNAME, T, 1)                                      \
  NMK_TWIN_GROUP(min, MinOp, TNAME, T, TMAX)                                   \
  NMK_TWIN_GROUP(max, MaxOp, TNAME, T, TMIN)
NMK_TWIN_GROUP_ALL(i32, int32_t, INT32_MIN, INT32_MAX)
NMK_TWIN_GROUP_ALL(i64, int64_t, INT64_MIN, INT64_MAX)
NMK_TWIN_GROUP_ALL(f32, float, -__builtin_inff(), __builtin_inff())

// c[i] = a[i] <op> b[i] with Python semantics (test_gpu_ops_binary, 551-566):
// `/` is true division (the result is converted back to the array dtype),
// `//` floors, `%` takes the sign of the divisor, `**` is pow.
namespace {
template <typename T> struct PyOps {
  __device__ static T floordiv(T a, T b) { return T(floor(double(a) / double(b))); }
  __device__ static T mod(T a, T b) {
    T r = T(fmod(double(a), double(b)));
    return (r != T(0) && ((r < T(0)) != (b < T(0)))) ? r + b : r;
  }
  __device__ static T truediv(T a, T b) { return a / b; }
  __device__ static T power(T a, T b) { return T(pow(double(a), double(b))); }
};
template <> struct PyOps<int32_t> {
  __device__ static int32_t floordiv(int32_t a, int32_t b) {
    int32_t q = a / b;
    return ((a % b != 0) && ((a < 0) != (b < 0))) ? q - 1 : q;
  }
  __device__ static int32_t mod(int32_t a, int32_t b) {
    int32_t r = a % b;
    return (r != 0 && ((r < 0) != (b < 0))) ? r + b : r;
  }
  __device__ static int32_t truediv(int32_t a, int32_t b) {
    return int32_t(double(a) / double(b));
  }
  __device__ static int32_t power(int32_t a, int32_t b) {
    int64_t r = 1, base = a;
    for (int32_t e = b; e > 0; e >>= 1) {
      if (e & 1)
        r *= base;
      base *= base;
    }
    return int32_t(r);
  }
};
} // namespace

#define NMK_TWIN_BINARY(OPNAME, TNAME, T, EXPR)                                \
  NMK_KERNEL(256)                                                              \
  nmk_twin_binary_##OPNAME##_##TNAME(const T *a, int64_t an, int64_t as,       \
                                     const T *b, int64_t bn, int64_t bs, T *c, \
                                     int64_t cn, int64_t cs, int64_t gs0,      \
                                     int64_t gs1, int64_t gs2) {               \
    Ids t = ids(gs0, gs1, gs2);                                                \
    if (t.inside) {                                                            \
      const T x = a[t.g[0] * as], y = b[t.g[0] * bs];                          \
      c[t.g[0] * cs] = EXPR;                                                   \
    }                                                                          \
  }
#define NMK_TWIN_BINARY_ALL(TNAME, T)                                          \
  NMK_TWIN_BINARY(add, TNAME, T, x + y)                                        \
  NMK_TWIN_BINARY(sub, TNAME, T, x - y)                                        \
  NMK_TWIN_BINARY(mul, TNAME, T, x *y)                                         \
  NMK_TWIN_BINARY(truediv, TNAME, T, PyOps<T>::truediv(x, y))                  \
  NMK_TWIN_BINARY(floordiv, TNAME, T, PyOps<T>::floordiv(x, y))                \
  NMK_TWIN_BINARY(mod, TNAME, T, PyOps<T>::mod(x, y))                          \
  NMK_TWIN_BINARY(pow, TNAME, T, PyOps<T>::power(x, y))
NMK_TWIN_BINARY_ALL(i32, int32_t)
NMK_TWIN_BINARY_ALL(f32, float)
NMK_TWIN_BINARY_ALL(f64, double)
