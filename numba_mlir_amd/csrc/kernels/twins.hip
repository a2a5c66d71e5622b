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
