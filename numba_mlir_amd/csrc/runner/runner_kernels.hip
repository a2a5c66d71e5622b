// Kernels of the standalone runner's cases (HipRunner.cpp): what the
// reference's runner pipeline (mlir/tools/level_zero_runner/
// LevelZeroRunner.cpp:39-104 -- linalg to parallel loops, the loops' parallel
// dimensions mapped to blocks, one work-item per iteration, reduction
// dimensions a sequential loop inside it) turns the gpu.launch and
// linalg.generic bodies of mlir/test/L0_RUNNER/*.mlir into.  Strides are in
// elements; a stride of 0 reads a rank-0 operand for every iteration.
// Built with -ffp-contract=off: a multiply and an add stay two roundings.
#include <hip/hip_runtime.h>
#include <stdint.h>

// addf.mlir:21-28: 8 blocks of one thread, indexed by the block id.
extern "C" __global__ void rk_addf_blocks_f32(const float *a, const float *b,
                                              float *c) {
  const int64_t i = blockIdx.x;
  c[i] = a[i] + b[i];
}

enum { RK_ADD = 0, RK_SUB = 1, RK_MUL = 2, RK_DIV = 3 };
enum { RK_YIELD = 0, RK_NEG = 1, RK_EXP = 2 };

template <typename T> __device__ T rkExp(T x);
template <> __device__ float rkExp<float>(float x) { return expf(x); }
template <> __device__ double rkExp<double>(double x) { return exp(x); }

// linalg.generic with parallel iterators and a one-op body, rank <= 2:
// iteration (blockIdx.x, blockIdx.y).
template <typename T>
__device__ void rkMap2(int op, const T *a, int64_t sa0, int64_t sa1, const T *b,
                       int64_t sb0, int64_t sb1, T *out, int64_t so0,
                       int64_t so1) {
  const int64_t i = blockIdx.x, j = blockIdx.y;
  const T x = a[i * sa0 + j * sa1], y = b[i * sb0 + j * sb1];
  T r;
  switch (op) {
  case RK_ADD: r = x + y; break;
  case RK_SUB: r = x - y; break;
  case RK_MUL: r = x * y; break;
  default: r = x / y; break;
  }
  out[i * so0 + j * so1] = r;
}
template <typename T>
__device__ void rkMap1(int op, const T *a, int64_t sa0, int64_t sa1, T *out,
                       int64_t so0, int64_t so1) {
  const int64_t i = blockIdx.x, j = blockIdx.y;
  const T x = a[i * sa0 + j * sa1];
  out[i * so0 + j * so1] = op == RK_NEG ? -x : op == RK_EXP ? rkExp<T>(x) : x;
}

#define RK_MAPS(NAME, T)                                                       \
  extern "C" __global__ void rk_map2_##NAME(                                   \
      int op, const T *a, int64_t sa0, int64_t sa1, const T *b, int64_t sb0,   \
      int64_t sb1, T *out, int64_t so0, int64_t so1) {                         \
    rkMap2<T>(op, a, sa0, sa1, b, sb0, sb1, out, so0, so1);                    \
  }                                                                            \
  extern "C" __global__ void rk_map1_##NAME(int op, const T *a, int64_t sa0,   \
                                            int64_t sa1, T *out, int64_t so0,  \
                                            int64_t so1) {                     \
    rkMap1<T>(op, a, sa0, sa1, out, so0, so1);                                 \
  }
RK_MAPS(f32, float)
RK_MAPS(f64, double)

// linalg_gemvf.mlir:20-31: iterators (parallel, reduction), y[i] += A[i,j] x[j].
extern "C" __global__ void rk_gemv_f32(const float *A, int64_t lda,
                                       const float *x, float *y, int64_t n1) {
  const int64_t i = blockIdx.x;
  for (int64_t j = 0; j < n1; ++j) {
    const float p = A[i * lda + j] * x[j];
    y[i] = y[i] + p;
  }
}

// linalg_gemmf.mlir:23-34: iterators (parallel, parallel, reduction),
// C[i,j] += A[i,k] B[k,j].
extern "C" __global__ void rk_gemm_f32(const float *A, int64_t lda,
                                       const float *B, int64_t ldb, float *C,
                                       int64_t ldc, int64_t nk) {
  const int64_t i = blockIdx.x, j = blockIdx.y;
  for (int64_t k = 0; k < nk; ++k) {
    const float p = A[i * lda + k] * B[k * ldb + j];
    C[i * ldc + j] = C[i * ldc + j] + p;
  }
}

// OpTest.ExplicitPadding.mlir:18-29: out[d0 + 2, d1 + 1] = (in[d0, d1] +
// out[d0 + 2, d1 + 1]) - 0.
extern "C" __global__ void rk_explicit_padding_f32(const float *in, int64_t ldi,
                                                   float *out, int64_t ldo) {
  const int64_t d0 = blockIdx.x, d1 = blockIdx.y;
  float *o = out + (d0 + 2) * ldo + (d1 + 1);
  const float e = in[d0 * ldi + d1] + *o;
  *o = e - 0.0f;
}
