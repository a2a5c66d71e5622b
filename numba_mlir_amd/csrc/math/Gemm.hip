// HIP math runtime: device gemm behind mkl_gemm_<dtype>_device
// (include/numba_mlir_hip/MathRuntime.h).
//
// Entry points, argument meaning and layout rules follow the oneMKL-backed
// runtime they replace (reference:
// numba_mlir/numba_mlir/math_runtime/sycl/lib/NumpyLinalg.cpp:67-183); the
// arithmetic is a hand-written LDS-tiled fp32 MFMA kernel for gfx950 plus a
// strided fallback.
#include "numba_mlir_hip/GpuQueueInterface.hpp"
#include "numba_mlir_hip/MathRuntime.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// fatal_failure of the reference prints to stderr and aborts
// (math_runtime/include/Common.hpp:10-15).
[[noreturn]] void fatal(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  std::vfprintf(stderr, fmt, ap);
  va_end(ap);
  std::fflush(stderr);
  std::abort();
}

void checkHip(hipError_t err, const char *what) {
  if (err != hipSuccess)
    fatal("%s failed: %s (%d)\n", what, hipGetErrorString(err),
          static_cast<int>(err));
}

thread_local const char *lastKernel = "";

// ---------------------------------------------------------------------------
// C[M,N] = alpha * A[M,K] * B[K,N] + beta * C with C row-major (ldc), fp32 in,
// fp32 accumulate on the matrix cores.  Each input operand may be stored with
// either of its two dimensions contiguous:
//   A_KC: A(m,k) = A[m * lda + k]   (row-major A)   else A[k * lda + m]
//   B_NC: B(k,n) = B[k * ldb + n]   (row-major B)   else B[n * ldb + k]
// which covers the four transpose cases of a BLAS gemm; a column-major C is
// handled by the host as C^T = B^T A^T.
//
// 256 threads = 4 waves in a 2 x 2 grid; each wave owns TM x TN tiles of
// v_mfma_f32_32x32x2_f32, so the block tile is (64 TM) x (64 TN) and a wave
// keeps 16 TM TN accumulator registers.  K advances in slabs of BK = 16.
//
// LDS holds both operands K-major ([k][m] and [k][n], rows padded by 4 floats)
// so that the MFMA operand fetch -- lane l needs element (l % 32) of row
// (k + l / 32) -- is a conflict-free ds_read_b32.  Global fetches are float4
// along the operand's contiguous dimension: an operand contiguous in m / n
// is written to LDS as float4, one contiguous in k is scattered over four LDS
// rows.  Two LDS stages: the next K slab is fetched from global memory into
// registers before the MFMAs of the current slab are issued and written to
// the other stage after them, one barrier per slab.
//
// MFMA 32x32x2 operand layout (64 lanes):
//   A (32 x 2): lane l holds A[l % 32][l / 32]
//   B (2 x 32): lane l holds B[l / 32][l % 32]
//   D (32 x 32): lane l, register r holds D[8*(r/4) + 4*(l/32) + r%4][l % 32]
//
// Requirements (checked by the host): M % (64 TM) == 0, N % (64 TN) == 0,
// K % 16 == 0, lda/ldb % 4 == 0, A and B 16-byte aligned.
constexpr int BK = 16, PAD = 4;

// One operand's slab of X x 16 (X = BM or BN) on its way from global memory
// to LDS[stage][k][x].  T float4 per thread.
template <int X, bool K_CONTIG> struct SlabFetch {
  static constexpr int T = X / 64;
  // K_CONTIG: thread -> (x = tid / 4 + 64 i, k = 4 (tid % 4) .. +3)
  // else    : thread -> (k = tid / (X / 4) + (1024 / X) i, x = 4 (tid % (X/4)) .. +3)
  static constexpr int K_ROWS = 1024 / X;
  int x, k;
  const float *base;
  int64_t ld;
  floatx4 reg[T];

  __device__ __forceinline__ void init(const float *p, int64_t ld_, int origin,
                                       int tid) {
    ld = ld_;
    if (K_CONTIG) {
      x = tid / 4;
      k = (tid % 4) * 4;
      base = p + int64_t(origin + x) * ld + k;
    } else {
      k = tid / (X / 4);
      x = (tid % (X / 4)) * 4;
      base = p + int64_t(k) * ld + origin + x;
    }
  }
  __device__ __forceinline__ void fetch(int k0) {
#pragma unroll
    for (int i = 0; i < T; ++i)
      reg[i] = *reinterpret_cast<const floatx4 *>(
          K_CONTIG ? base + int64_t(64 * i) * ld + k0
                   : base + int64_t(k0 + K_ROWS * i) * ld);
  }
  __device__ __forceinline__ void stash(float (*lds)[X + PAD]) const {
#pragma unroll
    for (int i = 0; i < T; ++i) {
      if (K_CONTIG) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          lds[k + q][x + 64 * i] = reg[i][q];
      } else {
        *reinterpret_cast<floatx4 *>(&lds[k + K_ROWS * i][x]) = reg[i];
      }
    }
  }
};

template <int TM, int TN, bool A_KC, bool B_NC>
__global__ __launch_bounds__(256) void
sgemm_mfma(const float *__restrict__ A, const float *__restrict__ B,
           float *__restrict__ C, int M, int N, int K, int64_t lda, int64_t ldb,
           int64_t ldc, float alpha, float beta) {
  constexpr int BM = 64 * TM, BN = 64 * TN;
  __shared__ float As[2][BK][BM + PAD];
  __shared__ float Bs[2][BK][BN + PAD];

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;
  const int bm = blockIdx.y * BM;
  const int bn = blockIdx.x * BN;

  SlabFetch<BM, A_KC> fa;
  SlabFetch<BN, !B_NC> fb;
  fa.init(A, lda, bm, tid);
  fb.init(B, ldb, bn, tid);

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = 0.f;

  fa.fetch(0);
  fb.fetch(0);
  fa.stash(As[0]);
  fb.stash(Bs[0]);
  __syncthreads();

  const int nSlabs = K / BK;
  const int kLane = lane / 32, xLane = lane % 32;
  for (int s = 0; s < nSlabs; ++s) {
    const int cur = s & 1;
    if (s + 1 < nSlabs) {
      fa.fetch((s + 1) * BK);
      fb.fetch((s + 1) * BK);
    }
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a[i] = As[cur][kk + kLane][wm * (32 * TM) + i * 32 + xLane];
#pragma unroll
      for (int j = 0; j < TN; ++j)
        b[j] = Bs[cur][kk + kLane][wn * (32 * TN) + j * 32 + xLane];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j],
                                                           acc[i][j], 0, 0, 0);
    }
    if (s + 1 < nSlabs) {
      fa.stash(As[cur ^ 1]);
      fb.stash(Bs[cur ^ 1]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = bn + wn * (32 * TN) + j * 32 + xLane;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row =
            bm + wm * (32 * TM) + i * 32 + 8 * (r / 4) + 4 * kLane + r % 4;
        float *dst = C + int64_t(row) * ldc + col;
        float v = alpha * acc[i][j][r];
        if (beta != 0.f)
          v += beta * *dst;
        *dst = v;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Any shape, any strides (element strides per dimension), float or double:
// classic 32 x 32 LDS tiling, one output per thread x 4 rows, bounds checked.
// Used for the transposed / column-major / ragged cases the MFMA kernel does
// not take.
template <typename T>
__global__ __launch_bounds__(256) void
gemm_generic(const T *A, const T *B, T *C, int64_t M, int64_t N, int64_t K,
             int64_t as0, int64_t as1, int64_t bs0, int64_t bs1, int64_t cs0,
             int64_t cs1, T alpha, T beta) {
  constexpr int TILE = 32;
  __shared__ T As[TILE][TILE + 1];
  __shared__ T Bs[TILE][TILE + 1];
  const int tx = threadIdx.x % TILE; // column within the tile
  const int ty = threadIdx.x / TILE; // 0..7, rows ty, ty+8, ty+16, ty+24
  const int64_t row0 = int64_t(blockIdx.y) * TILE;
  const int64_t col = int64_t(blockIdx.x) * TILE + tx;
  T acc[4] = {T(0), T(0), T(0), T(0)};
  for (int64_t k0 = 0; k0 < K; k0 += TILE) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = ty + 8 * i;
      const int64_t ar = row0 + r, ak = k0 + tx;
      As[r][tx] = (ar < M && ak < K) ? A[ar * as0 + ak * as1] : T(0);
      const int64_t bk = k0 + r;
      Bs[r][tx] = (bk < K && col < N) ? B[bk * bs0 + col * bs1] : T(0);
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TILE; ++k) {
      const T b = Bs[k][tx];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[i] += As[ty + 8 * i][k] * b;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t row = row0 + ty + 8 * i;
    if (row < M && col < N) {
      T *dst = C + row * cs0 + col * cs1;
      T v = alpha * acc[i];
      if (beta != T(0))
        v += beta * *dst;
      *dst = v;
    }
  }
}

template <typename T> struct MemrefOf;
template <> struct MemrefOf<float> {
  typedef NmhipMemref2F32 type;
};
template <> struct MemrefOf<double> {
  typedef NmhipMemref2F64 type;
};

template <typename T>
void requireUnitStride(const typename MemrefOf<T>::type *arr, char name) {
  if (arr->strides[0] != 1 && arr->strides[1] != 1)
    fatal("mkl gemm suports only arrays contiguous on inner dimension.\n"
          "stride for at least one dimension should be equal to 1.\n"
          "'%c' parameter is not contiguous. '%c' strides are %d and %d.\n",
          name, name, int(arr->strides[0]), int(arr->strides[1]));
}

bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

template <typename T>
void deviceGemm(void *queueObj, const typename MemrefOf<T>::type *a,
                const typename MemrefOf<T>::type *b,
                typename MemrefOf<T>::type *c, T alpha, T beta) {
  if (!queueObj || !a || !b || !c)
    fatal("mkl_gemm_device: null argument\n");
  auto *base = static_cast<numba::GPUQueueInterface *>(queueObj);
  auto *queue = static_cast<numba::HipQueueInterface *>(base);
  if (queue->hipMagic() != numba::HipQueueInterface::kMagic)
    fatal("mkl_gemm_device: queue '%.*s' was not created by the HIP GPU "
          "runtime\n",
          int(base->getDeviceName().size()), base->getDeviceName().data());

  requireUnitStride<T>(a, 'a');
  requireUnitStride<T>(b, 'b');
  requireUnitStride<T>(c, 'c');

  const int64_t M = int64_t(a->dims[0]);
  const int64_t N = int64_t(b->dims[1]);
  const int64_t K = int64_t(a->dims[1]);
  if (int64_t(b->dims[0]) != K || int64_t(c->dims[0]) != M ||
      int64_t(c->dims[1]) != N)
    fatal("mkl_gemm_device: shape mismatch: a [%lld,%lld] b [%lld,%lld] c "
          "[%lld,%lld]\n",
          (long long)a->dims[0], (long long)a->dims[1], (long long)b->dims[0],
          (long long)b->dims[1], (long long)c->dims[0], (long long)c->dims[1]);

  const T *aData = a->data + a->offset;
  const T *bData = b->data + b->offset;
  T *cData = c->data + c->offset;

  checkHip(hipSetDevice(queue->hipDevice()), "hipSetDevice");
  auto stream = static_cast<hipStream_t>(queue->hipStream());

  if (M > 0 && N > 0) {
    bool launched = false;
    if constexpr (sizeof(T) == 4) {
      // Operands as the kernel sees them: X(m,k), Y(k,n), Z row-major.  A
      // column-major C is computed as C^T = B^T A^T (swap and transpose the
      // inputs); which dimension of each input is contiguous follows from
      // its unit stride (NumpyLinalg.cpp:87-102).
      const bool cRow = c->strides[1] == 1;
      const float *X = cRow ? aData : bData;
      const float *Y = cRow ? bData : aData;
      // strides of X over (m, k) and Y over (k, n)
      const int64_t xm = cRow ? a->strides[0] : b->strides[1];
      const int64_t xk = cRow ? a->strides[1] : b->strides[0];
      const int64_t yk = cRow ? b->strides[0] : a->strides[1];
      const int64_t yn = cRow ? b->strides[1] : a->strides[0];
      const int64_t Mz = cRow ? M : N, Nz = cRow ? N : M;
      const int64_t ldz = cRow ? c->strides[0] : c->strides[1];
      const bool xKc = xk == 1, yNc = yn == 1;
      const int64_t ldx = xKc ? xm : xk, ldy = yNc ? yk : yn;
      // 256 x 256 block tiles (one block per CU on a 4096^2 problem) when the
      // shape allows and there are enough tiles to fill the 256 CUs; 128 x
      // 128 otherwise.  Measured within 3 % of each other; the larger tile
      // halves the operand traffic.
      const bool big = Mz % 256 == 0 && Nz % 256 == 0 &&
                       (Mz / 256) * (Nz / 256) >= 192;
      const int BM = big ? 256 : 128, BN = BM;
      const bool unitOk = (xk == 1 || xm == 1) && (yk == 1 || yn == 1);
      if (unitOk && K > 0 && Mz % BM == 0 && Nz % BN == 0 && K % BK == 0 &&
          ldx % 4 == 0 && ldy % 4 == 0 && ldx > 0 && ldy > 0 && aligned16(X) &&
          aligned16(Y) && M <= 0x7fffffff && N <= 0x7fffffff &&
          K <= 0x7fffffff && Mz / BM <= 65535) {
        dim3 grid(unsigned(Nz / BN), unsigned(Mz / BM), 1);
#define NMHIP_SGEMM_LAUNCH(TM, TN, XKC, YNC)                                   \
  hipLaunchKernelGGL((sgemm_mfma<TM, TN, XKC, YNC>), grid, dim3(256), 0,       \
                     stream, X, Y, cData, int(Mz), int(Nz), int(K), ldx, ldy,  \
                     ldz, alpha, beta)
#define NMHIP_SGEMM_LAYOUTS(TM, TN)                                            \
  do {                                                                         \
    if (xKc && yNc)                                                            \
      NMHIP_SGEMM_LAUNCH(TM, TN, true, true);                                  \
    else if (xKc)                                                              \
      NMHIP_SGEMM_LAUNCH(TM, TN, true, false);                                 \
    else if (yNc)                                                              \
      NMHIP_SGEMM_LAUNCH(TM, TN, false, true);                                 \
    else                                                                       \
      NMHIP_SGEMM_LAUNCH(TM, TN, false, false);                                \
  } while (0)
        if (big) {
          NMHIP_SGEMM_LAYOUTS(4, 4);
          lastKernel = "sgemm_mfma_256x256";
        } else {
          NMHIP_SGEMM_LAYOUTS(2, 2);
          lastKernel = "sgemm_mfma_128x128";
        }
#undef NMHIP_SGEMM_LAYOUTS
#undef NMHIP_SGEMM_LAUNCH
        launched = true;
      }
    }
    if (!launched) {
      const int64_t gx = (N + 31) / 32, gy = (M + 31) / 32;
      if (gy > 65535)
        fatal("mkl_gemm_device: M = %lld is too large for the strided "
              "kernel\n",
              (long long)M);
      dim3 grid{unsigned(gx), unsigned(gy), 1};
      hipLaunchKernelGGL(gemm_generic<T>, grid, dim3(256), 0, stream, aData,
                         bData, cData, M, N, K, int64_t(a->strides[0]),
                         int64_t(a->strides[1]), int64_t(b->strides[0]),
                         int64_t(b->strides[1]), int64_t(c->strides[0]),
                         int64_t(c->strides[1]), alpha, beta);
      lastKernel = sizeof(T) == 4 ? "sgemm_generic" : "dgemm_generic";
    }
    checkHip(hipGetLastError(), "gemm launch");
  }
  // The reference call returns only when C is complete (.wait(), 127/145).
  checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
}

} // namespace

#define NMHIP_MATH_EXPORT extern "C" __attribute__((visibility("default")))

NMHIP_MATH_EXPORT void mkl_gemm_float32_device(void *queue,
                                               const NmhipMemref2F32 *a,
                                               const NmhipMemref2F32 *b,
                                               float alpha, float beta,
                                               NmhipMemref2F32 *c) {
  deviceGemm<float>(queue, a, b, c, alpha, beta);
}

NMHIP_MATH_EXPORT void mkl_gemm_float64_device(void *queue,
                                               const NmhipMemref2F64 *a,
                                               const NmhipMemref2F64 *b,
                                               double alpha, double beta,
                                               NmhipMemref2F64 *c) {
  deviceGemm<double>(queue, a, b, c, alpha, beta);
}

NMHIP_MATH_EXPORT void nmrtMathRuntimeInit(void) {}
NMHIP_MATH_EXPORT void nmrtMathRuntimeFinalize(void) {}

NMHIP_MATH_EXPORT const char *nmhipMathLastKernel(void) { return lastKernel; }
