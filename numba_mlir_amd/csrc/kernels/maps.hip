// Elementwise / broadcasting maps for gfx950.
//
// These replace the kernels the reference generates from an all-parallel
// linalg.generic (reference: numba_mlir/numba_mlir/mlir/linalg_builder.py:297-325,
// broadcast rule mlir/lib/Conversion/NtensorToLinalg.cpp:487-557, tiling
// mlir/lib/Conversion/GpuToGpuRuntime.cpp:1395-1584), which run one element
// per work-item with scalar loads.  Here the contiguous cases move 128 bits
// per lane per access and keep a row-broadcast operand in registers.
//
// Kernel signatures are owned by the dispatcher (csrc/offload/Dispatch.cpp);
// sizes and strides are int64 element counts, as the reference's flattened
// memref ABI passes them (mlir/lib/Conversion/DecomposeMemrefs.cpp:85-206).
#include "common.h"

using namespace nmk;

namespace {

struct OpAdd {
  template <typename T> __device__ static T apply(T a, T b) { return a + b; }
};
struct OpSub {
  template <typename T> __device__ static T apply(T a, T b) { return a - b; }
};
struct OpMul {
  template <typename T> __device__ static T apply(T a, T b) { return a * b; }
};
struct OpDiv {
  template <typename T> __device__ static T apply(T a, T b) { return a / b; }
};

template <typename T> struct Vec128;
template <> struct Vec128<double> {
  typedef double2_t type;
  static constexpr int N = 2;
};
template <> struct Vec128<float> {
  typedef float4_t type;
  static constexpr int N = 4;
};

// out[r, c] = op(a[r, c], b[c]) for C-contiguous a/out of shape [rows, cols]
// and a [1, cols] (or [cols]) operand b.  Requires cols % N == 0 and 16-byte
// aligned bases (N = 128 bits / sizeof(T)); the dispatcher checks both.
//
// grid.x tiles the columns (256 lanes x 128 bit), grid.y tiles the rows in
// chunks of rowsPerBlock.  A lane loads its slice of b once and reuses it for
// every row of the chunk; row loads are issued four at a time so each lane
// has 4 x 16 B reads in flight.
template <typename T, typename Op>
__device__ __forceinline__ void
mapRowBroadcast(const T *__restrict__ a, const T *__restrict__ b,
                T *__restrict__ out, int64_t rows, int64_t cols,
                int64_t rowsPerBlock) {
  typedef typename Vec128<T>::type V;
  constexpr int N = Vec128<T>::N;
  const int64_t col = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) * N;
  if (col >= cols)
    return;
  const V bv = *reinterpret_cast<const V *>(b + col);
  int64_t r = int64_t(blockIdx.y) * rowsPerBlock;
  int64_t rEnd = r + rowsPerBlock;
  if (rEnd > rows)
    rEnd = rows;
  const T *ap = a + r * cols + col;
  T *op = out + r * cols + col;
  for (; r + 4 <= rEnd; r += 4) {
    V v0 = __builtin_nontemporal_load(reinterpret_cast<const V *>(ap));
    V v1 = __builtin_nontemporal_load(reinterpret_cast<const V *>(ap + cols));
    V v2 =
        __builtin_nontemporal_load(reinterpret_cast<const V *>(ap + 2 * cols));
    V v3 =
        __builtin_nontemporal_load(reinterpret_cast<const V *>(ap + 3 * cols));
    V o0, o1, o2, o3;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      o0[i] = Op::apply(v0[i], bv[i]);
      o1[i] = Op::apply(v1[i], bv[i]);
      o2[i] = Op::apply(v2[i], bv[i]);
      o3[i] = Op::apply(v3[i], bv[i]);
    }
    __builtin_nontemporal_store(o0, reinterpret_cast<V *>(op));
    __builtin_nontemporal_store(o1, reinterpret_cast<V *>(op + cols));
    __builtin_nontemporal_store(o2, reinterpret_cast<V *>(op + 2 * cols));
    __builtin_nontemporal_store(o3, reinterpret_cast<V *>(op + 3 * cols));
    ap += 4 * cols;
    op += 4 * cols;
  }
  for (; r < rEnd; ++r) {
    V v0 = *reinterpret_cast<const V *>(ap);
    V o0;
#pragma unroll
    for (int i = 0; i < N; ++i)
      o0[i] = Op::apply(v0[i], bv[i]);
    *reinterpret_cast<V *>(op) = o0;
    ap += cols;
    op += cols;
  }
}

// out[i] = op(a[i], b[i]) over n contiguous elements, n % N == 0, 16-byte
// aligned bases.  Grid-stride over 128-bit vectors, two per lane in flight.
template <typename T, typename Op>
__device__ __forceinline__ void
mapContiguous(const T *__restrict__ a, const T *__restrict__ b,
              T *__restrict__ out, int64_t n) {
  typedef typename Vec128<T>::type V;
  constexpr int N = Vec128<T>::N;
  const int64_t nvec = n / N;
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  const V *av = reinterpret_cast<const V *>(a);
  const V *bv = reinterpret_cast<const V *>(b);
  V *ov = reinterpret_cast<V *>(out);
  int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  for (; i + stride < nvec; i += 2 * stride) {
    V a0 = __builtin_nontemporal_load(av + i);
    V a1 = __builtin_nontemporal_load(av + i + stride);
    V b0 = __builtin_nontemporal_load(bv + i);
    V b1 = __builtin_nontemporal_load(bv + i + stride);
    V o0, o1;
#pragma unroll
    for (int k = 0; k < N; ++k) {
      o0[k] = Op::apply(a0[k], b0[k]);
      o1[k] = Op::apply(a1[k], b1[k]);
    }
    __builtin_nontemporal_store(o0, ov + i);
    __builtin_nontemporal_store(o1, ov + i + stride);
  }
  if (i < nvec) {
    V a0 = av[i], b0 = bv[i], o0;
#pragma unroll
    for (int k = 0; k < N; ++k)
      o0[k] = Op::apply(a0[k], b0[k]);
    ov[i] = o0;
  }
}

// General rank-2 strided binary map, one element per work-item, x <-> the
// last (fastest) dimension, tail guarded: the shape the reference's own
// lowering produces.  A broadcast dimension has stride 0.
template <typename T, typename Op>
__device__ __forceinline__ void
mapStrided2(const T *a, int64_t sa0, int64_t sa1, const T *b, int64_t sb0,
            int64_t sb1, T *out, int64_t so0, int64_t so1, int64_t n0,
            int64_t n1) {
  const int64_t j = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t i = int64_t(blockIdx.y) * blockDim.y + threadIdx.y;
  if (i >= n0 || j >= n1)
    return;
  out[i * so0 + j * so1] =
      Op::apply(a[i * sa0 + j * sa1], b[i * sb0 + j * sb1]);
}

} // namespace

#define NMK_DEFINE_MAP2(OPNAME, OP, TNAME, T)                                  \
  NMK_KERNEL(256)                                                              \
  nmk_map2_strided_##OPNAME##_##TNAME(                                         \
      const T *a, int64_t sa0, int64_t sa1, const T *b, int64_t sb0,           \
      int64_t sb1, T *out, int64_t so0, int64_t so1, int64_t n0, int64_t n1) { \
    mapStrided2<T, OP>(a, sa0, sa1, b, sb0, sb1, out, so0, so1, n0, n1);       \
  }

#define NMK_DEFINE_MAP2_FAST(OPNAME, OP, TNAME, T)                             \
  NMK_KERNEL(256)                                                              \
  nmk_map2_rowbcast_##OPNAME##_##TNAME(const T *a, const T *b, T *out,         \
                                       int64_t rows, int64_t cols,             \
                                       int64_t rowsPerBlock) {                 \
    mapRowBroadcast<T, OP>(a, b, out, rows, cols, rowsPerBlock);               \
  }                                                                            \
  NMK_KERNEL(256)                                                              \
  nmk_map2_contig_##OPNAME##_##TNAME(const T *a, const T *b, T *out,           \
                                     int64_t n) {                              \
    mapContiguous<T, OP>(a, b, out, n);                                        \
  }

#define NMK_DEFINE_MAP2_ALL_T(OPNAME, OP)                                      \
  NMK_DEFINE_MAP2(OPNAME, OP, f32, float)                                      \
  NMK_DEFINE_MAP2(OPNAME, OP, f64, double)                                     \
  NMK_DEFINE_MAP2(OPNAME, OP, i32, int32_t)                                    \
  NMK_DEFINE_MAP2(OPNAME, OP, i64, int64_t)                                    \
  NMK_DEFINE_MAP2_FAST(OPNAME, OP, f32, float)                                 \
  NMK_DEFINE_MAP2_FAST(OPNAME, OP, f64, double)

NMK_DEFINE_MAP2_ALL_T(add, OpAdd)
NMK_DEFINE_MAP2_ALL_T(sub, OpSub)
NMK_DEFINE_MAP2_ALL_T(mul, OpMul)

// ---------------------------------------------------------------------------
// Fused Black-Scholes map (formula: reference
// numba_mlir/numba_mlir/mlir/tests/test_numpy.py:2827-2852; the reference
// asserts the whole body fuses into one loop, 2865-2866).
//
// W is the type of the intermediates that involve a Python float or int
// literal.  In the reference a Python literal is float64/int64
// (linalg_builder.py:278-291) and float32 (x) float64 promotes to float64
// (261-275), so `volatility * volatility * 2`, `T * sig_sig_two`, `0.25 * z`,
// `1.0 / sqrt(z)`, w1, w2, d1, d2, r and the put expression are float64 and
// only log(P / S), T * mr and exp(b) * S stay float32: that is W = double.
// W = float evaluates the same expression tree entirely in float32 (what
// NumPy computes for the same source, and what the reference computes when
// the literals are written as np.float32).
template <typename W> struct BsMath;
template <> struct BsMath<double> {
  __device__ static double sqrt_(double x) { return sqrt(x); }
  __device__ static double erf_(double x) { return erf(x); }
};
template <> struct BsMath<float> {
  __device__ static float sqrt_(float x) { return sqrtf(x); }
  __device__ static float erf_(float x) { return erff(x); }
};

template <typename W>
__device__ __forceinline__ void blackScholesOne(float P, float S, float T,
                                                float mr, W sigSigTwo,
                                                float &call, float &put) {
  const float a = logf(P / S);
  const float b = T * mr;
  const W z = W(T) * sigSigTwo;
  const W c = W(0.25) * z;
  const W y = W(1.0) / BsMath<W>::sqrt_(z);
  const float amb = a - b;
  const W w1 = (W(amb) + c) * y;
  const W w2 = (W(amb) - c) * y;
  const W d1 = W(0.5) + W(0.5) * BsMath<W>::erf_(w1);
  const W d2 = W(0.5) + W(0.5) * BsMath<W>::erf_(w2);
  const float Se = expf(b) * S;
  const W r = W(P) * d1 - W(Se) * d2;
  call = float(r);
  put = float(r - W(P) + W(Se));
}

template <typename W>
__device__ __forceinline__ void
blackScholes(const float *__restrict__ price, const float *__restrict__ strike,
             const float *__restrict__ t, float rate, float volatility,
             float *__restrict__ call, float *__restrict__ put, int64_t n) {
  const float mr = -rate;
  const W sigSigTwo = W(volatility * volatility) * W(2);
  const int64_t nvec = n / 4;
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  const float4_t *pv = reinterpret_cast<const float4_t *>(price);
  const float4_t *sv = reinterpret_cast<const float4_t *>(strike);
  const float4_t *tv = reinterpret_cast<const float4_t *>(t);
  float4_t *cv = reinterpret_cast<float4_t *>(call);
  float4_t *uv = reinterpret_cast<float4_t *>(put);
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec;
       i += stride) {
    const float4_t P = __builtin_nontemporal_load(pv + i);
    const float4_t S = __builtin_nontemporal_load(sv + i);
    const float4_t T = __builtin_nontemporal_load(tv + i);
    float4_t c, u;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float ck, uk;
      blackScholesOne<W>(P[k], S[k], T[k], mr, sigSigTwo, ck, uk);
      c[k] = ck;
      u[k] = uk;
    }
    __builtin_nontemporal_store(c, cv + i);
    __builtin_nontemporal_store(u, uv + i);
  }
  // n % 4 trailing options, one per lane of the first block.
  const int64_t tail = nvec * 4 + threadIdx.x;
  if (blockIdx.x == 0 && tail < n) {
    float ck, uk;
    blackScholesOne<W>(price[tail], strike[tail], t[tail], mr, sigSigTwo, ck,
                       uk);
    call[tail] = ck;
    put[tail] = uk;
  }
}

NMK_KERNEL(256)
nmk_black_scholes_f32_w64(const float *price, const float *strike,
                          const float *t, float rate, float volatility,
                          float *call, float *put, int64_t n) {
  blackScholes<double>(price, strike, t, rate, volatility, call, put, n);
}

NMK_KERNEL(256)
nmk_black_scholes_f32_w32(const float *price, const float *strike,
                          const float *t, float rate, float volatility,
                          float *call, float *put, int64_t n) {
  blackScholes<float>(price, strike, t, rate, volatility, call, put, n);
}

// Fills n 32-bit words with a value (used to zero ticket counters: a
// hipMemset node would not be safe inside a captured graph).
NMK_KERNEL(256) nmk_fill_u32(uint32_t *dst, uint32_t value, int64_t n) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride)
    dst[i] = value;
}
