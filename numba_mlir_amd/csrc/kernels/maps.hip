// Elementwise / broadcasting maps for gfx950.
//
// These replace the kernels the reference generates from an all-parallel
// linalg.generic (reference: numba_mlir/numba_mlir/mlir/linalg_builder.py:297-325,
// broadcast rule mlir/lib/Conversion/NtensorToLinalg.cpp:487-557, tiling
// mlir/lib/Conversion/GpuToGpuRuntime.cpp:1395-1584), which run one element
// per work-item with scalar loads.  Here the contiguous cases move 128 bits
// per lane per access and keep a row-broadcast operand in registers.
//
// Kernel signatures are owned by the dispatcher (csrc/offload/Offload.cpp);
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
// every row of the chunk; rows are taken two at a time.  Short chunks (1-2
// rows, thousands of blocks each streaming a few KiB) measured fastest.
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
  for (; r + 2 <= rEnd; r += 2) {
    V v0 = streamLoad(reinterpret_cast<const V *>(ap));
    V v1 = streamLoad(reinterpret_cast<const V *>(ap + cols));
    V o0, o1;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      o0[i] = Op::apply(v0[i], bv[i]);
      o1[i] = Op::apply(v1[i], bv[i]);
    }
    streamStore(o0, reinterpret_cast<V *>(op));
    streamStore(o1, reinterpret_cast<V *>(op + cols));
    ap += 2 * cols;
    op += 2 * cols;
  }
  if (r < rEnd) {
    V v0 = streamLoad(reinterpret_cast<const V *>(ap));
    V o0;
#pragma unroll
    for (int i = 0; i < N; ++i)
      o0[i] = Op::apply(v0[i], bv[i]);
    streamStore(o0, reinterpret_cast<V *>(op));
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
    V a0 = streamLoad(av + i);
    V a1 = streamLoad(av + i + stride);
    V b0 = streamLoad(bv + i);
    V b1 = streamLoad(bv + i + stride);
    V o0, o1;
#pragma unroll
    for (int k = 0; k < N; ++k) {
      o0[k] = Op::apply(a0[k], b0[k]);
      o1[k] = Op::apply(a1[k], b1[k]);
    }
    streamStore(o0, ov + i);
    streamStore(o1, ov + i + stride);
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
//
// Transcendentals.  log(P/S) and exp(b) are the float32 library routines.
// The two float64 erf calls and 1.0 / sqrt(z) dominate the instruction count
// (the kernel is ALU-bound, not HBM-bound), so the float64 path evaluates
//   0.5 + 0.5 erf(x)  by a piecewise degree-9 polynomial for erf / 2 on 24
//        intervals of [0, 6) (erf_table.inc, absolute error < 1e-14;
//        erf(|x| >= 6) = 1 in double), coefficients staged in LDS; halving is
//        exact, so the sum rounds as 0.5 + 0.5 * erf(x) would;
//   1/sqrt(z)  by v_rsq_f64 refined with two Newton steps (relative error a
//        few 1e-16), falling back to 1.0 / sqrt(z) outside [1e-290, 1e290].
// Both stay within a few ulp of the library results, far inside the
// tolerance the path is checked at.
#include "erf_table.inc"

template <typename W> struct BsMath;
template <> struct BsMath<double> {
  __device__ static __forceinline__ double rsqrt_(double z) {
    if (!(z > 1e-290 && z < 1e290))
      return 1.0 / sqrt(z);
    double y = __builtin_amdgcn_rsq(z);
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const double r = __builtin_fma(-z, y * y, 1.0); // 1 - z y^2
      y = __builtin_fma(0.5 * y, r, y);
    }
    return y;
  }
  // 0.5 + 0.5 * erf(x)
  __device__ static __forceinline__ double cdfTerm(double x, const double *tab) {
    const double ax = __builtin_fabs(x);
    const double t = ax * 4.0; // interval index + fraction
    // int(NaN) is 0 and int(huge) saturates, so the row index is always valid
    const int idx = min(int(t), NMK_ERF_INTERVALS - 1);
    // u = 8 |x| - (2 idx + 1) = 2 frac(t) - 1; NaN stays NaN
    const double u = __builtin_fma(t - double(idx), 2.0, -1.0);
    const double *c = tab + __mul24(idx, NMK_ERF_ROW);
    double p = c[NMK_ERF_COEFFS - 1];
#pragma unroll
    for (int k = NMK_ERF_COEFFS - 2; k >= 0; --k)
      p = __builtin_fma(p, u, c[k]);
    // erf(|x| >= 6) rounds to exactly 1 in double (erfc(6) = 2e-17)
    p = ax >= 6.0 ? 0.5 : p;
    return 0.5 + __builtin_copysign(p, x);
  }
};
template <> struct BsMath<float> {
  __device__ static __forceinline__ float rsqrt_(float z) {
    return 1.0f / sqrtf(z);
  }
  __device__ static __forceinline__ float cdfTerm(float x, const double *) {
    return 0.5f + 0.5f * erff(x);
  }
};

template <typename W>
__device__ __forceinline__ void
blackScholesOne(float P, float S, float T, float mr, W sigSigTwo,
                const double *erfTab, float &call, float &put) {
  const float a = logf(P / S);
  const float b = T * mr;
  const W z = W(T) * sigSigTwo;
  const W c = W(0.25) * z;
  const W y = BsMath<W>::rsqrt_(z);
  const float amb = a - b;
  const W w1 = (W(amb) + c) * y;
  const W w2 = (W(amb) - c) * y;
  const W d1 = BsMath<W>::cdfTerm(w1, erfTab); // 0.5 + 0.5 * erf(w1)
  const W d2 = BsMath<W>::cdfTerm(w2, erfTab);
  const float Se = expf(b) * S;
  const W r = W(P) * d1 - W(Se) * d2;
  call = float(r);
  put = float(r - W(P) + W(Se));
}

// VEC options per lane per iteration (float4 or float2 accesses).  The
// float64 variant is ALU-bound and register-hungry: two options per lane at
// five to six waves per SIMD measured fastest (no spills at five); the
// float32 variant takes four.
template <int VEC> struct BsVec;
template <> struct BsVec<4> {
  typedef float4_t type;
};
template <> struct BsVec<2> {
  typedef float type __attribute__((ext_vector_type(2)));
};

template <typename W, int VEC>
__device__ __forceinline__ void
blackScholes(const float *__restrict__ price, const float *__restrict__ strike,
             const float *__restrict__ t, float rate, float volatility,
             float *__restrict__ call, float *__restrict__ put, int64_t n) {
  typedef typename BsVec<VEC>::type V;
  __shared__ __attribute__((aligned(16))) double
      erfTab[sizeof(W) == 8 ? NMK_ERF_INTERVALS * NMK_ERF_ROW : 1];
  if (sizeof(W) == 8) {
    for (int i = threadIdx.x; i < NMK_ERF_INTERVALS * NMK_ERF_ROW;
         i += blockDim.x)
      erfTab[i] = kHalfErfTable[i];
    __syncthreads();
  }
  const float mr = -rate;
  const W sigSigTwo = W(volatility * volatility) * W(2);
  const int64_t nvec = n / VEC;
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  const V *pv = reinterpret_cast<const V *>(price);
  const V *sv = reinterpret_cast<const V *>(strike);
  const V *tv = reinterpret_cast<const V *>(t);
  V *cv = reinterpret_cast<V *>(call);
  V *uv = reinterpret_cast<V *>(put);
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec;
       i += stride) {
    const V P = streamLoad(pv + i);
    const V S = streamLoad(sv + i);
    const V T = streamLoad(tv + i);
    V c, u;
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      float ck, uk;
      blackScholesOne<W>(P[k], S[k], T[k], mr, sigSigTwo, erfTab, ck, uk);
      c[k] = ck;
      u[k] = uk;
    }
    streamStore(c, cv + i);
    streamStore(u, uv + i);
  }
  // n % VEC trailing options, one per lane of the first block.
  const int64_t tail = nvec * VEC + threadIdx.x;
  if (blockIdx.x == 0 && tail < n) {
    float ck, uk;
    blackScholesOne<W>(price[tail], strike[tail], t[tail], mr, sigSigTwo,
                       erfTab, ck, uk);
    call[tail] = ck;
    put[tail] = uk;
  }
}

extern "C" __global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(6, 6))) void
nmk_black_scholes_f32_w64(const float *price, const float *strike,
                          const float *t, float rate, float volatility,
                          float *call, float *put, int64_t n) {
  blackScholes<double, 2>(price, strike, t, rate, volatility, call, put, n);
}

NMK_KERNEL(256)
nmk_black_scholes_f32_w32(const float *price, const float *strike,
                          const float *t, float rate, float volatility,
                          float *call, float *put, int64_t n) {
  blackScholes<float, 4>(price, strike, t, rate, volatility, call, put, n);
}

// Plain copy of nvec 128-bit words (force_copy of a contiguous operand; also
// the known-size yardstick the HBM counters are scaled against).  One 4 KiB
// piece per block iteration.
NMK_KERNEL(256)
nmk_copy_b128(const int4_t *__restrict__ src, int4_t *__restrict__ dst,
              int64_t nvec) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec;
       i += stride)
    streamStore(streamLoad(src + i), dst + i);
}

// Fills n 32-bit words with a value (used to zero ticket counters: a
// hipMemset node would not be safe inside a captured graph).
NMK_KERNEL(256) nmk_fill_u32(uint32_t *dst, uint32_t value, int64_t n) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride)
    dst[i] = value;
}
