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
// Cost.  Arithmetic and HBM traffic take about the same time here (about
// 40 us of vector-ALU issue against 52 us for the five streams of 2^24
// options), so every instruction counts:
//   0.5 + 0.5 erf(x)  is a degree-7 polynomial for erf / 2 around the nearest
//        of 97 nodes 1/16 apart on [0, 6] (erf_table.inc, absolute error of
//        erf below 1e-15; erf(|x| >= 5.97) = 1 in double), coefficients
//        staged in LDS; halving is exact, so the sum rounds as
//        0.5 + 0.5 * erf(x) would;
//   1 / sqrt(z)  is v_rsq_f64 with one third-order correction (below one unit
//        in the last place);
//   log(P / S) and exp(b)  are the float32 library routines' own operation
//        sequences without their range handling wherever every lane of the
//        wave has everyday operands (bit-identical results), and the library
//        routines otherwise.
#include "erf_table.inc"

template <typename W> struct BsMath;
template <> struct BsMath<double> {
  // 1 / sqrt(z) for z = T * sigSigTwo: the product of a float and of the
  // double of a float, so z is 0, inf, NaN, negative or a normal double far
  // from the ends of the range, and neither y * y nor z * y * y can overflow.
  // The hardware seed (relative error e below 2^-20) gets one third-order
  // step y (1 + e/2 + 3 e^2 / 8), leaving 5/16 e^3: below 2^-60.
  __device__ static __forceinline__ double rsqrt_(double z) {
    const double y = __builtin_amdgcn_rsq(z);
    const double e = __builtin_fma(-z, y * y, 1.0); // 1 - z y^2
    const double step = __builtin_fma(y * e, __builtin_fma(0.375, e, 0.5), y);
    // z = 0 -> inf and z = inf -> 0 come from the seed (e is NaN there);
    // a negative or NaN z gives NaN either way.
    return __builtin_amdgcn_class(z, 0x260 /* -0 | +0 | +inf */) ? y : step;
  }
  // 0.5 + 0.5 * erf(x) for a non-NaN x (a NaN x gives a finite value: the
  // caller tests for it).
  __device__ static __forceinline__ double cdfTerm(double x, const double *tab) {
    const double ax = __builtin_fmin(__builtin_fabs(x), 6.0);
    // Adding 1.5 * 2^48 rounds ax to the nearest sixteenth and leaves that
    // count, 0..96, in the low word of the sum.
    const double magic = 0x1.8p48;
    const double t = ax + magic;
    const int node = __double2loint(t);
    const double u = ax - (t - magic); // exact, |u| <= 1/32
    const double *c = tab + __mul24(node, NMK_ERF_ROW);
    double p = c[NMK_ERF_COEFFS - 1];
#pragma unroll
    for (int k = NMK_ERF_COEFFS - 2; k >= 0; --k)
      p = __builtin_fma(p, u, c[k]);
    return 0.5 + __builtin_copysign(p, x);
  }
  __device__ static __forceinline__ bool eitherNaN(double a, double b) {
    return __builtin_isunordered(a, b);
  }
};
template <> struct BsMath<float> {
  __device__ static __forceinline__ float rsqrt_(float z) {
    return 1.0f / sqrtf(z);
  }
  __device__ static __forceinline__ float cdfTerm(float x, const double *) {
    return 0.5f + 0.5f * erff(x);
  }
  __device__ static __forceinline__ bool eitherNaN(float, float) {
    return false; // erff propagates NaN by itself
  }
};

// The float32 steps log(P / S) and exp(b) without the range handling of the
// general routines: the same operations in the same order, so log and exp
// are bit-identical to logf and expf whenever bsEveryday() holds -- P and S
// positive with exponents in [-60, 60) (the quotient and the reciprocal are
// then normal numbers) and |b| <= 80 (exp(b) is normal).  The division is
// the reciprocal times P with one residual correction: it equals the
// correctly rounded quotient unless that quotient lies within 2e-7 units in
// the last place of a rounding boundary (no case among the 2^24 options of
// the benchmark input).  It is the general routines' handling of zeros,
// infinities, NaNs, denormals and overflow that costs two thirds of their
// instructions.
__device__ __forceinline__ bool bsEveryday(float P, float S, float b) {
  const uint32_t lo = 0x21800000u;   // bits of 2^-60
  const uint32_t span = 0x3C000000u; // up to, not including, 2^60
  return (__float_as_uint(P) - lo) < span && (__float_as_uint(S) - lo) < span &&
         __builtin_fabsf(b) <= 80.0f;
}
__device__ __forceinline__ float bsDivEveryday(float P, float S) {
  const float y = __builtin_amdgcn_rcpf(S);
  const float q = P * y;
  const float e = __builtin_fmaf(-q, S, P);
  return __builtin_fmaf(e, y, q);
}
__device__ __forceinline__ float bsLogEveryday(float q) {
  const float y = __builtin_amdgcn_logf(q); // log2
  const float r = y * 0x1.62e42ep-1f;
  float e = __builtin_fmaf(y, 0x1.62e42ep-1f, -r);
  e = __builtin_fmaf(y, 0x1.efa39ep-25f, e);
  return r + e;
}
__device__ __forceinline__ float bsExpEveryday(float b) {
  const float p = b * 0x1.715476p+0f; // b log2(e), then its rounding error
  float e = __builtin_fmaf(b, 0x1.715476p+0f, -p);
  e = __builtin_fmaf(b, 0x1.4ae0bep-26f, e);
  const float n = __builtin_rintf(p);
  const float v = __builtin_amdgcn_exp2f((p - n) + e);
  return __builtin_ldexpf(v, int(n));
}

template <typename W, bool EVERYDAY>
__device__ __forceinline__ void
blackScholesOne(float P, float S, float T, float mr, W sigSigTwo,
                const double *erfTab, float &call, float &put) {
  const float b = T * mr;
  const float a = EVERYDAY ? bsLogEveryday(bsDivEveryday(P, S)) : logf(P / S);
  const W z = W(T) * sigSigTwo;
  const W c = W(0.25) * z;
  const W y = BsMath<W>::rsqrt_(z);
  const float amb = a - b;
  const W w1 = (W(amb) + c) * y;
  const W w2 = (W(amb) - c) * y;
  const W d1 = BsMath<W>::cdfTerm(w1, erfTab); // 0.5 + 0.5 * erf(w1)
  const W d2 = BsMath<W>::cdfTerm(w2, erfTab);
  const float Se = (EVERYDAY ? bsExpEveryday(b) : expf(b)) * S;
  const W r = W(P) * d1 - W(Se) * d2;
  const bool nan = BsMath<W>::eitherNaN(w1, w2);
  call = nan ? __builtin_nanf("") : float(r);
  put = nan ? __builtin_nanf("") : float(r - W(P) + W(Se));
}

// One trip of VEC options per lane.  The everyday forms are taken when every
// lane of the wave qualifies, so each version stays one straight-line block.
template <typename W, int VEC, typename V>
__device__ __forceinline__ void bsTrip(const V &P, const V &S, const V &T,
                                       float mr, W sigSigTwo,
                                       const double *erfTab, V &c, V &u) {
  bool everyday = true;
#pragma unroll
  for (int k = 0; k < VEC; ++k)
    everyday = everyday && bsEveryday(P[k], S[k], T[k] * mr);
  if (__builtin_amdgcn_ballot_w64(!everyday) == 0) {
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      float ck, uk;
      blackScholesOne<W, true>(P[k], S[k], T[k], mr, sigSigTwo, erfTab, ck, uk);
      c[k] = ck;
      u[k] = uk;
    }
  } else {
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      float ck, uk;
      blackScholesOne<W, false>(P[k], S[k], T[k], mr, sigSigTwo, erfTab, ck, uk);
      c[k] = ck;
      u[k] = uk;
    }
  }
}

// VEC options per lane per iteration (float4 or float2 accesses).  Both
// variants take four: the float64 one then needs 78 registers a lane, six
// waves per SIMD without spills (60.6 us on 2^24 options against 63.1 us
// with two options and 64-bit accesses; eight waves spill).
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
      erfTab[sizeof(W) == 8 ? NMK_ERF_NODES * NMK_ERF_ROW : 1];
  if (sizeof(W) == 8) {
    for (int i = threadIdx.x; i < NMK_ERF_NODES * NMK_ERF_ROW;
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
    bsTrip<W, VEC>(P, S, T, mr, sigSigTwo, erfTab, c, u);
    streamStore(c, cv + i);
    streamStore(u, uv + i);
  }
  // n % VEC trailing options, one per lane of the first block.
  const int64_t tail = nvec * VEC + threadIdx.x;
  if (blockIdx.x == 0 && tail < n) {
    float ck, uk;
    blackScholesOne<W, false>(price[tail], strike[tail], t[tail], mr, sigSigTwo,
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
  blackScholes<double, 4>(price, strike, t, rate, volatility, call, put, n);
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
