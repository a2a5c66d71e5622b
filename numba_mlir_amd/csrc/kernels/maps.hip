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
  // (a launch has 65535 blocks along y: the rows of a taller array go on
  // along z)
  const int64_t i =
      (int64_t(blockIdx.y) + int64_t(gridDim.y) * blockIdx.z) * blockDim.y + threadIdx.y;
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
// True division of floats (numpy/funcs.py:457ff: the result type of an
// integer division is float64, which is not a same-type map: the generated
// kernels take it).  The quotient is the correctly rounded one.
NMK_DEFINE_MAP2(div, OpDiv, f32, float)
NMK_DEFINE_MAP2(div, OpDiv, f64, double)
NMK_DEFINE_MAP2_FAST(div, OpDiv, f32, float)
NMK_DEFINE_MAP2_FAST(div, OpDiv, f64, double)

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
// The float64 kernel moves 20 bytes per option and, done naively, spends more
// time in the vector ALU than in memory.  It therefore has two bodies:
//
//  * the plain body, taken by a wave whose 256 options all have everyday
//    operands (bsWaveIsPlain): about 60 vector instructions per option,
//      0.5 + 0.5 erf(x)   a degree-5 polynomial for erf / 2 around the nearest
//          of 97 nodes 1/16 apart on [0, 6] (erf_table.inc; absolute error of
//          erf 1.5e-12, far below what a float32 price can show), three
//          128-bit LDS reads of the node's 48-byte row per erf;
//      1 / sqrt(z)        v_rsq_f64 (relative error e about 2^-24) with one
//          second-order step y (1 + e / 2): 3/8 e^2, below 1e-14;
//      P / S, log, exp    the hardware reciprocal, log2 and exp2 with one
//          multiply each: within 2 units in the last place of the float32
//          library results (|rate T| <= 1 keeps exp2's argument small enough
//          for that);
//      P d1 - Se d2       one fused multiply-add in float64: it differs from
//          two roundings by 1e-16 relative, invisible after the result is
//          rounded to float32;
//    none of it can produce or lose a NaN: the operands are positive normal
//    numbers, so z > 0 and w1, w2 are finite;
//
//  * the careful body for any other wave: the float32 library routines, the
//    rsq special cases (z = 0, inf), NaN propagation.  It is kept out of line
//    and rolled up so that it does not cost the plain body registers (54
//    instead of 78 a lane with both inlined).
//
// A wave that contains one odd option computes all its options with the
// careful body, so a price can differ in the last places of float32 from what
// the same option gets inside an all-plain wave; both are within the stated
// tolerance of the reference (rel 1e-4), by orders of magnitude.
//
// The float32 kernel has the same two bodies with every step in float32 (its
// 0.5 + 0.5 erf also comes from the float64 table, rounded once); there the
// careful body takes the plain forms for each option that qualifies on its
// own, so an option gets the same price whichever body its wave runs.
#include "erf_table.inc"

typedef double double2_lds __attribute__((ext_vector_type(2)));

// 0.5 + 0.5 * erf(x) for a non-NaN x on the LDS copy of the table.
__device__ __forceinline__ double bsCdfTerm(double x, const double2_lds *tab) {
  static_assert(NMK_ERF_COEFFS == 6 && NMK_ERF_ROW == 6, "three 128-bit words a row");
  const double ax = __builtin_fmin(__builtin_fabs(x), 6.0);
  // Adding 1.5 * 2^48 rounds ax to the nearest sixteenth and leaves that
  // count, 0..96, in the low word of the sum.
  const double magic = 0x1.8p48;
  const double t = ax + magic;
  const int node = __double2loint(t);
  const double u = ax - (t - magic); // exact, |u| <= 1/32
  const double2_lds *row = tab + __mul24(node, 3);
  const double2_lds c01 = row[0], c23 = row[1], c45 = row[2];
  double p = c45[1];
  p = __builtin_fma(p, u, c45[0]);
  p = __builtin_fma(p, u, c23[1]);
  p = __builtin_fma(p, u, c23[0]);
  p = __builtin_fma(p, u, c01[1]);
  p = __builtin_fma(p, u, c01[0]);
  return 0.5 + __builtin_copysign(p, x);
}

template <typename W> struct BsMath;
template <> struct BsMath<double> {
  // 1 / sqrt(z) for z = T * sigSigTwo: the product of a float and of the
  // double of a float, so z is 0, inf, NaN, negative or a normal double far
  // from the ends of the range, and neither y * y nor z * y * y can overflow.
  // The hardware seed gets one third-order step y (1 + e/2 + 3 e^2 / 8).
  __device__ static __forceinline__ double rsqrt_(double z) {
    const double y = __builtin_amdgcn_rsq(z);
    const double e = __builtin_fma(-z, y * y, 1.0); // 1 - z y^2
    const double step = __builtin_fma(y * e, __builtin_fma(0.375, e, 0.5), y);
    // z = 0 -> inf and z = inf -> 0 come from the seed (e is NaN there);
    // a negative or NaN z gives NaN either way.
    return __builtin_amdgcn_class(z, 0x260 /* -0 | +0 | +inf */) ? y : step;
  }
  __device__ static __forceinline__ double cdfTerm(double x, const double2_lds *tab) {
    return bsCdfTerm(x, tab);
  }
  __device__ static __forceinline__ bool eitherNaN(double a, double b) {
    return __builtin_isunordered(a, b); // bsCdfTerm maps NaN to a number
  }
};
template <> struct BsMath<float> {
  // 1 / sqrt(z) of a positive normal float whose exponent lies within
  // [-120, 122) (z y y then neither overflows nor goes denormal; the plain
  // body's z is the product of a T in [2^-60, 2^60) and 2 vol^2 in
  // [2^-59, 2^61]): the hardware seed (one unit in the last place) with one
  // Newton step, which leaves about half a unit -- what the two roundings of
  // 1.0f / sqrtf(z) leave as well.
  __device__ static __forceinline__ float rsqrtNormal(float z) {
    const float y = __builtin_amdgcn_rsqf(z);
    const float e = __builtin_fmaf(-(z * y), y, 1.0f); // 1 - z y^2
    return __builtin_fmaf(y * e, 0.5f, y);
  }
  // Any z, for options outside the plain body's range: the Newton form for
  // ordinary magnitudes, the library's two operations for the rest (zero,
  // denormals, infinities, NaN, negative numbers).
  __device__ static __forceinline__ float rsqrt_(float z) {
    return (__float_as_uint(z) - 0x21800000u) < 0x3C000000u ? rsqrtNormal(z)
                                                            : 1.0f / sqrtf(z);
  }
  // 0.5 + 0.5 erf(x) rounded once to float32, from the float64 table (the
  // library's erff, two multiply-adds and two roundings later, lands within
  // one unit in the last place of the same value).
  __device__ static __forceinline__ float cdfTerm(float x, const double2_lds *tab) {
    return float(bsCdfTerm(double(x), tab));
  }
  __device__ static __forceinline__ bool eitherNaN(float a, float b) {
    return __builtin_isunordered(a, b); // bsCdfTerm maps NaN to a number
  }
};

// P / S for positive P and S with exponents in [-60, 60) (the quotient and
// the reciprocal are then normal numbers): the reciprocal times P with one
// residual correction, which equals the correctly rounded quotient unless
// that quotient lies within 2e-7 units in the last place of a rounding
// boundary.  With logNormalF32 and expNormalF32 it gives the library's
// log(P / S) and exp(b) bit for bit (NMK_BS_EXACT_F32_STEPS).
__device__ __forceinline__ float bsDivEveryday(float P, float S) {
  const float y = __builtin_amdgcn_rcpf(S);
  const float q = P * y;
  const float e = __builtin_fmaf(-q, S, P);
  return __builtin_fmaf(e, y, q);
}

// One option by the general routines, any operands.
template <typename W>
__device__ __forceinline__ void
blackScholesOne(float P, float S, float T, float mr, W sigSigTwo,
                const double2_lds *erfTab, float &call, float &put) {
  const float b = T * mr;
  const float a = logf(P / S);
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
  const bool nan = BsMath<W>::eitherNaN(w1, w2);
  call = nan ? __builtin_nanf("") : float(r);
  put = nan ? __builtin_nanf("") : float(r - W(P) + W(Se));
}

// ---- float64 typing: plain and careful bodies ------------------------------

struct BsPrices {
  float call, put;
};

__device__ __attribute__((noinline)) BsPrices
bsCareful(float P, float S, float T, float mr, double sigSigTwo,
          const double2_lds *erfTab) {
  BsPrices out;
  blackScholesOne<double>(P, S, T, mr, sigSigTwo, erfTab, out.call, out.put);
  return out;
}

#ifndef NMK_BS_EXACT_F32_STEPS
#define NMK_BS_EXACT_F32_STEPS 0 // 1: library-identical division, log and exp
#endif

__device__ __forceinline__ void
bsPlain(float P, float S, float T, float mr, double sigSigTwo,
        const double2_lds *erfTab, float &call, float &put) {
  const float b = T * mr;
#if NMK_BS_EXACT_F32_STEPS
  const float a = logNormalF32(bsDivEveryday(P, S));
  const float eb = expNormalF32(b);
#else
  const float a =
      __builtin_amdgcn_logf(P * __builtin_amdgcn_rcpf(S)) * 0x1.62e430p-1f;
  const float eb = __builtin_amdgcn_exp2f(b * 0x1.715476p+0f);
#endif
  const double z = double(T) * sigSigTwo;
  const double c = 0.25 * z;
  double y = __builtin_amdgcn_rsq(z);
  const double e = __builtin_fma(-z, y * y, 1.0);
  y = __builtin_fma(y * e, 0.5, y);
  const float amb = a - b;
  const double w1 = (double(amb) + c) * y;
  const double w2 = (double(amb) - c) * y;
  const double d1 = bsCdfTerm(w1, erfTab);
  const double d2 = bsCdfTerm(w2, erfTab);
  const float Se = eb * S;
  const double Pd = double(P), Sed = double(Se);
  const double r = __builtin_fma(Pd, d1, -(Sed * d2));
  call = float(r);
  put = float(r - Pd + Sed);
}

// Wave-uniform constants of the plain-body test: a lane's four options
// qualify when P and S are positive with exponents in [-60, 60) and T lies
// in [2^-60, tLimit), where tLimit keeps |rate T| <= 1 (80 with the exact
// float32 steps); rate must be finite and |volatility| in [2^-50, 2^50], or
// no option qualifies (tLimitBits == 0).
struct BsPlainTest {
  uint32_t tLimitBits;
  // |volatility| must lie in [1 / volSpan, volSpan]: 2^50 where z = 2 vol^2 T
  // is a double, 2^30 where it is a float (z then stays a normal number).
  // (from the limit another instance worked out)
  __device__ __forceinline__ explicit BsPlainTest(uint32_t limitBits)
      : tLimitBits(limitBits) {}
  __device__ __forceinline__ BsPlainTest(float rate, float volatility, float volSpan) {
    const float av = __builtin_fabsf(volatility);
    const bool scalarsOk = __builtin_fabsf(rate) < 0x1p60f &&
                           av >= 1.0f / volSpan && av <= volSpan;
    const float bMax = NMK_BS_EXACT_F32_STEPS ? 80.0f : 1.0f;
    float tLimit =
        __builtin_fminf(0x1p60f, bMax * 0.999f / __builtin_fabsf(rate));
    if (!(tLimit > 0x1p-59f))
      tLimit = 0.f;
    tLimitBits = scalarsOk ? __float_as_uint(tLimit) : 0u;
  }
  // The bit patterns of positive floats order like the floats; negative
  // numbers, infinities and NaNs are above every finite positive pattern, zero
  // and denormals below 2^-60's: three unsigned compares settle twelve values.
  __device__ __forceinline__ bool operator()(const float4_t &P, const float4_t &S,
                                             const float4_t &T) const {
    uint32_t p[4], s[4], t[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      p[k] = __float_as_uint(P[k]);
      s[k] = __float_as_uint(S[k]);
      t[k] = __float_as_uint(T[k]);
    }
    auto lo3 = [](uint32_t a, uint32_t b, uint32_t c) { return min(min(a, b), c); };
    auto hi3 = [](uint32_t a, uint32_t b, uint32_t c) { return max(max(a, b), c); };
    const uint32_t least = lo3(lo3(lo3(p[0], p[1], p[2]), p[3], s[0]),
                               lo3(s[1], s[2], s[3]),
                               lo3(lo3(t[0], t[1], t[2]), t[3], t[3]));
    const uint32_t mostPS = hi3(hi3(p[0], p[1], p[2]), hi3(p[3], s[0], s[1]),
                                max(s[2], s[3]));
    const uint32_t mostT = max(hi3(t[0], t[1], t[2]), t[3]);
    return least >= 0x21800000u /* 2^-60 */ && mostPS < 0x5D800000u /* 2^60 */ &&
           mostT < tLimitBits;
  }
  // The same test for one option.
  __device__ __forceinline__ bool lane(float P, float S, float T) const {
    const uint32_t p = __float_as_uint(P), s = __float_as_uint(S), t = __float_as_uint(T);
    return min(min(p, s), t) >= 0x21800000u && max(p, s) < 0x5D800000u &&
           t < tLimitBits;
  }
};

// ---- float32 typing: the same two bodies with every step in float32 --------
// 0.5 + 0.5 erf comes from the float64 table in both (rounded once to
// float32: the library's erff with its two further roundings lands within a
// unit in the last place of it), so the float32 kernel's arithmetic is a
// subset of the float64 one's and no longer bound by it.
__device__ __forceinline__ void
bsPlain32(float P, float S, float T, float mr, float sigSigTwo,
          const double2_lds *erfTab, float &call, float &put) {
  const float b = T * mr;
#if NMK_BS_EXACT_F32_STEPS
  const float a = logNormalF32(bsDivEveryday(P, S));
  const float eb = expNormalF32(b);
#else
  const float a =
      __builtin_amdgcn_logf(P * __builtin_amdgcn_rcpf(S)) * 0x1.62e430p-1f;
  const float eb = __builtin_amdgcn_exp2f(b * 0x1.715476p+0f);
#endif
  const float z = T * sigSigTwo;
  const float c = 0.25f * z;
  const float y = BsMath<float>::rsqrtNormal(z);
  const float amb = a - b;
  const float w1 = (amb + c) * y;
  const float w2 = (amb - c) * y;
  const float d1 = BsMath<float>::cdfTerm(w1, erfTab);
  const float d2 = BsMath<float>::cdfTerm(w2, erfTab);
  const float Se = eb * S;
  const float r = P * d1 - Se * d2;
  call = r;
  put = r - P + Se;
}

// Any option: the plain forms where the option qualifies for them (so that
// it gets the same price whichever body its wave runs), the general routines
// otherwise.  Out of line, like bsCareful.
__device__ __attribute__((noinline)) BsPrices
bsCareful32(float P, float S, float T, float mr, float sigSigTwo,
            const double2_lds *erfTab, uint32_t tLimitBits) {
  BsPrices out;
  const BsPlainTest test(tLimitBits);
  if (test.lane(P, S, T))
    bsPlain32(P, S, T, mr, sigSigTwo, erfTab, out.call, out.put);
  else
    blackScholesOne<float>(P, S, T, mr, sigSigTwo, erfTab, out.call, out.put);
  return out;
}

// Which 128-bit words a lane takes.  The array is cut into pieces of one
// word a lane of a block (4 KiB of a float32 array at 256 lanes); block b
// takes `count` pieces `distance` pieces apart,
//   piece(b, trip) = (b / distance) * count * distance + b % distance + trip * distance,
// so every run of count * distance pieces is shared out among `distance`
// consecutive blocks.  `distance` is a power of two (quotient and remainder
// are a shift and a mask: a division of 64-bit integers is some 150 scalar
// instructions at the head of every wave, 1 us of this kernel) or at least
// the number of blocks, which is the usual grid-stride walk.  Two trips 128
// pieces (512 KiB) apart measured fastest for the five streams of this kernel
// at 2^24 options: 55.3-55.8 us against 56.4-57.2 for two trips a grid
// apart, 58-62 for pieces 2 to 64 apart and 57-59 for 256 to 1024 (the
// memory-only kernel with the same walk: 53.4-54.0 against 55.2-55.8).
struct BsTrips {
  int distance, count;
  __device__ __forceinline__ int64_t word(int trip) const {
    const uint32_t b = blockIdx.x, d = uint32_t(distance);
    const bool shared = (d & (d - 1)) == 0; // else d >= gridDim.x > b
    const uint32_t run = shared ? b >> (31 - __builtin_clz(d)) : 0;
    const uint32_t place = shared ? b & (d - 1) : b;
    const int64_t piece = int64_t(run) * (int64_t(count) * d) + place + int64_t(trip) * d;
    return piece * blockDim.x + threadIdx.x;
  }
};

// Copies the erf table into LDS (97 rows of three 128-bit words).
__device__ __forceinline__ void bsStageTable(double2_lds *tab) {
  const double2_lds *src = reinterpret_cast<const double2_lds *>(kHalfErfTable);
  for (int i = threadIdx.x; i < NMK_ERF_NODES * 3; i += blockDim.x)
    tab[i] = src[i];
  __syncthreads();
}

// Four options per lane per trip: 128-bit non-temporal loads of price, strike
// and t, stores of call and put.  The launch uses many short blocks (two
// trips a lane at 2^24 options): they stream better than a few long ones.
// Which words a lane's trips take: BsTrips.
__device__ __forceinline__ void
blackScholesWide(const float *__restrict__ price, const float *__restrict__ strike,
                 const float *__restrict__ t, float rate, float volatility,
                 float *__restrict__ call, float *__restrict__ put, int64_t n,
                 BsTrips trips) {
  __shared__ __attribute__((aligned(16))) double2_lds erfTab[NMK_ERF_NODES * 3];
  bsStageTable(erfTab);
  const float mr = -rate;
  const double sigSigTwo = double(volatility * volatility) * 2.0;
  const BsPlainTest isPlain(rate, volatility, 0x1p50f);
  const int64_t nvec = n / 4;
  const float4_t *pv = reinterpret_cast<const float4_t *>(price);
  const float4_t *sv = reinterpret_cast<const float4_t *>(strike);
  const float4_t *tv = reinterpret_cast<const float4_t *>(t);
  float4_t *cv = reinterpret_cast<float4_t *>(call);
  float4_t *uv = reinterpret_cast<float4_t *>(put);
  for (int trip = 0; trip < trips.count; ++trip) {
    const int64_t i = trips.word(trip);
    if (i >= nvec)
      break;
    const float4_t P = streamLoad(pv + i);
    const float4_t S = streamLoad(sv + i);
    const float4_t T = streamLoad(tv + i);
    float4_t c, u;
    if (__builtin_amdgcn_ballot_w64(!isPlain(P, S, T)) == 0) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float ck, uk;
        bsPlain(P[k], S[k], T[k], mr, sigSigTwo, erfTab, ck, uk);
        c[k] = ck;
        u[k] = uk;
      }
    } else {
#pragma unroll 1
      for (int k = 0; k < 4; ++k) {
        const BsPrices o = bsCareful(P[k], S[k], T[k], mr, sigSigTwo, erfTab);
        c[k] = o.call;
        u[k] = o.put;
      }
    }
    streamStore(c, cv + i);
    streamStore(u, uv + i);
  }
  // n % 4 trailing options, one per lane of the first block.
  const int64_t tail = nvec * 4 + threadIdx.x;
  if (blockIdx.x == 0 && tail < n) {
    const BsPrices o =
        bsCareful(price[tail], strike[tail], t[tail], mr, sigSigTwo, erfTab);
    call[tail] = o.call;
    put[tail] = o.put;
  }
}

__device__ __forceinline__ void
blackScholesNarrow(const float *__restrict__ price, const float *__restrict__ strike,
                   const float *__restrict__ t, float rate, float volatility,
                   float *__restrict__ call, float *__restrict__ put, int64_t n,
                   BsTrips trips) {
  __shared__ __attribute__((aligned(16))) double2_lds erfTab[NMK_ERF_NODES * 3];
  bsStageTable(erfTab);
  const float mr = -rate;
  const float sigSigTwo = (volatility * volatility) * 2.0f;
  const BsPlainTest isPlain(rate, volatility, 0x1p30f);
  const int64_t nvec = n / 4;
  const float4_t *pv = reinterpret_cast<const float4_t *>(price);
  const float4_t *sv = reinterpret_cast<const float4_t *>(strike);
  const float4_t *tv = reinterpret_cast<const float4_t *>(t);
  float4_t *cv = reinterpret_cast<float4_t *>(call);
  float4_t *uv = reinterpret_cast<float4_t *>(put);
  for (int trip = 0; trip < trips.count; ++trip) {
    const int64_t i = trips.word(trip);
    if (i >= nvec)
      break;
    const float4_t P = streamLoad(pv + i);
    const float4_t S = streamLoad(sv + i);
    const float4_t T = streamLoad(tv + i);
    float4_t c, u;
    if (__builtin_amdgcn_ballot_w64(!isPlain(P, S, T)) == 0) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        float ck, uk;
        bsPlain32(P[k], S[k], T[k], mr, sigSigTwo, erfTab, ck, uk);
        c[k] = ck;
        u[k] = uk;
      }
    } else {
#pragma unroll 1
      for (int k = 0; k < 4; ++k) {
        const BsPrices o =
            bsCareful32(P[k], S[k], T[k], mr, sigSigTwo, erfTab, isPlain.tLimitBits);
        c[k] = o.call;
        u[k] = o.put;
      }
    }
    streamStore(c, cv + i);
    streamStore(u, uv + i);
  }
  const int64_t tail = nvec * 4 + threadIdx.x;
  if (blockIdx.x == 0 && tail < n) {
    const BsPrices o = bsCareful32(price[tail], strike[tail], t[tail], mr, sigSigTwo,
                                   erfTab, isPlain.tLimitBits);
    call[tail] = o.call;
    put[tail] = o.put;
  }
}

extern "C" __global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(6, 8))) void
nmk_black_scholes_f32_w64(const float *price, const float *strike,
                          const float *t, float rate, float volatility,
                          float *call, float *put, int64_t n, int distance,
                          int trips) {
  blackScholesWide(price, strike, t, rate, volatility, call, put, n,
                   BsTrips{distance, trips});
}

extern "C" __global__ __launch_bounds__(256)
__attribute__((amdgpu_waves_per_eu(6, 8))) void
nmk_black_scholes_f32_w32(const float *price, const float *strike,
                          const float *t, float rate, float volatility,
                          float *call, float *put, int64_t n, int distance,
                          int trips) {
  blackScholesNarrow(price, strike, t, rate, volatility, call, put, n,
                     BsTrips{distance, trips});
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

// Copy of nbytes bytes between any two device-visible buffers (host <-> device
// staging: one side is pinned host memory).  Where source and destination sit
// alike within a 128-bit word (the host places the staged bytes so), the bytes
// up to the first word boundary and behind the last one go singly and all
// between as 128-bit words; otherwise everything goes by single bytes.
NMK_KERNEL(256)
nmk_copy_bytes(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
               int64_t nbytes) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  const int64_t first = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const uintptr_t s = reinterpret_cast<uintptr_t>(src);
  const uintptr_t d = reinterpret_cast<uintptr_t>(dst);
  int64_t head = 0, nvec = 0;
  if (((s ^ d) & 15u) == 0) {
    head = int64_t((16u - (s & 15u)) & 15u);
    if (head > nbytes)
      head = nbytes;
    nvec = (nbytes - head) / 16;
  }
  for (int64_t i = first; i < head; i += stride)
    dst[i] = src[i];
  const int4_t *sv = reinterpret_cast<const int4_t *>(src + head);
  int4_t *dv = reinterpret_cast<int4_t *>(dst + head);
  for (int64_t i = first; i < nvec; i += stride)
    dv[i] = sv[i];
  for (int64_t i = head + nvec * 16 + first; i < nbytes; i += stride)
    dst[i] = src[i];
}

// Fills n 32-bit words with a value (used to zero ticket counters: a
// hipMemset node would not be safe inside a captured graph).
NMK_KERNEL(256) nmk_fill_u32(uint32_t *dst, uint32_t value, int64_t n) {
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += stride)
    dst[i] = value;
}
