// Arithmetic shared by the hand-written kernels and the kernels generated
// from Python @kernel bodies.
#pragma once

#include <hip/hip_runtime.h>

namespace nmk {

// sqrt of a double for distances and norms: v_rsq_f64 seed, one coupled
// Newton step on (g ~ sqrt d, h ~ 1 / (2 sqrt d)), then the final fused
// correction g + (d - g*g) * h, which rounds correctly for every input it was
// checked on (bit-equal to the correctly rounded root on all 2^26 distances
// of the benchmark input).  About half the instructions of the library
// routine, which spends the rest on range scaling; inputs outside
// [1e-280, 1e280] (zero, denormals, inf, NaN, negatives) take the library
// routine instead.
__device__ __forceinline__ double sqrtF64(double d) {
  if (!(d >= 1e-280 && d <= 1e280))
    return sqrt(d);
  const double y = __builtin_amdgcn_rsq(d);
  double g = d * y;
  double h = 0.5 * y;
  const double r = __builtin_fma(-h, g, 0.5);
  g = __builtin_fma(g, r, g);
  h = __builtin_fma(h, r, h);
  const double e = __builtin_fma(-g, g, d);
  return __builtin_fma(e, h, g);
}

// float32 log and exp without the range handling of the general routines:
// the same operations in the same order (the extended-precision product with
// ln 2 or log2 e around the hardware log2 / exp2), so the results are the
// general routines' bit for bit wherever the guards hold -- a positive normal
// argument of log within [2^-120, 2^120), |x| <= 80 for exp (the result is a
// normal number).  Everything else -- zeros, infinities, NaNs, denormals,
// overflow -- takes the general routine; that handling is two thirds of its
// instructions.
__device__ __forceinline__ float logNormalF32(float q) {
  const float y = __builtin_amdgcn_logf(q); // log2
  const float r = y * 0x1.62e42ep-1f;
  float e = __builtin_fmaf(y, 0x1.62e42ep-1f, -r);
  e = __builtin_fmaf(y, 0x1.efa39ep-25f, e);
  return r + e;
}
__device__ __forceinline__ float logF32(float q) {
  // positive, exponent in [-120, 120)
  return (__float_as_uint(q) - 0x03800000u) < 0x78000000u ? logNormalF32(q) : logf(q);
}
__device__ __forceinline__ float expNormalF32(float b) {
  const float p = b * 0x1.715476p+0f; // b log2(e), then its rounding error
  float e = __builtin_fmaf(b, 0x1.715476p+0f, -p);
  e = __builtin_fmaf(b, 0x1.4ae0bep-26f, e);
  const float n = __builtin_rintf(p);
  const float v = __builtin_amdgcn_exp2f((p - n) + e);
  return __builtin_ldexpf(v, int(n));
}
__device__ __forceinline__ float expF32(float b) {
  return __builtin_fabsf(b) <= 80.0f ? expNormalF32(b) : expf(b);
}

// 1 / sqrt(z) of a double: the hardware seed (relative error e about 2^-24)
// with one third-order step y (1 + e/2 + 3 e^2 / 8), below one unit in the
// last place.  z = 0 -> inf and z = inf -> 0 come from the seed (e is NaN
// there); a negative or NaN z gives NaN either way.  z must be far enough
// from the ends of the range that z y^2 cannot overflow or underflow:
// [1e-300, 1e300] is; other finite positive z take the division.
__device__ __forceinline__ double rsqrtF64Core(double z) {
  const double y = __builtin_amdgcn_rsq(z);
  const double e = __builtin_fma(-z, y * y, 1.0); // 1 - z y^2
  const double step = __builtin_fma(y * e, __builtin_fma(0.375, e, 0.5), y);
  return __builtin_amdgcn_class(z, 0x260 /* -0 | +0 | +inf */) ? y : step;
}
__device__ __forceinline__ double rsqrtF64(double z) {
  if (z > 0.0 && !(z >= 1e-300 && z <= 1e300))
    return 1.0 / sqrt(z);
  return rsqrtF64Core(z);
}

// log(a / b) in float32 for positive a, b with exponents in [-60, 60) (the
// reciprocal and the quotient are then normal numbers): reciprocal times a
// with one residual correction -- the correctly rounded quotient unless that
// lies within 2e-7 units in the last place of a rounding boundary -- then the
// library's own log arithmetic.
__device__ __forceinline__ bool quotientIsPlainF32(float a, float b) {
  const uint32_t lo = 0x21800000u;   // bits of 2^-60
  const uint32_t span = 0x3C000000u; // up to, not including, 2^60
  return ((__float_as_uint(a) - lo) < span) & ((__float_as_uint(b) - lo) < span);
}
__device__ __forceinline__ float divNormalF32(float a, float b) {
  const float y = __builtin_amdgcn_rcpf(b);
  const float q = a * y;
  const float e = __builtin_fmaf(-q, b, a);
  return __builtin_fmaf(e, y, q);
}
__device__ __forceinline__ float logQuotientF32(float a, float b) {
  return quotientIsPlainF32(a, b) ? logNormalF32(divNormalF32(a, b)) : logf(a / b);
}

} // namespace nmk
