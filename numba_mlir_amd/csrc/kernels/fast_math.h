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

} // namespace nmk
