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

} // namespace nmk
