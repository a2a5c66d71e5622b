// Yardstick kernels for bench.py; not part of the offloaded path.
//
// bench_streams_3r2w_f32 moves exactly the five streams of the Black-Scholes
// kernel -- three float32 arrays read, two written, 128-bit non-temporal
// accesses, four elements a lane per trip, the same grid -- with two
// instructions of arithmetic per output.  Its duration, measured in the same
// run on the same arrays, is the time the memory system needs for that
// pattern: the floor any Black-Scholes kernel over these arrays can reach.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float float4_y __attribute__((ext_vector_type(4)));

extern "C" __global__ __launch_bounds__(256) void
bench_streams_3r2w_f32(const float *__restrict__ a, const float *__restrict__ b,
                       const float *__restrict__ c, float *__restrict__ x,
                       float *__restrict__ y, int64_t n) {
  const int64_t nvec = n / 4;
  const float4_y *av = reinterpret_cast<const float4_y *>(a);
  const float4_y *bv = reinterpret_cast<const float4_y *>(b);
  const float4_y *cv = reinterpret_cast<const float4_y *>(c);
  float4_y *xv = reinterpret_cast<float4_y *>(x);
  float4_y *yv = reinterpret_cast<float4_y *>(y);
  const int64_t stride = int64_t(gridDim.x) * blockDim.x;
  for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec;
       i += stride) {
    const float4_y A = __builtin_nontemporal_load(av + i);
    const float4_y B = __builtin_nontemporal_load(bv + i);
    const float4_y C = __builtin_nontemporal_load(cv + i);
    __builtin_nontemporal_store(A + B, xv + i);
    __builtin_nontemporal_store(C * B, yv + i);
  }
}

// Dispatch-overhead yardsticks: eight work-items write their index into the
// first of 1, 2, 6 or 12 int32 array arguments (the kernels of the
// reference's kernel_dispatcher microbenchmark,
// benchmarks/benchmarks/microbenchmarks/kernel_dispatcher/numba_mlir.py:16-48);
// bench.py times launch -> wait -> destroy event around them.
#define TOUCH_BODY                                                             \
  const int i = blockIdx.x * blockDim.x + threadIdx.x;                         \
  if (i < 8)                                                                   \
    a1[i] = i;
extern "C" __global__ void bench_touch_1(int *a1) { TOUCH_BODY }
extern "C" __global__ void bench_touch_2(int *a1, int *a2) { TOUCH_BODY }
extern "C" __global__ void bench_touch_6(int *a1, int *a2, int *a3, int *a4,
                                         int *a5, int *a6) {
  TOUCH_BODY
}
extern "C" __global__ void bench_touch_12(int *a1, int *a2, int *a3, int *a4,
                                          int *a5, int *a6, int *a7, int *a8,
                                          int *a9, int *a10, int *a11,
                                          int *a12) {
  TOUCH_BODY
}
