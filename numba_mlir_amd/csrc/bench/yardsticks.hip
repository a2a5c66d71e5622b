// Yardstick kernels for bench.py; not part of the offloaded path.
//
// bench_streams_3r2w_f32 moves exactly the five streams of the Black-Scholes
// kernel -- three float32 arrays read, two written, 128-bit non-temporal
// accesses, four elements a lane per trip, the same grid and the same walk
// over the arrays (block b takes `trips` pieces of 256 words `distance`
// pieces apart, as BsTrips in kernels/maps.hip) -- with two instructions of
// arithmetic per output.  Its duration, measured in the same run on the same
// arrays, is the time the memory system needs for that pattern.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float float4_y __attribute__((ext_vector_type(4)));

// (distance: a power of two, or at least the number of blocks)
__device__ __forceinline__ int64_t walkWord(int distance, int trips, int trip) {
  const uint32_t b = blockIdx.x, d = uint32_t(distance);
  const bool shared = (d & (d - 1)) == 0;
  const uint32_t run = shared ? b >> (31 - __builtin_clz(d)) : 0;
  const uint32_t place = shared ? b & (d - 1) : b;
  const int64_t piece = int64_t(run) * (int64_t(trips) * d) + place + int64_t(trip) * d;
  return piece * blockDim.x + threadIdx.x;
}

extern "C" __global__ __launch_bounds__(256) void
bench_streams_3r2w_f32(const float *__restrict__ a, const float *__restrict__ b,
                       const float *__restrict__ c, float *__restrict__ x,
                       float *__restrict__ y, int64_t n, int distance, int trips) {
  const int64_t nvec = n / 4;
  const float4_y *av = reinterpret_cast<const float4_y *>(a);
  const float4_y *bv = reinterpret_cast<const float4_y *>(b);
  const float4_y *cv = reinterpret_cast<const float4_y *>(c);
  float4_y *xv = reinterpret_cast<float4_y *>(x);
  float4_y *yv = reinterpret_cast<float4_y *>(y);
  for (int trip = 0; trip < trips; ++trip) {
    const int64_t i = walkWord(distance, trips, trip);
    if (i >= nvec)
      break;
    const float4_y A = __builtin_nontemporal_load(av + i);
    const float4_y B = __builtin_nontemporal_load(bv + i);
    const float4_y C = __builtin_nontemporal_load(cv + i);
    __builtin_nontemporal_store(A + B, xv + i);
    __builtin_nontemporal_store(C * B, yv + i);
  }
}

// The ladder: R float32 arrays read and W written with the same accesses and
// grid as above (1r0w, 0r1w, 0r2w, 1r1w, 2r1w, 3r1w; bench_streams_3r2w_f32
// is the top rung).  It shows what each additional stream costs on this memory
// system, i.e. whether the five-stream mix is slower than fewer streams of
// the same total size.  A read-only rung consumes what it loads through a
// store that no input ever triggers.
struct StreamSet {
  const float4_y *r[3];
  float4_y *w[2];
};

template <int R, int W>
__device__ __forceinline__ void streamsBody(const StreamSet &p, int64_t n, int distance,
                                            int trips) {
  const int64_t nvec = n / 4;
  for (int trip = 0; trip < trips; ++trip) {
    const int64_t i = walkWord(distance, trips, trip);
    if (i >= nvec)
      break;
    float4_y acc = {1.f, 1.f, 1.f, 1.f};
    float4_y v[R > 0 ? R : 1];
#pragma unroll
    for (int k = 0; k < R; ++k)
      v[k] = __builtin_nontemporal_load(p.r[k] + i);
#pragma unroll
    for (int k = 0; k < R; ++k)
      acc += v[k];
    if (W == 0 && acc[0] == 12345.678f && acc[3] == -1.f)
      p.w[0][i] = acc;
#pragma unroll
    for (int k = 0; k < W; ++k)
      __builtin_nontemporal_store(acc * float(k + 1), p.w[k] + i);
  }
}

#define BENCH_STREAMS(NAME, R, W)                                              \
  extern "C" __global__ __launch_bounds__(256) void NAME(                      \
      const float *a, const float *b, const float *c, float *x, float *y,      \
      int64_t n, int distance, int trips) {                                    \
    StreamSet p;                                                               \
    p.r[0] = reinterpret_cast<const float4_y *>(a);                            \
    p.r[1] = reinterpret_cast<const float4_y *>(b);                            \
    p.r[2] = reinterpret_cast<const float4_y *>(c);                            \
    p.w[0] = reinterpret_cast<float4_y *>(x);                                  \
    p.w[1] = reinterpret_cast<float4_y *>(y);                                  \
    streamsBody<R, W>(p, n, distance, trips);                                  \
  }
BENCH_STREAMS(bench_streams_1r0w_f32, 1, 0)
BENCH_STREAMS(bench_streams_0r1w_f32, 0, 1)
BENCH_STREAMS(bench_streams_0r2w_f32, 0, 2)
BENCH_STREAMS(bench_streams_1r1w_f32, 1, 1)
BENCH_STREAMS(bench_streams_2r1w_f32, 2, 1)
BENCH_STREAMS(bench_streams_3r1w_f32, 3, 1)

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
