// Shared device helpers for the gfx950 kernel families.
//
// All kernels are built for wave64 CDNA4 only, with -ffp-contract=off so a
// separate multiply and add stay two IEEE roundings, as on the reference's
// CPU path (fma contraction there needs fastmath=True; reference:
// numba_mlir/numba_mlir/mlir/tests/test_gpu.py:980-1008).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fast_math.h"

#define NMK_WAVE 64

#define NMK_KERNEL(threads)                                                    \
  extern "C" __global__ __launch_bounds__(threads) void

namespace nmk {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef double double2_t __attribute__((ext_vector_type(2)));
typedef int int4_t __attribute__((ext_vector_type(4)));

// Streaming accesses: data that is touched once carries the non-temporal
// hint on loads and stores (measured on MI355X on the kernels of this
// directory: 5-25 % faster than unhinted stores for the write-heavy ones).
#ifndef NMK_NT_LOAD
#define NMK_NT_LOAD 1
#endif
#ifndef NMK_NT_STORE
#define NMK_NT_STORE 1
#endif

template <typename V> __device__ __forceinline__ V streamLoad(const V *p) {
#if NMK_NT_LOAD
  return __builtin_nontemporal_load(p);
#else
  return *p;
#endif
}

template <typename V> __device__ __forceinline__ void streamStore(V v, V *p) {
#if NMK_NT_STORE
  __builtin_nontemporal_store(v, p);
#else
  *p = v;
#endif
}

// Butterfly reduction over the 64 lanes of a wave; every lane ends up with
// the total.  The combination tree is fixed, so the result is deterministic.
template <typename T, typename Op>
__device__ __forceinline__ T waveAllReduce(T v, Op op) {
#pragma unroll
  for (int off = NMK_WAVE / 2; off > 0; off >>= 1)
    v = op(v, __shfl_xor(v, off, NMK_WAVE));
  return v;
}

struct AddOp {
  template <typename T> __device__ __forceinline__ T operator()(T a, T b) const {
    return a + b;
  }
};
struct MulOp {
  template <typename T> __device__ __forceinline__ T operator()(T a, T b) const {
    return a * b;
  }
};
struct MinOp {
  template <typename T> __device__ __forceinline__ T operator()(T a, T b) const {
    return b < a ? b : a;
  }
};
struct MaxOp {
  template <typename T> __device__ __forceinline__ T operator()(T a, T b) const {
    return a < b ? b : a;
  }
};

// Block-wide reduction for blocks of THREADS (multiple of 64): wave butterfly,
// one LDS slot per wave, then every thread folds the slots in wave order.
template <int THREADS, typename T, typename Op>
__device__ __forceinline__ T blockAllReduce(T v, Op op, T *slots) {
  constexpr int WAVES = THREADS / NMK_WAVE;
  v = waveAllReduce(v, op);
  if (WAVES == 1)
    return v;
  const int wave = threadIdx.x / NMK_WAVE;
  const int lane = threadIdx.x % NMK_WAVE;
  __syncthreads(); // slots may still be read from a previous call
  if (lane == 0)
    slots[wave] = v;
  __syncthreads();
  T total = slots[0];
#pragma unroll
  for (int w = 1; w < WAVES; ++w)
    total = op(total, slots[w]);
  return total;
}

// ---------------------------------------------------------------------------
// Hand-off of per-block partial results to the last block of a launch.
//
// A device-wide fence (__threadfence) writes back and invalidates the whole
// L2 of the XCD; issued once per block it costs more than the reduction
// itself.  Instead every value that crosses blocks moves through agent-scope
// accesses, which the hardware keeps coherent across the XCDs' L2s on their
// own: partials are published with agent-scope stores (written through), the
// publishing wave waits until the stores are acknowledged, then takes a
// ticket with an agent-scope add; the block that draws the last ticket reads
// the partials back with agent-scope loads.  The ticket only orders blocks;
// no value is ever accumulated with an atomic.
template <typename T> __device__ __forceinline__ void publish(T *p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T> __device__ __forceinline__ T collect(const T *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Blocks until every store this wave issued has been acknowledged
// (s_waitcnt vmcnt(0) expcnt(0) lgkmcnt(0)).
__device__ __forceinline__ void awaitStores() { __builtin_amdgcn_s_waitcnt(0); }

__device__ __forceinline__ uint32_t takeTicket(uint32_t *ticket) {
  return __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT);
}

} // namespace nmk
