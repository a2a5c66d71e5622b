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
// min / max as the reference folds them: select(x < acc, x, acc) starting from
// +inf (select(x > acc, ...) from -inf), numba_mlir/mlir/builtin/funcs.py:
// 145-146, 176-177 and numpy/funcs.py:283-303 -- a NaN element never wins a
// comparison, so NaNs are skipped (NumPy's amin / amax would propagate them)
// and an all-NaN or empty input gives the starting value.  Here partial
// results meet in any order: a NaN on either side loses.  (a != a is false
// for integers and folds away.)
struct MinOp {
  template <typename T> __device__ __forceinline__ T operator()(T a, T b) const {
    return (b < a || a != a) ? b : a;
  }
};
struct MaxOp {
  template <typename T> __device__ __forceinline__ T operator()(T a, T b) const {
    return (a < b || a != a) ? b : a;
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

// Index of the block in a launch whose blocks are counted along x, then y:
// a launch may run at most 2^32 - 1 work-items along a dimension (the
// dispatch packet counts them in 32 bits), so a kernel with a block per row
// of a very tall matrix gets its blocks in an x-by-y grid.
__device__ __forceinline__ int64_t blockLinearXY() {
  return int64_t(blockIdx.x) + int64_t(gridDim.x) * blockIdx.y;
}

// ---------------------------------------------------------------------------
// Hand-off of per-block partial results to the last block of a launch.
//
// Every value that crosses blocks moves through agent-scope atomic accesses:
// partials are published with agent-scope stores (written through the XCD's
// L2), the ticket is an agent-scope add, and the block that draws the last
// ticket reads the partials back with agent-scope loads (served past the
// XCD's L2).  No value is ever accumulated with an atomic; the ticket only
// orders blocks.
//
// Two ways to order "my partials, then my ticket":
//
//  NMK_HANDOFF_RELEASE == 0 (default).  Every publishing wave waits until its
//    stores have been acknowledged (s_waitcnt vmcnt(0): a written-through
//    store is acknowledged once it is visible device-wide), the block meets
//    at a barrier, one thread draws the ticket with a relaxed add.  Compiler
//    fences on both sides of the wait keep the stores above it and the add
//    below it, so the order in the instruction stream is the order written
//    here; that an acknowledged agent-scope store is visible to a later
//    agent-scope load of another CU is a property of the hardware, not of
//    the language's memory model, which would call this a race.
//
//  NMK_HANDOFF_RELEASE == 1.  The ticket is an agent-scope RELEASE add and
//    the last block issues an agent-scope ACQUIRE fence: correct by the
//    memory model alone.  The release writes back the whole L2 of the XCD
//    (buffer_wbl2) once per block, under the blocks that are still
//    streaming; measured on MI355X: sqrt(sum(x*x)) over 512 MiB 78 -> 89 us,
//    column sums 82 -> 89 us.  Built as a second code object of the
//    reduction kernels ("reduce_release"), which the offload library carries
//    and a tuning knob selects; a GPU test holds the two code objects to
//    identical bits on the full-size benchmark reductions.
#ifndef NMK_HANDOFF_RELEASE
#define NMK_HANDOFF_RELEASE 0
#endif

template <typename T> __device__ __forceinline__ void publish(T *p, T v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T> __device__ __forceinline__ T collect(const T *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Called by every thread that has publish()ed, before the barrier (or, in a
// single publishing thread, before the draw).
__device__ __forceinline__ void awaitStores() {
#if !NMK_HANDOFF_RELEASE
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0); // vmcnt(0) expcnt(0) lgkmcnt(0)
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
#endif
}

// Draws the calling block's ticket: ONE thread, after awaitStores() and a
// barrier behind the block's publish() calls.  True in the block that drew
// the last of `count` tickets; its other threads may collect() after the
// next barrier.
__device__ __forceinline__ bool drawLastTicket(uint32_t *ticket,
                                               uint32_t count) {
#if NMK_HANDOFF_RELEASE
  const uint32_t mine = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELEASE,
                                               __HIP_MEMORY_SCOPE_AGENT);
  const bool last = mine == count - 1;
  if (last)
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  return last;
#else
  const uint32_t mine = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
  __atomic_signal_fence(__ATOMIC_SEQ_CST); // collect() stays below the draw
  return mine == count - 1;
#endif
}

// The same for launches of many blocks that end together.  Device-wide
// atomics on one 256-byte line of memory are served one after the other,
// about 7 ns each: 2048 tickets from one counter added 16 us to a generated
// kernel of 79 us (at the 512 blocks of the kernels here no difference was
// measured).  Here block `me` of `count` draws from one of
// sixteen counters 256 bytes apart (`me` modulo sixteen), and only the last of
// each group draws from the counter behind them.  `tickets`: 17 * 64 counters,
// zero between launches (the blocks that empty a counter put it back).
constexpr uint32_t kTicketGroups = 16;
constexpr uint32_t kTicketStride = 64;
constexpr uint32_t kSpreadTickets = (kTicketGroups + 1) * kTicketStride;

__device__ __forceinline__ bool drawLastTicketSpread(uint32_t *tickets, uint32_t count,
                                                     uint32_t me) {
  const uint32_t group = me % kTicketGroups;
  const uint32_t inGroup = (count - group + kTicketGroups - 1) / kTicketGroups;
  const uint32_t groups = count < kTicketGroups ? count : kTicketGroups;
  if (!drawLastTicket(tickets + group * kTicketStride, inGroup))
    return false;
  publish(tickets + group * kTicketStride, 0u);
  if (!drawLastTicket(tickets + kTicketGroups * kTicketStride, groups))
    return false;
  publish(tickets + kTicketGroups * kTicketStride, 0u);
  return true;
}

} // namespace nmk
