// Reductions for gfx950: axis sums, full sum-of-squares norm, and generic
// kernels for sum/prod/min/max of every type (strided, column-wise, chunked).
//
// They replace what the reference generates from a linalg.generic with
// `reduction` iterators (reference: numba_mlir/numba_mlir/mlir/numpy/funcs.py:163-229).
// There an axis reduction makes ONE work-item walk a whole row or column
// (mlir_compiler/lib/pipelines/LowerToGpu.cpp:228-245) and a full reduction
// stores per-workgroup partials to host-shared memory and finishes on the
// host (mlir/lib/Conversion/GpuToGpuRuntime.cpp:2161-2277).  Here a wave owns
// a row (axis=1), a block owns a column strip (axis=0), and full reductions
// finish on the device in the last block to arrive: a single launch, no
// arithmetic atomics, a fixed combination order.
//
// Integer reductions accumulate in, and produce, int64 (promote_int,
// numpy/funcs.py:120-123, 176, 210); min/max start from the accumulator
// type's extreme or +-inf (numpy/funcs.py:275-300).
#include "common.h"

#include <limits>

using namespace nmk;

// ---------------------------------------------------------------------------
// out[r] = sum_c x[r * ld + c], float32 (NORM == false), or the fused row
// norm out[r] = sqrt(sum_c x[r,c]^2) (NORM == true: np.sqrt(np.square(a).sum(
// axis=1)), the reference's test_l2_norm, tests/test_gpu.py:2198-2223).
//
// WPR waves of a 4-wave block share one row: WPR = 1 gives a wave per row
// (four rows per block, short rows), WPR = 4 a block per row (long rows: the
// block streams 16 KiB of the row per iteration, measured 4 % faster at 8192
// columns).  When ld and cols are multiples of 4 and x is 16-byte aligned
// (vec != 0) lanes read float4, four loads in flight; lane partials are
// folded pairwise, then a wave butterfly, then the waves of the row in wave
// order.
template <bool NORM, int WPR>
__device__ __forceinline__ void
rowSumF32(const float *__restrict__ x, float *__restrict__ out, int64_t rows,
          int64_t cols, int64_t ld, int32_t vec) {
  __shared__ float slots[4];
  const int lane = threadIdx.x % NMK_WAVE;
  const int wave = threadIdx.x / NMK_WAVE;
  const int sub = wave % WPR; // this wave's share of the row
  const int64_t row = int64_t(blockIdx.x) * (4 / WPR) + wave / WPR;
  constexpr int STEP = NMK_WAVE * WPR;
  float total = 0.f;
  if (row < rows) {
    const float *p = x + row * ld;
    if (vec) {
      const float4_t *pv = reinterpret_cast<const float4_t *>(p);
      const int64_t nvec = cols / 4;
      float4_t a0 = {0.f, 0.f, 0.f, 0.f}, a1 = a0, a2 = a0, a3 = a0;
      int64_t i = sub * NMK_WAVE + lane;
      for (; i + 3 * STEP < nvec; i += 4 * STEP) {
        float4_t v0 = streamLoad(pv + i);
        float4_t v1 = streamLoad(pv + i + STEP);
        float4_t v2 = streamLoad(pv + i + 2 * STEP);
        float4_t v3 = streamLoad(pv + i + 3 * STEP);
        if (NORM) {
          v0 *= v0;
          v1 *= v1;
          v2 *= v2;
          v3 *= v3;
        }
        a0 += v0;
        a1 += v1;
        a2 += v2;
        a3 += v3;
      }
      for (; i < nvec; i += STEP) {
        float4_t v0 = pv[i];
        if (NORM)
          v0 *= v0;
        a0 += v0;
      }
      float4_t a = (a0 + a1) + (a2 + a3);
      total = (a[0] + a[1]) + (a[2] + a[3]);
    } else {
      for (int64_t i = sub * NMK_WAVE + lane; i < cols; i += STEP) {
        const float v = p[i];
        total += NORM ? v * v : v;
      }
    }
    total = waveAllReduce(total, AddOp());
  }
  if (WPR > 1) {
    if (lane == 0)
      slots[wave] = total;
    __syncthreads();
    if (threadIdx.x == 0 && row < rows) {
      float s = slots[0];
#pragma unroll
      for (int w = 1; w < WPR; ++w)
        s += slots[w];
      out[row] = NORM ? sqrtf(s) : s;
    }
  } else if (lane == 0 && row < rows) {
    out[row] = NORM ? sqrtf(total) : total;
  }
}

#define NMK_DEFINE_ROWSUM(NAME, NORM, WPR)                                     \
  NMK_KERNEL(256)                                                              \
  NAME(const float *x, float *out, int64_t rows, int64_t cols, int64_t ld,     \
       int32_t vec) {                                                          \
    rowSumF32<NORM, WPR>(x, out, rows, cols, ld, vec);                         \
  }
NMK_DEFINE_ROWSUM(nmk_sum_axis1_f32, false, 1)
NMK_DEFINE_ROWSUM(nmk_sum_axis1_wide_f32, false, 4)
NMK_DEFINE_ROWSUM(nmk_norm2_axis1_f32, true, 1)
NMK_DEFINE_ROWSUM(nmk_norm2_axis1_wide_f32, true, 4)

// ---------------------------------------------------------------------------
// out[c] = sum_r int64(x[r * ld + c]), int32 input.  Requires cols % 4 == 0,
// ld % 4 == 0 and a 16-byte aligned base (the dispatcher falls back to the
// generic kernel otherwise).
//
// grid.x = column strips of 256 columns (64 lanes x int4 = 1 KiB of a row),
// grid.y = row chunks of rowsPerBlock.  The four waves of a block take
// interleaved rows of the chunk, NMK_AX0_UNROLL row loads in flight per lane, fold
// through LDS, and publish one int64 partial per column to
// partial[chunk][col].  The block that draws the last ticket of its strip
// adds the chunks in index order and writes out[]; it also resets the ticket,
// so the counters are zero again when the kernel ends.
#ifndef NMK_AX0_UNROLL
#define NMK_AX0_UNROLL 16 // row loads in flight per lane
#endif

NMK_KERNEL(256)
nmk_sum_axis0_i32_i64(const int32_t *__restrict__ x, int64_t *__restrict__ out,
                      int64_t rows, int64_t cols, int64_t ld,
                      int64_t rowsPerBlock, int64_t *partial,
                      uint32_t *tickets) {
  __shared__ int64_t fold[4][256];
  __shared__ uint32_t isLast;
  const int lane = threadIdx.x % NMK_WAVE;
  const int wave = threadIdx.x / NMK_WAVE;
  const int64_t strip = blockIdx.x;
  const int64_t chunk = blockIdx.y;
  const int64_t col = strip * 256 + lane * 4;
  int64_t acc[4] = {0, 0, 0, 0};
  if (col < cols) {
    int64_t r = chunk * rowsPerBlock + wave;
    int64_t rEnd = (chunk + 1) * rowsPerBlock;
    if (rEnd > rows)
      rEnd = rows;
    const int32_t *p = x + r * ld + col;
    const int64_t step = 4 * ld; // the block's waves interleave rows
    for (; r + 4 * (NMK_AX0_UNROLL - 1) < rEnd; r += 4 * NMK_AX0_UNROLL) {
      int4_t v[NMK_AX0_UNROLL];
#pragma unroll
      for (int u = 0; u < NMK_AX0_UNROLL; ++u)
        v[u] = streamLoad(reinterpret_cast<const int4_t *>(p + u * step));
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        int64_t s = 0;
#pragma unroll
        for (int u = 0; u < NMK_AX0_UNROLL; ++u)
          s += int64_t(v[u][k]);
        acc[k] += s;
      }
      p += NMK_AX0_UNROLL * step;
    }
    for (; r < rEnd; r += 4) {
      int4_t v0 = *reinterpret_cast<const int4_t *>(p);
#pragma unroll
      for (int k = 0; k < 4; ++k)
        acc[k] += int64_t(v0[k]);
      p += step;
    }
  }
#pragma unroll
  for (int k = 0; k < 4; ++k)
    fold[wave][lane * 4 + k] = acc[k];
  __syncthreads();
  const int64_t myCol = strip * 256 + threadIdx.x;
  if (myCol < cols) {
    int64_t s = (fold[0][threadIdx.x] + fold[1][threadIdx.x]) +
                (fold[2][threadIdx.x] + fold[3][threadIdx.x]);
    publish(partial + chunk * cols + myCol, s);
  }
  awaitStores();
  __syncthreads();
  if (threadIdx.x == 0)
    isLast = drawLastTicket(&tickets[strip], gridDim.y) ? 1u : 0u;
  __syncthreads();
  if (!isLast)
    return;
  if (myCol < cols) {
    const int64_t nChunks = gridDim.y;
    const int64_t *p = partial + myCol;
    int64_t s = 0;
    int64_t c = 0;
    for (; c + 8 <= nChunks; c += 8) {
      int64_t v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        v[u] = collect(p + (c + u) * cols);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        s += v[u];
    }
    for (; c < nChunks; ++c)
      s += collect(p + c * cols);
    out[myCol] = s;
  }
  if (threadIdx.x == 0)
    publish(&tickets[strip], 0u);
}

// ---------------------------------------------------------------------------
// out[0] = sqrt(sum_i x[i] * x[i]) or sum_i x[i], float32, n contiguous
// elements (np.sqrt(np.sum(x * x)): the square is fused into the reduction as
// the reference's elementwise fusion does,
// mlir_compiler/lib/pipelines/PlierToLinalg.cpp:3149-3199; the sqrt of the 0-d
// result is the scalar path, numpy/funcs.py:364-368).
//
// Each block streams 16 KiB pieces (256 lanes x 4 float4, vec != 0 needs a
// 16-byte aligned base), piece index strided by the grid, float32 lane
// partials folded pairwise, block tree, one published partial per block; the
// block that draws the last ticket folds the partials in block order and
// applies sqrtf.  The result depends on the grid size only.
template <bool SQUARE_ROOT_OF_SQUARES>
__device__ __forceinline__ void
fullSumF32(const float *__restrict__ x, float *__restrict__ out, int64_t n,
           int32_t vec, float *partial, uint32_t *ticket) {
  __shared__ float slots[4];
  __shared__ uint32_t isLast;
  float total = 0.f;
  int64_t done = 0;
  if (vec) {
    const float4_t *pv = reinterpret_cast<const float4_t *>(x);
    const int64_t nvec = n / 4;
    const int64_t nPieces = nvec / 1024;
    float4_t a0 = {0.f, 0.f, 0.f, 0.f}, a1 = a0, a2 = a0, a3 = a0;
    for (int64_t piece = blockIdx.x; piece < nPieces; piece += gridDim.x) {
      const float4_t *q = pv + piece * 1024 + threadIdx.x;
      float4_t v0 = streamLoad(q);
      float4_t v1 = streamLoad(q + 256);
      float4_t v2 = streamLoad(q + 512);
      float4_t v3 = streamLoad(q + 768);
      if (SQUARE_ROOT_OF_SQUARES) {
        v0 *= v0;
        v1 *= v1;
        v2 *= v2;
        v3 *= v3;
      }
      a0 += v0;
      a1 += v1;
      a2 += v2;
      a3 += v3;
    }
    // Vectors past the last whole piece: grid-strided, one per lane.
    for (int64_t i = nPieces * 1024 + int64_t(blockIdx.x) * blockDim.x +
                     threadIdx.x;
         i < nvec; i += int64_t(gridDim.x) * blockDim.x) {
      float4_t v0 = pv[i];
      if (SQUARE_ROOT_OF_SQUARES)
        v0 *= v0;
      a0 += v0;
    }
    float4_t a = (a0 + a1) + (a2 + a3);
    total = (a[0] + a[1]) + (a[2] + a[3]);
    done = nvec * 4;
  }
  for (int64_t i = done + int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += int64_t(gridDim.x) * blockDim.x) {
    float v = x[i];
    total += SQUARE_ROOT_OF_SQUARES ? v * v : v;
  }
  total = blockAllReduce<256>(total, AddOp(), slots);
  if (threadIdx.x == 0) {
    publish(partial + blockIdx.x, total);
    awaitStores();
    isLast = drawLastTicket(ticket, gridDim.x) ? 1u : 0u;
  }
  __syncthreads();
  if (!isLast)
    return;
  float s = 0.f;
  for (int64_t b = threadIdx.x; b < int64_t(gridDim.x); b += blockDim.x)
    s += collect(partial + b);
  s = blockAllReduce<256>(s, AddOp(), slots);
  if (threadIdx.x == 0) {
    out[0] = SQUARE_ROOT_OF_SQUARES ? sqrtf(s) : s;
    publish(ticket, 0u);
  }
}

NMK_KERNEL(256)
nmk_norm2_f32(const float *x, float *out, int64_t n, int32_t vec,
              float *partial, uint32_t *ticket) {
  fullSumF32<true>(x, out, n, vec, partial, ticket);
}

NMK_KERNEL(256)
nmk_sum_all_f32(const float *x, float *out, int64_t n, int32_t vec,
                float *partial, uint32_t *ticket) {
  fullSumF32<false>(x, out, n, vec, partial, ticket);
}

// ---------------------------------------------------------------------------
// Generic strided reduction: out[k * so] = fold_r op(x[k * sk + r * sr]) for
// k < nKeep, r < nRed, accumulating in ACC starting from `init`.  One wave per
// kept index; lanes stride over the reduced axis, then a wave butterfly.
// Covers every (op, dtype, axis) combination at modest speed; a full
// reduction is nKeep == 1.
template <typename IN, typename ACC, typename Op>
__device__ __forceinline__ void
reduceStrided(const IN *x, ACC *out, int64_t nKeep, int64_t nRed, int64_t sk,
              int64_t sr, int64_t so, ACC init, Op op) {
  const int lane = threadIdx.x % NMK_WAVE;
  const int64_t k =
      int64_t(blockIdx.x) * (blockDim.x / NMK_WAVE) + threadIdx.x / NMK_WAVE;
  if (k >= nKeep)
    return;
  ACC acc = init, a1 = init, a2 = init, a3 = init;
  const IN *p = x + k * sk;
  int64_t r = lane;
  for (; r + 3 * NMK_WAVE < nRed; r += 4 * NMK_WAVE) { // four loads in flight
    const IN v0 = p[r * sr], v1 = p[(r + NMK_WAVE) * sr],
             v2 = p[(r + 2 * NMK_WAVE) * sr], v3 = p[(r + 3 * NMK_WAVE) * sr];
    acc = op(acc, ACC(v0));
    a1 = op(a1, ACC(v1));
    a2 = op(a2, ACC(v2));
    a3 = op(a3, ACC(v3));
  }
  for (; r < nRed; r += NMK_WAVE)
    acc = op(acc, ACC(p[r * sr]));
  acc = waveAllReduce(op(op(acc, a1), op(a2, a3)), op);
  if (lane == 0)
    out[k * so] = acc;
}

// Generic reduction over the slow axis of a matrix whose kept index has unit
// stride (column sums of a row-major matrix, row sums of a column-major one):
// out[chunk * nKeep + k] = fold_{r in chunk} op(x[r * ld + k]).  A block owns
// 256 consecutive kept indices (adjacent lanes read adjacent elements) and one
// chunk of rowsPerChunk reduced indices, eight loads in flight per lane; with
// more than one chunk the same kernel folds the partial results.
template <typename IN, typename ACC, typename Op>
__device__ __forceinline__ void
reduceColumns(const IN *__restrict__ x, ACC *__restrict__ out, int64_t nRed,
              int64_t nKeep, int64_t ld, int64_t rowsPerChunk, ACC init, Op op) {
  const int64_t k = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (k >= nKeep)
    return;
  int64_t r = int64_t(blockIdx.y) * rowsPerChunk;
  int64_t rEnd = r + rowsPerChunk;
  if (rEnd > nRed)
    rEnd = nRed;
  const IN *p = x + r * ld + k;
  ACC a[8];
#pragma unroll
  for (int u = 0; u < 8; ++u)
    a[u] = init;
  for (; r + 8 <= rEnd; r += 8) {
    IN v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      v[u] = p[u * ld];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      a[u] = op(a[u], ACC(v[u]));
    p += 8 * ld;
  }
  for (; r < rEnd; ++r) {
    a[0] = op(a[0], ACC(*p));
    p += ld;
  }
  out[int64_t(blockIdx.y) * nKeep + k] =
      op(op(op(a[0], a[1]), op(a[2], a[3])), op(op(a[4], a[5]), op(a[6], a[7])));
}

// Generic reduction of a long contiguous run in chunks: out[c] = fold of
// x[c * chunk .. min(n, (c + 1) * chunk)), one wave per chunk, four loads in
// flight per lane.  A full reduction is this kernel followed by the strided
// one over the partial results.
template <typename IN, typename ACC, typename Op>
__device__ __forceinline__ void
reduceChunks(const IN *__restrict__ x, ACC *__restrict__ out, int64_t n,
             int64_t chunk, int64_t nChunks, ACC init, Op op) {
  const int lane = threadIdx.x % NMK_WAVE;
  const int64_t c =
      int64_t(blockIdx.x) * (blockDim.x / NMK_WAVE) + threadIdx.x / NMK_WAVE;
  if (c >= nChunks)
    return;
  int64_t i = c * chunk + lane;
  int64_t end = (c + 1) * chunk;
  if (end > n)
    end = n;
  ACC a0 = init, a1 = init, a2 = init, a3 = init;
  for (; i + 3 * NMK_WAVE < end; i += 4 * NMK_WAVE) {
    const IN v0 = x[i], v1 = x[i + NMK_WAVE], v2 = x[i + 2 * NMK_WAVE],
             v3 = x[i + 3 * NMK_WAVE];
    a0 = op(a0, ACC(v0));
    a1 = op(a1, ACC(v1));
    a2 = op(a2, ACC(v2));
    a3 = op(a3, ACC(v3));
  }
  for (; i < end; i += NMK_WAVE)
    a0 = op(a0, ACC(x[i]));
  ACC acc = waveAllReduce(op(op(a0, a1), op(a2, a3)), op);
  if (lane == 0)
    out[c] = acc;
}

#define NMK_DEFINE_REDUCE(OPNAME, OP, INIT, TNAME, IN, ACC)                    \
  NMK_KERNEL(256)                                                              \
  nmk_reduce_##OPNAME##_##TNAME(const IN *x, ACC *out, int64_t nKeep,          \
                                int64_t nRed, int64_t sk, int64_t sr,          \
                                int64_t so) {                                  \
    reduceStrided<IN, ACC>(x, out, nKeep, nRed, sk, sr, so, ACC(INIT), OP());  \
  }                                                                            \
  NMK_KERNEL(256)                                                              \
  nmk_reducecols_##OPNAME##_##TNAME(const IN *x, ACC *out, int64_t nRed,       \
                                    int64_t nKeep, int64_t ld,                 \
                                    int64_t rowsPerChunk) {                    \
    reduceColumns<IN, ACC>(x, out, nRed, nKeep, ld, rowsPerChunk, ACC(INIT),   \
                           OP());                                              \
  }                                                                            \
  NMK_KERNEL(256)                                                              \
  nmk_reducechunks_##OPNAME##_##TNAME(const IN *x, ACC *out, int64_t n,        \
                                      int64_t chunk, int64_t nChunks) {        \
    reduceChunks<IN, ACC>(x, out, n, chunk, nChunks, ACC(INIT), OP());         \
  }

NMK_DEFINE_REDUCE(sum, AddOp, 0, i32, int32_t, int64_t)
NMK_DEFINE_REDUCE(sum, AddOp, 0, i64, int64_t, int64_t)
NMK_DEFINE_REDUCE(sum, AddOp, 0, f32, float, float)
NMK_DEFINE_REDUCE(sum, AddOp, 0, f64, double, double)
NMK_DEFINE_REDUCE(prod, MulOp, 1, i32, int32_t, int64_t)
NMK_DEFINE_REDUCE(prod, MulOp, 1, i64, int64_t, int64_t)
NMK_DEFINE_REDUCE(prod, MulOp, 1, f32, float, float)
NMK_DEFINE_REDUCE(prod, MulOp, 1, f64, double, double)
NMK_DEFINE_REDUCE(min, MinOp, std::numeric_limits<int64_t>::max(), i32,
                  int32_t, int64_t)
NMK_DEFINE_REDUCE(min, MinOp, std::numeric_limits<int64_t>::max(), i64,
                  int64_t, int64_t)
NMK_DEFINE_REDUCE(min, MinOp, __builtin_inff(), f32, float, float)
NMK_DEFINE_REDUCE(min, MinOp, __builtin_inf(), f64, double, double)
NMK_DEFINE_REDUCE(max, MaxOp, std::numeric_limits<int64_t>::min(), i32,
                  int32_t, int64_t)
NMK_DEFINE_REDUCE(max, MaxOp, std::numeric_limits<int64_t>::min(), i64,
                  int64_t, int64_t)
NMK_DEFINE_REDUCE(max, MaxOp, -__builtin_inff(), f32, float, float)
NMK_DEFINE_REDUCE(max, MaxOp, -__builtin_inf(), f64, double, double)
