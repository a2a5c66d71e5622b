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
  const int64_t row = blockLinearXY() * (4 / WPR) + wave / WPR;
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

// The block-per-row kernels also come capped at three and at four waves a
// SIMD (three or four blocks a CU): with the eight that fit, the memory
// system queues more loads than it can use.  Which cap wins depends on how
// many 16 KiB batches a row holds; the host chooses (measured on MI355X,
// 8 / 4 / 3 waves: [16384, 8192] 78.6 / 76.6 / 74.5 us, [16384, 12288]
// 117.1 / 115.1 / 112.9, [32768, 4096] 78.5 / 74.2 / 84.4, [65536, 4096]
// 156 / 146 / 167; rows that do not end on a batch and rows of four batches
// or more are as fast or faster uncapped).
#define NMK_DEFINE_ROWSUM(NAME, NORM, WPR, WAVES)                              \
  extern "C" __global__ __launch_bounds__(256)                                 \
  __attribute__((amdgpu_waves_per_eu(1, WAVES))) void                          \
  NAME(const float *x, float *out, int64_t rows, int64_t cols, int64_t ld,     \
       int32_t vec) {                                                          \
    rowSumF32<NORM, WPR>(x, out, rows, cols, ld, vec);                         \
  }
NMK_DEFINE_ROWSUM(nmk_sum_axis1_f32, false, 1, 8)
NMK_DEFINE_ROWSUM(nmk_sum_axis1_wide_f32, false, 4, 8)
NMK_DEFINE_ROWSUM(nmk_sum_axis1_wide_w4_f32, false, 4, 4)
NMK_DEFINE_ROWSUM(nmk_sum_axis1_wide_w3_f32, false, 4, 3)
NMK_DEFINE_ROWSUM(nmk_norm2_axis1_f32, true, 1, 8)
NMK_DEFINE_ROWSUM(nmk_norm2_axis1_wide_f32, true, 4, 8)
NMK_DEFINE_ROWSUM(nmk_norm2_axis1_wide_w4_f32, true, 4, 4)
NMK_DEFINE_ROWSUM(nmk_norm2_axis1_wide_w3_f32, true, 4, 3)

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
// (Six loads in flight measured fastest on MI355X, 80.7 us for [16384, 8192]
// against 82.1 with sixteen and 84 with five; other shapes gain up to 5 %.)
#ifndef NMK_AX0_UNROLL
#define NMK_AX0_UNROLL 6 // row loads in flight per lane
#endif

// The counter of a strip: those of neighbouring strips, whose blocks end
// together, lie 256 bytes apart (device-wide atomics on one such line are
// served one after the other).  strip < 4096.
__device__ __forceinline__ uint32_t *stripTicket(uint32_t *tickets, int64_t strip) {
  return tickets + (strip % 64) * 64 + strip / 64;
}

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
    // the wave's last rows of the chunk (fewer than a full group), together
    int4_t v[NMK_AX0_UNROLL - 1];
#pragma unroll
    for (int u = 0; u < NMK_AX0_UNROLL - 1; ++u) {
      v[u] = int4_t{0, 0, 0, 0};
      if (r + 4 * u < rEnd)
        v[u] = *reinterpret_cast<const int4_t *>(p + u * step);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      int64_t s = 0;
#pragma unroll
      for (int u = 0; u < NMK_AX0_UNROLL - 1; ++u)
        s += int64_t(v[u][k]);
      acc[k] += s;
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
    isLast = drawLastTicket(stripTicket(tickets, strip), gridDim.y) ? 1u : 0u;
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
    publish(stripTicket(tickets, strip), 0u);
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
    isLast = drawLastTicketSpread(ticket, gridDim.x, blockIdx.x) ? 1u : 0u;
  }
  __syncthreads();
  if (!isLast)
    return;
  float s = 0.f;
  for (int64_t b = threadIdx.x; b < int64_t(gridDim.x); b += blockDim.x)
    s += collect(partial + b);
  s = blockAllReduce<256>(s, AddOp(), slots);
  if (threadIdx.x == 0)
    out[0] = SQUARE_ROOT_OF_SQUARES ? sqrtf(s) : s;
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
// Covers every (op, dtype, axis) combination; a full reduction is nKeep == 1.
// vec != 0 (the host has checked: sr == 1, x 16-byte aligned, sk a multiple
// of the elements in a 128-bit word): lanes read 128-bit words, four in
// flight, the elements beyond the last whole word one by one.
template <typename IN> struct WordOf {
  static constexpr int N = 16 / sizeof(IN);
  typedef IN type __attribute__((ext_vector_type(16 / sizeof(IN))));
};

template <typename IN, typename ACC, typename Op>
__device__ __forceinline__ ACC foldWord(ACC acc, typename WordOf<IN>::type w, Op op) {
#pragma unroll
  for (int q = 0; q < WordOf<IN>::N; ++q)
    acc = op(acc, ACC(w[q]));
  return acc;
}

// Fold of x[0 .. n), x 16-byte aligned, by LANES lanes (a wave's 64 or a
// block's 256) that read consecutive 128-bit words, four in flight a lane:
// the lanes together stream LANES x 64 contiguous bytes per trip.  `id` is
// the lane's index among them; every lane returns its share.
template <int LANES, typename IN, typename ACC, typename Op>
__device__ __forceinline__ ACC foldWords(const IN *__restrict__ x, int64_t n, int id,
                                         ACC init, Op op) {
  typedef typename WordOf<IN>::type Word;
  constexpr int N = WordOf<IN>::N;
  const Word *w = reinterpret_cast<const Word *>(x);
  const int64_t words = n / N;
  ACC a0 = init, a1 = init, a2 = init, a3 = init;
  int64_t i = id;
  for (; i + 3 * LANES < words; i += 4 * LANES) {
    const Word v0 = __builtin_nontemporal_load(w + i);
    const Word v1 = __builtin_nontemporal_load(w + i + LANES);
    const Word v2 = __builtin_nontemporal_load(w + i + 2 * LANES);
    const Word v3 = __builtin_nontemporal_load(w + i + 3 * LANES);
    a0 = foldWord<IN>(a0, v0, op);
    a1 = foldWord<IN>(a1, v1, op);
    a2 = foldWord<IN>(a2, v2, op);
    a3 = foldWord<IN>(a3, v3, op);
  }
  for (; i < words; i += LANES)
    a0 = foldWord<IN>(a0, __builtin_nontemporal_load(w + i), op);
  for (int64_t r = words * N + id; r < n; r += LANES)
    a1 = op(a1, ACC(x[r]));
  return op(op(a0, a1), op(a2, a3));
}

// The same over elements `stride` apart, one element a load.
template <int LANES, typename IN, typename ACC, typename Op>
__device__ __forceinline__ ACC foldElements(const IN *__restrict__ x, int64_t n,
                                            int64_t stride, int id, ACC init, Op op) {
  ACC a0 = init, a1 = init, a2 = init, a3 = init;
  int64_t r = id;
  for (; r + 3 * LANES < n; r += 4 * LANES) {
    const IN v0 = x[r * stride], v1 = x[(r + LANES) * stride],
             v2 = x[(r + 2 * LANES) * stride], v3 = x[(r + 3 * LANES) * stride];
    a0 = op(a0, ACC(v0));
    a1 = op(a1, ACC(v1));
    a2 = op(a2, ACC(v2));
    a3 = op(a3, ACC(v3));
  }
  for (; r < n; r += LANES)
    a0 = op(a0, ACC(x[r * stride]));
  return op(op(a0, a1), op(a2, a3));
}

// mode bit 0 (the host has checked: sr == 1, x 16-byte aligned, sk a multiple
// of the elements in a 128-bit word): 128-bit loads.  mode bit 1: a block,
// not a wave, per kept index (long rows: the block streams 16 KiB of its row
// per trip).
template <typename IN, typename ACC, typename Op>
__device__ __forceinline__ void
reduceStrided(const IN *x, ACC *out, int64_t nKeep, int64_t nRed, int64_t sk,
              int64_t sr, int64_t so, int32_t mode, ACC init, Op op) {
  __shared__ ACC slots[256 / NMK_WAVE];
  const bool vec = mode & 1;
  if (mode & 4) {
    // Short runs (a few coordinates or features a row): 2^(mode >> 8)
    // adjacent lanes a kept index, so that a wave reads whole runs of
    // neighbouring kept indices side by side; the group's lanes meet through
    // lane exchanges.
    const int gShift = mode >> 8, G = 1 << gShift;
    const int g = threadIdx.x & (G - 1);
    const int64_t k = (blockLinearXY() * blockDim.x + threadIdx.x) >> gShift;
    const bool live = k < nKeep; // (the others still take part in the exchanges)
    const IN *p = x + (live ? k : 0) * sk;
    ACC acc = init;
    for (int64_t r = g; r < nRed; r += G)
      acc = op(acc, ACC(p[r * sr]));
    for (int off = G >> 1; off > 0; off >>= 1)
      acc = op(acc, __shfl_xor(acc, off, NMK_WAVE));
    if (live && g == 0)
      out[k * so] = acc;
    return;
  }
  if (mode & 2) {
    const int64_t k = blockLinearXY();
    if (k >= nKeep)
      return;
    const IN *p = x + k * sk;
    ACC acc = vec ? foldWords<256, IN, ACC>(p, nRed, threadIdx.x, init, op)
                  : foldElements<256, IN, ACC>(p, nRed, sr, threadIdx.x, init, op);
    acc = blockAllReduce<256>(acc, op, slots);
    if (threadIdx.x == 0)
      out[k * so] = acc;
    return;
  }
  const int lane = threadIdx.x % NMK_WAVE;
  const int64_t k =
      blockLinearXY() * (blockDim.x / NMK_WAVE) + threadIdx.x / NMK_WAVE;
  if (k >= nKeep)
    return;
  const IN *p = x + k * sk;
  ACC acc = vec ? foldWords<NMK_WAVE, IN, ACC>(p, nRed, lane, init, op)
                : foldElements<NMK_WAVE, IN, ACC>(p, nRed, sr, lane, init, op);
  acc = waveAllReduce(acc, op);
  if (lane == 0)
    out[k * so] = acc;
}

// Generic reduction over the slow axis of a matrix whose kept index has unit
// stride (column sums of a row-major matrix, row sums of a column-major one):
// out[chunk * nKeep + k] = fold_{r in chunk} op(x[r * ld + k]); with more than
// one chunk the same kernel folds the partial results.
// vec == 0: a block owns 256 consecutive kept indices, one a lane, and a
// chunk of rowsPerChunk reduced indices, eight loads in flight per lane.
// vec != 0 (the host has checked: x 16-byte aligned, ld and nKeep multiples
// of the elements in a 128-bit word): a block owns a strip of 64 words (1 KiB
// of every row), a word a lane; its four waves take interleaved rows of the
// chunk, eight loads in flight per lane, and meet in LDS.
template <typename IN, typename ACC, typename Op>
__device__ __forceinline__ void
reduceColumns(const IN *__restrict__ x, ACC *__restrict__ out, int64_t nRed,
              int64_t nKeep, int64_t ld, int64_t rowsPerChunk, int32_t vec, ACC init,
              Op op) {
  int64_t r = int64_t(blockIdx.y) * rowsPerChunk;
  int64_t rEnd = r + rowsPerChunk;
  if (rEnd > nRed)
    rEnd = nRed;
  if (vec) {
    typedef typename WordOf<IN>::type Word;
    constexpr int N = WordOf<IN>::N;
    constexpr int WAVES = 256 / NMK_WAVE;
    constexpr int U = 8;
    __shared__ ACC meet[WAVES][NMK_WAVE * N];
    const int lane = threadIdx.x % NMK_WAVE;
    const int wave = threadIdx.x / NMK_WAVE;
    const int64_t k = (int64_t(blockIdx.x) * NMK_WAVE + lane) * N;
    ACC a[N];
#pragma unroll
    for (int q = 0; q < N; ++q)
      a[q] = init;
    if (k < nKeep) {
      r += wave;
      const IN *p = x + r * ld + k;
      const int64_t step = WAVES * ld;
      for (; r + WAVES * (U - 1) < rEnd; r += WAVES * U) {
        Word v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
          v[u] = __builtin_nontemporal_load(reinterpret_cast<const Word *>(p + u * step));
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
          for (int q = 0; q < N; ++q)
            a[q] = op(a[q], ACC(v[u][q]));
        p += U * step;
      }
      for (; r < rEnd; r += WAVES) {
        const Word v = __builtin_nontemporal_load(reinterpret_cast<const Word *>(p));
#pragma unroll
        for (int q = 0; q < N; ++q)
          a[q] = op(a[q], ACC(v[q]));
        p += step;
      }
    }
#pragma unroll
    for (int q = 0; q < N; ++q)
      meet[wave][lane * N + q] = a[q];
    __syncthreads();
    for (int c = threadIdx.x; c < NMK_WAVE * N; c += 256) {
      const int64_t kc = int64_t(blockIdx.x) * NMK_WAVE * N + c;
      if (kc < nKeep)
        out[int64_t(blockIdx.y) * nKeep + kc] =
            op(op(meet[0][c], meet[1][c]), op(meet[2][c], meet[3][c]));
    }
    return;
  }
  const int64_t k = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (k >= nKeep)
    return;
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
// x[c * chunk .. min(n, (c + 1) * chunk)), one block per chunk (its 256
// lanes stream 16 KiB per trip).  A full reduction is this kernel followed by
// the strided one over the partial results.  vec != 0 (the host has checked:
// x 16-byte aligned, chunk a multiple of the elements in a 128-bit word):
// 128-bit loads.
template <typename IN, typename ACC, typename Op>
__device__ __forceinline__ void
reduceChunks(const IN *__restrict__ x, ACC *__restrict__ out, int64_t n,
             int64_t chunk, int64_t nChunks, int32_t vec, ACC init, Op op) {
  __shared__ ACC slots[256 / NMK_WAVE];
  const int64_t c = blockIdx.x;
  if (c >= nChunks)
    return;
  const int64_t i = c * chunk;
  int64_t end = (c + 1) * chunk;
  if (end > n)
    end = n;
  ACC acc = vec ? foldWords<256, IN, ACC>(x + i, end - i, threadIdx.x, init, op)
                : foldElements<256, IN, ACC>(x + i, end - i, 1, threadIdx.x, init, op);
  acc = blockAllReduce<256>(acc, op, slots);
  if (threadIdx.x == 0)
    out[c] = acc;
}

#define NMK_DEFINE_REDUCE(OPNAME, OP, INIT, TNAME, IN, ACC)                    \
  NMK_KERNEL(256)                                                              \
  nmk_reduce_##OPNAME##_##TNAME(const IN *x, ACC *out, int64_t nKeep,          \
                                int64_t nRed, int64_t sk, int64_t sr,          \
                                int64_t so, int32_t vec) {                     \
    reduceStrided<IN, ACC>(x, out, nKeep, nRed, sk, sr, so, vec, ACC(INIT),    \
                           OP());                                              \
  }                                                                            \
  NMK_KERNEL(256)                                                              \
  nmk_reducecols_##OPNAME##_##TNAME(const IN *x, ACC *out, int64_t nRed,       \
                                    int64_t nKeep, int64_t ld,                 \
                                    int64_t rowsPerChunk, int32_t vec) {       \
    reduceColumns<IN, ACC>(x, out, nRed, nKeep, ld, rowsPerChunk, vec,         \
                           ACC(INIT), OP());                                   \
  }                                                                            \
  NMK_KERNEL(256)                                                              \
  nmk_reducechunks_##OPNAME##_##TNAME(const IN *x, ACC *out, int64_t n,        \
                                      int64_t chunk, int64_t nChunks,          \
                                      int32_t vec) {                           \
    reduceChunks<IN, ACC>(x, out, n, chunk, nChunks, vec, ACC(INIT), OP());    \
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
