// HIP math runtime: device gemm behind mkl_gemm_<dtype>_device
// (include/numba_mlir_hip/MathRuntime.h).
//
// Entry points, argument meaning and layout rules follow the oneMKL-backed
// runtime they replace (reference:
// numba_mlir/numba_mlir/math_runtime/sycl/lib/NumpyLinalg.cpp:67-183); the
// arithmetic is a hand-written LDS-tiled MFMA kernel for gfx950 (fp32 and
// fp64 matrix cores) plus a strided fallback.
#include "numba_mlir_hip/GpuQueueInterface.hpp"
#include "numba_mlir_hip/MathRuntime.h"

#include <hip/hip_runtime.h>
#include <type_traits>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <mutex>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef double doublex4 __attribute__((ext_vector_type(4)));
typedef double doublex2 __attribute__((ext_vector_type(2)));

// fatal_failure of the reference prints to stderr and aborts
// (math_runtime/include/Common.hpp:10-15).
[[noreturn]] void fatal(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  std::vfprintf(stderr, fmt, ap);
  va_end(ap);
  std::fflush(stderr);
  std::abort();
}

void checkHip(hipError_t err, const char *what) {
  if (err != hipSuccess)
    fatal("%s failed: %s (%d)\n", what, hipGetErrorString(err),
          static_cast<int>(err));
}

thread_local const char *lastKernel = "";
thread_local bool lastPacked = false; // operands went through gemm_pack_rows

// ---------------------------------------------------------------------------
// C[M,N] = alpha * A[M,K] * B[K,N] + beta * C with C row-major (ldc) on the
// matrix cores, float32 (v_mfma_f32_32x32x2_f32) or float64
// (v_mfma_f64_16x16x4_f64), accumulating in the operand type.  Each input
// operand may be stored with either of its two dimensions contiguous:
//   A_KC: A(m,k) = A[m * lda + k]   (row-major A)   else A[k * lda + m]
//   B_NC: B(k,n) = B[k * ldb + n]   (row-major B)   else B[n * ldb + k]
// which covers the four transpose cases of a BLAS gemm; a column-major C is
// handled by the host as C^T = B^T A^T.
//
// 256 threads = 4 waves in a 2 x 2 grid; each wave owns TM x TN MFMA tiles of
// edge TILE (32 for float32, 16 for float64), so the block tile is
// (2 TM TILE) x (2 TN TILE).  K advances in slabs of BK elements (16, or 32
// for the large float32 tile).
//
// LDS holds both operands K-major ([k][m] and [k][n], rows padded so that the
// rows one MFMA operand fetch touches fall on different banks): lane l needs
// element (l % TILE) of row (k + l / TILE), a conflict-free ds_read.  Global
// fetches are 128-bit along the operand's contiguous dimension: an operand
// contiguous in m / n is written to LDS as one 128-bit word, one contiguous
// in k is scattered over LDS rows.  Two LDS stages: the next K slab is
// fetched from global memory into registers during the first step of the
// current slab and written to the other stage during its later steps, one
// barrier per slab; every memory instruction is issued behind an MFMA (see
// the slab loop).
//
// MFMA operand layouts (64 lanes):
//   f32 32x32x2: A[l % 32][l / 32], B[l / 32][l % 32],
//                D reg r = D[8*(r/4) + 4*(l/32) + r%4][l % 32]   (16 regs)
//   f64 16x16x4: A[l % 16][l / 16], B[l / 16][l % 16],
//                D reg r = D[4*r + l/16][l % 16]                  (4 regs)
//
// Requirements (checked by the host): leading dimensions multiples of the
// 128-bit vector, A and B 16-byte aligned; M and N multiples of the block
// tile and K % BK == 0, or (GUARD) extents along each operand's contiguous
// dimension multiples of the vector.
template <typename T> struct Mfma;
template <> struct Mfma<float> {
  typedef floatx4 Vec;   // 128-bit global access
  typedef floatx16 Acc;  // one MFMA tile per lane
  static constexpr int TILE = 32, KSTEP = 2, BK = 16, VEC = 4, NACC = 16,
                       PAD = 4;
  // LDS reads after the compiler has paired them: one ds_read2_b32 for two
  // fragments a tile apart.
  static constexpr int fragmentReads(int fragments) { return fragments / 2; }
  __device__ static __forceinline__ Acc mma(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ int accRow(int r, int lane) {
    return 8 * (r / 4) + 4 * (lane / 32) + r % 4;
  }
};
template <> struct Mfma<double> {
  typedef doublex2 Vec;
  typedef doublex4 Acc;
  // PAD 16: consecutive k rows land 32 banks apart for a 128-wide tile
  static constexpr int TILE = 16, KSTEP = 4, BK = 16, VEC = 2, NACC = 4,
                       PAD = 16;
  // one ds_read2_b64 for two fragments a tile apart
  static constexpr int fragmentReads(int fragments) { return fragments / 2; }
  __device__ static __forceinline__ Acc mma(double a, double b, Acc c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ int accRow(int r, int lane) {
    return 4 * r + lane / 16;
  }
};

// One operand's slab of X x BK (X = BM or BN) on its way from global memory
// to LDS[k][x].  NV 128-bit words per thread.
//   K_CONTIG: thread -> (x = tid / (BK/VEC) + X_STEP i, k = VEC (tid % (BK/VEC)) ..)
//   else    : thread -> (k = tid / (X/VEC) + K_ROWS i, x = VEC (tid % (X/VEC)) ..)
// GUARD: the operand need not fill the tile or the last slab; a word that
// lies outside it (words are whole: the host checks that the extents along
// the contiguous dimension are multiples of the word) is read from the
// operand's first word instead and replaced by zeros.
template <typename T, int X, int BK, bool K_CONTIG, bool GUARD> struct SlabFetch {
  typedef Mfma<T> M;
  typedef typename M::Vec Vec;
  static constexpr int NV = X * BK / (M::VEC * 256);
  static constexpr int X_STEP = 256 * M::VEC / BK; // K_CONTIG: x rows per pass
  static constexpr int K_ROWS = 256 * M::VEC / X;     // else: k rows per pass
  static constexpr int WRITES = K_CONTIG ? NV * M::VEC : NV; // LDS instructions
  int x, k;
  const T *base;
  int64_t ld;
  Vec reg[NV];
  const T *first; // GUARD: the operand's first word
  int xLeft;      // GUARD: extent - origin - x: how many x from this thread's on
  int kEnd;       // GUARD: K

  __device__ __forceinline__ void init(const T *p, int64_t ld_, int origin,
                                       int tid, int extent = 0, int K = 0) {
    ld = ld_;
    first = p;
    kEnd = K;
    if (K_CONTIG) {
      x = tid / (BK / M::VEC);
      k = (tid % (BK / M::VEC)) * M::VEC;
      base = p + int64_t(origin + x) * ld + k;
    } else {
      k = tid / (X / M::VEC);
      x = (tid % (X / M::VEC)) * M::VEC;
      base = p + int64_t(k) * ld + origin + x;
    }
    xLeft = extent - origin - x;
  }
  __device__ __forceinline__ void fetch(int k0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const T *src = K_CONTIG ? base + int64_t(X_STEP * i) * ld + k0
                              : base + int64_t(k0 + K_ROWS * i) * ld;
      if (GUARD) {
        const bool inside = K_CONTIG ? (X_STEP * i < xLeft && k0 + k < kEnd)
                                     : (0 < xLeft && k0 + k + K_ROWS * i < kEnd);
        const Vec v = *reinterpret_cast<const Vec *>(inside ? src : first);
#pragma unroll
        for (int q = 0; q < M::VEC; ++q)
          reg[i][q] = inside ? v[q] : T(0);
      } else {
        reg[i] = *reinterpret_cast<const Vec *>(src);
      }
    }
  }
  // Words [i0, i1) of the slab to LDS.
  __device__ __forceinline__ void stash(T (*lds)[X + M::PAD], int i0 = 0,
                                        int i1 = NV) const {
#pragma unroll
    for (int i = i0; i < i1; ++i) {
      if (K_CONTIG) {
#pragma unroll
        for (int q = 0; q < M::VEC; ++q)
          lds[k + q][x + X_STEP * i] = reg[i][q];
      } else {
        *reinterpret_cast<Vec *>(&lds[k + K_ROWS * i][x]) = reg[i];
      }
    }
  }
};

// n consecutive one-instruction groups of the instruction scheduler.
template <int MASK> __device__ __forceinline__ void sched_groups(int n) {
  if (n > 0) __builtin_amdgcn_sched_group_barrier(MASK, 1, 0);
  if (n > 1) __builtin_amdgcn_sched_group_barrier(MASK, 1, 0);
  if (n > 2) __builtin_amdgcn_sched_group_barrier(MASK, 1, 0);
  if (n > 3) __builtin_amdgcn_sched_group_barrier(MASK, 1, 0);
}

// float64 tiles need under 256 registers a lane: two blocks share a CU and
// fill each other's stalls.  float32 256 x 256 tiles take a CU each.
//
// Split K (sliceK > 0): grid.z slices of sliceK elements of K (a multiple of
// BK) each; slice z leaves its unscaled partial product in the workspace,
// W[z][M][N] with row stride ldw, and gemm_splitk_fold adds the slices in
// index order.  Used when the tiles alone would leave most CUs idle.
//
// Even shares (streamSlabs > 0): the work is counted in units of one K slab of
// one block tile, tiles in row-major order, streamSlabs units a tile; the
// launch runs just as many blocks as are resident at once (grid.x of them,
// grid.y = grid.z = 1) and block g takes the units [g U / G, (g + 1) U / G):
// the end of one tile, whole tiles, the beginning of another.  A whole tile
// goes to C as usual; a piece of one is left, unscaled, in the workspace --
// a dense BM x BN tile at W[(2 g + j) BM BN], j = 0 for the block's first
// segment, 1 for a later one (which can only be its last) -- and
// gemm_even_fold adds a tile's pieces in K order.  Used when whole tiles
// would leave the last round of blocks mostly empty (576 tiles on 256 CUs:
// 2.25 rounds) or would not fill the first.
struct EvenShares {
  int slabs;  // K slabs a tile (0: not in use)
  int tilesN; // block tiles along N
};
__host__ __device__ inline int64_t evenSharesStart(int64_t g, int64_t units,
                                                   int64_t blocks) {
  const int64_t scaled = g * units; // (units * blocks stays far below 2^63)
  // (32-bit operands wherever they fit: on the device a division of 64-bit
  // integers is some 150 instructions, and the kernels call this per piece)
  if ((uint64_t(scaled) | uint64_t(blocks)) >> 32)
    return scaled / blocks;
  return int64_t(uint32_t(scaled) / uint32_t(blocks));
}

// GUARD: 0 whole tiles; 1 loads and stores guarded (operands and C of any
// extent); 2 stores alone guarded (operands padded with zeros to whole tiles
// and slabs, C of any extent).
template <typename T, int BK, int TM, int TN, bool A_KC, bool B_NC, int GUARD = 0>
__global__ __launch_bounds__(256, sizeof(T) == 8 ? 2 : 1) void
gemm_mfma(const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C,
          int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, T alpha,
          T beta, int sliceK, T *__restrict__ W, int64_t ldw, EvenShares even) {
  typedef Mfma<T> MF;
  constexpr int TILE = MF::TILE;
  constexpr int BM = 2 * TM * TILE, BN = 2 * TN * TILE;
  __shared__ __attribute__((aligned(16))) T As[2][BK][BM + MF::PAD];
  __shared__ __attribute__((aligned(16))) T Bs[2][BK][BN + MF::PAD];
  if (sliceK > 0) {
    const int k0 = blockIdx.z * sliceK;
    A += A_KC ? int64_t(k0) : int64_t(k0) * lda;
    B += B_NC ? int64_t(k0) * ldb : int64_t(k0);
    K = K - k0 < sliceK ? K - k0 : sliceK;
    C = W + int64_t(blockIdx.z) * int64_t(M) * ldw;
    ldc = ldw;
    alpha = T(1);
    beta = T(0);
  }

  const int tid = threadIdx.x;
  const int lane = tid % 64;
  const int wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;
  const int kLane = lane / TILE, xLane = lane % TILE;

  // This block's units (one segment, the whole of K of one tile, without
  // even shares).
  int64_t unit = 0, unitEnd = 0;
  const int slabsPerTile = even.slabs > 0 ? even.slabs : (K + BK - 1) / BK;
  if (even.slabs > 0) {
    const int64_t units = int64_t((M + BM - 1) / BM) * even.tilesN * even.slabs;
    unit = evenSharesStart(blockIdx.x, units, gridDim.x);
    unitEnd = evenSharesStart(int64_t(blockIdx.x) + 1, units, gridDim.x);
  } else {
    unitEnd = slabsPerTile;
  }
#pragma nounroll
  for (int segment = 0; unit < unitEnd; ++segment) {
  int bm = blockIdx.y * BM, bn = blockIdx.x * BN;
  int slab0 = 0, slab1 = slabsPerTile; // the K slabs of this segment
  if (even.slabs > 0) {
    const int64_t tile = unit / even.slabs;
    slab0 = int(unit - tile * even.slabs);
    slab1 = unitEnd - unit < even.slabs - slab0 ? slab0 + int(unitEnd - unit) : even.slabs;
    bm = int(tile / even.tilesN) * BM;
    bn = int(tile % even.tilesN) * BN;
    if (segment > 0)
      __syncthreads(); // every wave is done with the last segment's LDS slabs
  }
  unit += slab1 - slab0;
  const bool piece = even.slabs > 0 && !(slab0 == 0 && slab1 == even.slabs);

  SlabFetch<T, BM, BK, A_KC, GUARD == 1> fa;
  SlabFetch<T, BN, BK, !B_NC, GUARD == 1> fb;
  fa.init(A, lda, bm, tid, M, K);
  fb.init(B, ldb, bn, tid, N, K);

  typename MF::Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < MF::NACC; ++r)
        acc[i][j][r] = T(0);

  // Operand fragments of one step, double-buffered in registers.
  T a[2][TM], b[2][TN];
  auto fragments = [&](int stage, int slot, int kk) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
      a[slot][i] = As[stage][kk + kLane][wm * (TM * TILE) + i * TILE + xLane];
#pragma unroll
    for (int j = 0; j < TN; ++j)
      b[slot][j] = Bs[stage][kk + kLane][wn * (TN * TILE) + j * TILE + xLane];
  };

  fa.fetch(slab0 * BK);
  fb.fetch(slab0 * BK);
  fa.stash(As[0]);
  fb.stash(Bs[0]);
  __syncthreads();
  fragments(0, 0, 0);

  // One slab: STEPS = BK / KSTEP steps of TM x TN MFMAs.  A wave is alone on
  // its SIMD, so whatever it issues between two MFMAs beyond the ~60 cycles
  // one MFMA runs leaves the matrix core idle: a clump of eight global loads
  // or twelve LDS writes costs several hundred cycles a slab.  The
  // directives at the end of the slab spread every memory instruction over
  // the MFMAs, one or two behind each:
  //   step 0          the global loads of the next slab (into registers),
  //   every step      the LDS reads of the next step's fragments; in the last
  //                   step, behind the slab's one barrier, those of the next
  //                   slab's first step, so their latency runs under the last
  //                   step's MFMAs,
  //   the steps before the last, from the middle on
  //                   the LDS writes of the next slab to the other stage (the
  //                   loads have had a third of a slab or more to arrive).
  // The compiler cannot tell the two LDS stages apart, so LDS reads and
  // writes keep their program order: each sits in the step it is issued in.
  auto slab = [&](int s, auto more) {
    constexpr bool MORE = decltype(more)::value;
    constexpr int STEPS = BK / MF::KSTEP, NMFMA = TM * TN;
    static_assert(STEPS >= 4 && STEPS % 2 == 0, "fragment slots alternate over a slab");
    constexpr int WRITE_STEPS = STEPS / 2 - 1, WRITE_FROM = STEPS - 1 - WRITE_STEPS;
    const int cur = (s - slab0) & 1;
    if (MORE) {
      fa.fetch((s + 1) * BK);
      fb.fetch((s + 1) * BK);
    }
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      if (st + 1 < STEPS) {
        fragments(cur, (st + 1) & 1, (st + 1) * MF::KSTEP);
      } else if (MORE) {
        __syncthreads();
        fragments(cur ^ 1, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = MF::mma(a[st & 1][i], b[st & 1][j], acc[i][j]);
      const int t = st - WRITE_FROM;
      if (MORE && t >= 0 && t < WRITE_STEPS) {
        fa.stash(As[cur ^ 1], t * fa.NV / WRITE_STEPS, (t + 1) * fa.NV / WRITE_STEPS);
        fb.stash(Bs[cur ^ 1], t * fb.NV / WRITE_STEPS, (t + 1) * fb.NV / WRITE_STEPS);
      }
    }
    // Issue order (groups of the instruction scheduler; masks: 0x008 MFMA,
    // 0x020 global load, 0x100 LDS read, 0x200 LDS write).  Read counts are
    // of instructions after the compiler has paired them, write counts
    // before (it pairs some); a group that finds no instruction stays empty.
    constexpr int READS = MF::fragmentReads(TM + TN);
    constexpr int LOADS = MORE ? fa.NV + fb.NV : 0;
    static_assert(READS + LOADS <= 4 * NMFMA &&
                      READS + fa.WRITES + fb.WRITES <= 4 * NMFMA * WRITE_STEPS,
                  "at most four memory instructions behind one MFMA");
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      const int reads = st + 1 < STEPS || MORE ? READS : 0;
      const int loads = st == 0 ? LOADS : 0;
      const int t = st - WRITE_FROM;
      const int writes =
          !MORE || t < 0 || t >= WRITE_STEPS
              ? 0
              : ((t + 1) * fa.NV / WRITE_STEPS - t * fa.NV / WRITE_STEPS) * (fa.WRITES / fa.NV) +
                    ((t + 1) * fb.NV / WRITE_STEPS - t * fb.NV / WRITE_STEPS) * (fb.WRITES / fb.NV);
      // reads behind the first MFMAs of the step, writes behind the rest
      const int head = reads < NMFMA / 2 ? reads : NMFMA / 2, tail = NMFMA - head;
#pragma unroll
      for (int m = 0; m < NMFMA; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (m < head)
          sched_groups<0x100>((m + 1) * reads / head - m * reads / head);
        else
          sched_groups<0x200>((m - head + 1) * writes / tail - (m - head) * writes / tail);
        sched_groups<0x020>((m + 1) * loads / NMFMA - m * loads / NMFMA);
      }
    }
  };
  for (int s = slab0; s + 1 < slab1; ++s)
    slab(s, std::true_type());
  slab(slab1 - 1, std::false_type());

  // A whole tile goes to C, scaled; a piece of one goes to its workspace
  // slot as a dense BM x BN block, unscaled.
  T *out = C + int64_t(bm) * ldc + bn;
  int64_t ldo = ldc;
  T scale = alpha, keep = beta;
  int rowsLeft = GUARD != 0 ? M - bm : BM, colsLeft = GUARD != 0 ? N - bn : BN;
  if (piece) {
    out = W + (int64_t(blockIdx.x) * 2 + (segment > 0 ? 1 : 0)) * (BM * BN);
    ldo = BN;
    scale = T(1);
    keep = T(0);
    rowsLeft = BM;
    colsLeft = BN;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = wn * (TN * TILE) + j * TILE + xLane;
#pragma unroll
      for (int r = 0; r < MF::NACC; ++r) {
        const int row = wm * (TM * TILE) + i * TILE + MF::accRow(r, lane);
        if (GUARD != 0 && !(row < rowsLeft && col < colsLeft))
          continue;
        T *dst = out + int64_t(row) * ldo + col;
        T v = scale * acc[i][j][r];
        if (keep != T(0))
          v += keep * *dst;
        *dst = v;
      }
    }
  }
  } // segments
}

// ---------------------------------------------------------------------------
// The tiles that gemm_mfma's even shares cut into pieces: C[tile] = alpha *
// (piece + piece + ...) + beta * C[tile], pieces in K order (the order of the
// blocks that computed them: a fixed order).  One block per tile row-chunk:
// grid (tiles, BM * BN / (256 * VEC * ROWS))...  A thread owns one 128-bit
// word of the tile; stores to C are per element and stay inside C.
template <typename T, int BM, int BN>
__global__ __launch_bounds__(256) void
gemm_even_fold(const T *__restrict__ W, int64_t blocks, int slabs, int tilesN,
               int64_t units, T *__restrict__ C, int M, int N, int64_t ldc,
               T alpha, T beta) {
  typedef typename Mfma<T>::Vec Vec;
  constexpr int VEC = Mfma<T>::VEC;
  const int64_t tile = blockIdx.x;
  const int64_t u0 = tile * slabs, u1 = u0 + slabs;
  // the block whose share holds the tile's first unit
  int64_t g = evenSharesStart(u0, blocks, units); // u0 * blocks / units
  while (g > 0 && evenSharesStart(g, units, blocks) > u0)
    --g;
  while (g + 1 < blocks && evenSharesStart(g + 1, units, blocks) <= u0)
    ++g;
  {
    const int64_t b = evenSharesStart(g, units, blocks);
    const int64_t e = evenSharesStart(g + 1, units, blocks);
    if (b <= u0 && e >= u1)
      return; // one block computed the whole tile and stored it itself
  }
  const int word = blockIdx.y * 256 + threadIdx.x; // of BM * BN / VEC
  const int row = word / (BN / VEC), col = (word % (BN / VEC)) * VEC;
  Vec sum;
#pragma unroll
  for (int q = 0; q < VEC; ++q)
    sum[q] = T(0);
  for (; g < blocks; ++g) {
    const int64_t b = evenSharesStart(g, units, blocks);
    if (b >= u1)
      break;
    const T *slot = W + (g * 2 + (b >= u0 ? 0 : 1)) * int64_t(BM * BN);
    sum += *reinterpret_cast<const Vec *>(slot + row * BN + col);
  }
  const int gr = int(tile / tilesN) * BM + row, gc = int(tile % tilesN) * BN + col;
  if (gr >= M)
    return;
  T *dst = C + int64_t(gr) * ldc + gc;
#pragma unroll
  for (int q = 0; q < VEC; ++q) {
    if (gc + q < N) {
      T v = alpha * sum[q];
      if (beta != T(0))
        v += beta * dst[q];
      dst[q] = v;
    }
  }
}

// ---------------------------------------------------------------------------
// word = row * perRow + inRow, for a lane's word of a matrix of perRow words a
// row: with 32-bit operands wherever they fit (a division of 64-bit integers
// is a hundred vector instructions a lane, 0.8 us of a fold of 1024 x 1024).
__device__ __forceinline__ void splitWord(int64_t word, int64_t perRow, int64_t &row,
                                          int64_t &inRow) {
  if ((uint64_t(word) | uint64_t(perRow)) >> 32) {
    row = word / perRow;
    inRow = word % perRow;
  } else {
    const uint32_t w = uint32_t(word), p = uint32_t(perRow);
    row = w / p;
    inRow = w % p;
  }
}

// ---------------------------------------------------------------------------
// C[m][n] = alpha * (W[0][m][n] + W[1][m][n] + ...) + beta * C[m][n]: the
// slices of a split-K product added in index order (a fixed order, so the
// result does not depend on which block finished first).  One thread per
// 128-bit word of a row of W (ldw and the slice stride are multiples of the
// word); stores to C are per element, C may end inside the last word.
template <typename T>
__global__ __launch_bounds__(256) void
gemm_splitk_fold(const T *__restrict__ W, int slices, int64_t sliceStride,
                 int64_t ldw, T *__restrict__ C, int M, int N, int64_t ldc,
                 T alpha, T beta) {
  typedef typename Mfma<T>::Vec Vec;
  constexpr int VEC = Mfma<T>::VEC;
  const int wordsPerRow = (N + VEC - 1) / VEC;
  const int64_t word = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (word >= int64_t(M) * wordsPerRow)
    return;
  int64_t row, inRow;
  splitWord(word, wordsPerRow, row, inRow);
  const int m = int(row);
  const int n = int(inRow) * VEC;
  const T *src = W + int64_t(m) * ldw + n;
  Vec sum = *reinterpret_cast<const Vec *>(src);
  for (int z = 1; z < slices; ++z)
    sum += *reinterpret_cast<const Vec *>(src + z * sliceStride);
  T *dst = C + int64_t(m) * ldc + n;
#pragma unroll
  for (int q = 0; q < VEC; ++q) {
    if (n + q < N) {
      T v = alpha * sum[q];
      if (beta != T(0))
        v += beta * dst[q];
      dst[q] = v;
    }
  }
}

// ---------------------------------------------------------------------------
// Any shape, any strides (element strides per dimension), float or double:
// classic 32 x 32 LDS tiling, one output per thread x 4 rows, bounds checked.
// Used for the transposed / column-major / ragged cases the MFMA kernel does
// not take.
template <typename T>
__global__ __launch_bounds__(256) void
gemm_generic(const T *A, const T *B, T *C, int64_t M, int64_t N, int64_t K,
             int64_t as0, int64_t as1, int64_t bs0, int64_t bs1, int64_t cs0,
             int64_t cs1, T alpha, T beta, int64_t kSlice, T *part) {
  constexpr int TILE = 32;
  __shared__ T As[TILE][TILE + 1];
  __shared__ T Bs[TILE][TILE + 1];
  const int tx = threadIdx.x % TILE; // column within the tile
  const int ty = threadIdx.x / TILE; // 0..7, rows ty, ty+8, ty+16, ty+24
  // The tiles in row-major order, counted along the grid's x, then y (a tall
  // matrix has more tile rows than grid.y holds).
  const int64_t tilesN = (N + TILE - 1) / TILE;
  const int64_t tile = int64_t(blockIdx.x) + int64_t(gridDim.x) * blockIdx.y;
  if (tile >= tilesN * ((M + TILE - 1) / TILE))
    return;
  const int64_t row0 = tile / tilesN * TILE;
  const int64_t col0 = tile % tilesN * TILE, col = col0 + tx;
  // Adjacent lanes read along each operand's unit stride: A along k or along
  // m, B along n or along k (a transposed tall operand, X.T @ Y, is read in
  // whole rows instead of one element per row).
  const bool aAlongM = as0 == 1 && as1 != 1;
  const bool bAlongK = bs0 == 1 && bs1 != 1;
  T acc[4] = {T(0), T(0), T(0), T(0)};
  // blockIdx.z: the slice of K (multiples of the tile), whose partial sums go
  // to part + z M N for gemm_thin_fold when there is more than one
  const int64_t kBegin = int64_t(blockIdx.z) * kSlice;
  if (kBegin + kSlice < K)
    K = kBegin + kSlice;
  for (int64_t k0 = kBegin; k0 < K; k0 += TILE) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = ty + 8 * i;
      if (aAlongM) {
        const int64_t ar = row0 + tx, ak = k0 + r;
        As[tx][r] = (ar < M && ak < K) ? A[ar * as0 + ak * as1] : T(0);
      } else {
        const int64_t ar = row0 + r, ak = k0 + tx;
        As[r][tx] = (ar < M && ak < K) ? A[ar * as0 + ak * as1] : T(0);
      }
      if (bAlongK) {
        const int64_t bk = k0 + tx, bn = col0 + r;
        Bs[tx][r] = (bk < K && bn < N) ? B[bk * bs0 + bn * bs1] : T(0);
      } else {
        const int64_t bk = k0 + r;
        Bs[r][tx] = (bk < K && col < N) ? B[bk * bs0 + col * bs1] : T(0);
      }
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TILE; ++k) {
      const T b = Bs[k][tx];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc[i] += As[ty + 8 * i][k] * b;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t row = row0 + ty + 8 * i;
    if (row < M && col < N && part) {
      part[(int64_t(blockIdx.z) * M + row) * N + col] = acc[i];
    } else if (row < M && col < N) {
      T *dst = C + row * cs0 + col * cs1;
      T v = alpha * acc[i];
      if (beta != T(0))
        v += beta * *dst;
      *dst = v;
    }
  }
}

// ---------------------------------------------------------------------------
// Z[M, N] = alpha X[M, K] Y[K, N] + beta Z for a tall X with few columns and a
// small Y (K, N <= 32): coordinates times a small matrix.  The work is moving
// X and Z once; a 128 x 128 tile would spend its time on rows of zeros and on
// filling and draining its pipeline every four slabs.  A block takes tiles of
// 128 rows or more in turn: the tile of X goes to LDS with coalesced loads, Y sits in
// LDS for the whole launch, and every lane computes four adjacent columns of
// one row at a time (one read of X and one 128-bit read of Y per four
// multiply-adds).  X has unit stride along k, Z along n; Y any strides.
template <typename T>
__global__ __launch_bounds__(256) void
gemm_skinny(const T *__restrict__ X, int64_t ldx, const T *__restrict__ Y, int64_t yk,
            int64_t yn, T *__restrict__ Z, int64_t ldz, int64_t M, int N, int K, T alpha,
            T beta, int wordStores) {
  constexpr int MAXD = 32, XS_WORDS = 128 * (MAXD + 1);
  typedef T Four __attribute__((ext_vector_type(4)));
  __shared__ __attribute__((aligned(32))) T Ys[MAXD][MAXD];
  // rows of K + 1 words (an odd pitch for K a power of two: lanes on
  // different rows read different banks); the fewer columns, the more rows
  // a tile holds, so that a block always has some 16 KiB of X in flight
  __shared__ T Xs[XS_WORDS];
  const int pitch = K + 1;
  const int ROWS = XS_WORDS / pitch;
  const int tid = threadIdx.x;
  for (int i = tid; i < MAXD * MAXD; i += 256) {
    const int k = i / MAXD, n = i % MAXD;
    Ys[k][n] = (k < K && n < N) ? Y[k * yk + n * yn] : T(0);
  }
  // Lanes per row of X and per row of Z: the next powers of two (shifts and
  // masks instead of divisions by K and N; the lanes beyond idle).
  int kLanes = 1, kShift = 0;
  while (kLanes < K)
    kLanes <<= 1, ++kShift;
  const int groups = (N + 3) / 4; // of four adjacent columns
  int gLanes = 1, gShift = 0;
  while (gLanes < groups)
    gLanes <<= 1, ++gShift;
  const int kk = tid & (kLanes - 1), rk = tid >> kShift, rkStep = 256 >> kShift;
  const int gg = tid & (gLanes - 1), rg = tid >> gShift, rgStep = 256 >> gShift;
  const int n0 = gg * 4;
  const int64_t tiles = (M + ROWS - 1) / ROWS;
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int64_t row0 = tile * ROWS;
    __syncthreads(); // the last tile's rows are used up (and Ys is written)
    if (kk < K)
      for (int r = rk; r < ROWS; r += 8 * rkStep) { // eight loads in flight a lane
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int rr = r + u * rkStep;
          v[u] = rr < ROWS && row0 + rr < M
                     ? __builtin_nontemporal_load(X + (row0 + rr) * ldx + kk)
                     : T(0);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int rr = r + u * rkStep;
          if (rr < ROWS)
            Xs[rr * pitch + kk] = v[u];
        }
      }
    __syncthreads();
    if (gg < groups)
      for (int r = rg; r < ROWS && row0 + r < M; r += rgStep) {
        Four acc = {T(0), T(0), T(0), T(0)};
        const T *xr = Xs + r * pitch;
        for (int k = 0; k < K; ++k)
          acc += xr[k] * *reinterpret_cast<const Four *>(&Ys[k][n0]);
        T *dst = Z + (row0 + r) * ldz + n0;
        if (wordStores) {
          Four v = alpha * acc;
          if (beta != T(0))
            v += beta * *reinterpret_cast<const Four *>(dst);
          __builtin_nontemporal_store(v, reinterpret_cast<Four *>(dst));
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (n0 + j < N) {
              T v = alpha * acc[j];
              if (beta != T(0))
                v += beta * dst[j];
              dst[j] = v;
            }
        }
      }
  }
}

// ---------------------------------------------------------------------------
// The same the other way round: Z[M, N] = alpha X[M, K] Y[K, N] + beta Z for a
// small X (M, K <= 32) and a long Y with unit stride along n.  A lane owns a
// column n: it reads Y(k, n) for every k (adjacent lanes adjacent words),
// keeps the M sums of its column in registers and stores them down the
// column.  X sits in LDS.  MB: M rounded up to 4, 8, 16 or 32, the
// accumulators a lane holds.
template <typename T, int MB>
__global__ __launch_bounds__(256) void
gemm_wide(const T *__restrict__ X, int64_t xm, int64_t xk, const T *__restrict__ Y,
          int64_t ldy, T *__restrict__ Z, int64_t ldz, int M, int64_t N, int K, T alpha,
          T beta) {
  typedef T Four __attribute__((ext_vector_type(4)));
  // X transposed and padded with zeros: four sums advance with one 128-bit
  // read that is the same for every lane
  __shared__ __attribute__((aligned(32))) T Xs[32][MB];
  for (int i = threadIdx.x; i < 32 * MB; i += 256) {
    const int k = i / MB, m = i % MB;
    Xs[k][m] = (k < K && m < M) ? X[m * xm + k * xk] : T(0);
  }
  __syncthreads();
  const int64_t n = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (n >= N)
    return;
  Four acc[MB / 4];
#pragma unroll
  for (int q = 0; q < MB / 4; ++q)
    acc[q] = Four{T(0), T(0), T(0), T(0)};
  const T *y = Y + n;
#pragma unroll 4
  for (int k = 0; k < K; ++k) {
    const T v = __builtin_nontemporal_load(y + k * ldy);
#pragma unroll
    for (int q = 0; q < MB / 4; ++q)
      acc[q] += *reinterpret_cast<const Four *>(&Xs[k][4 * q]) * v;
  }
  T *z = Z + n;
#pragma unroll
  for (int m = 0; m < MB; ++m)
    if (m < M) {
      T v = alpha * acc[m / 4][m % 4];
      if (beta != T(0))
        v += beta * z[m * ldz];
      __builtin_nontemporal_store(v, z + m * ldz);
    }
}

// ---------------------------------------------------------------------------
// A long matrix times a thin one (a matrix times a vector or a few of them):
// the work is reading the long matrix once.  W elements a load: the 128-bit
// word when the rows of the long matrix begin and end on words, 1 otherwise.
template <typename T, int W> struct ThinWord {
  typedef T Type __attribute__((ext_vector_type(W)));
  __device__ static __forceinline__ void load(const T *p, T (&out)[W]) {
    const Type v = __builtin_nontemporal_load(reinterpret_cast<const Type *>(p));
#pragma unroll
    for (int q = 0; q < W; ++q)
      out[q] = v[q];
  }
};
template <typename T> struct ThinWord<T, 1> {
  __device__ static __forceinline__ void load(const T *p, T (&out)[1]) {
    out[0] = __builtin_nontemporal_load(p);
  }
};

// O(r, j) = alpha * sum_k S(r, k) P(k, j) + beta * O(r, j) for a long S with
// unit stride along k (rows `ld` apart) and a thin P (n <= NB columns, any
// strides).  G adjacent lanes (a power of two up to a wave, or the 256 of the
// block when there are few rows) share a set of R rows: each takes every G-th
// word along k of those rows and the rows of P that go with it (P is read by
// every group: it stays in the caches), the G partial sums meet through lane
// exchanges (and LDS, for the block), and the first lane of the group stores.
// R rows at once divide the reads of P by R; 8 / R steps along k are in
// flight at once, eight loads of S a lane.  PV: how P is read -- 0 by
// element; 1 by rows (unit stride along j, n == NB, rows aligned to
// min(16, row) bytes); 2 by words along k (unit stride along k, columns
// aligned to the word; W > 1).
template <typename T, int NB, int R, int W, int PV>
__global__ __launch_bounds__(256) void
gemm_thin_rows(const T *__restrict__ S, int64_t ld, int64_t rows, int64_t K,
               const T *__restrict__ P, int64_t pk, int64_t pn, int n, T *__restrict__ O,
               int64_t orow, int64_t ocol, T alpha, T beta, int G, int gShift,
               int64_t sliceWords, T *__restrict__ part) {
  constexpr int U = R < 8 ? 8 / R : 1;
  constexpr int ROW_BYTES = NB * int(sizeof(T)) < 16 ? NB * int(sizeof(T)) : 16;
  typedef T PRow __attribute__((ext_vector_type(NB), aligned(ROW_BYTES)));
  typedef T PWord __attribute__((ext_vector_type(W)));
  __shared__ T cross[4][R * NB];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool wholeBlock = G == 256;
  const int g = wholeBlock ? int(threadIdx.x) : lane & (G - 1);
  const int64_t set = wholeBlock ? int64_t(blockIdx.x)
                                 : (int64_t(blockIdx.x) * 4 + wave) * (64 >> gShift) +
                                       (lane >> gShift);
  const int64_t r0 = set * R;
  const T *row[R];
#pragma unroll
  for (int r = 0; r < R; ++r) // (rows beyond the last read the last: nothing of theirs is stored)
    row[r] = S + (r0 + r < rows ? r0 + r : rows - 1) * ld;
  T acc[R][NB];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int j = 0; j < NB; ++j)
      acc[r][j] = T(0);
  // blockIdx.y: the slice of K (sliceWords words each; the last one takes the
  // elements behind the last whole word), whose sums go to part for
  // gemm_thin_fold when there is more than one
  const int64_t allWords = K / W;
  const int64_t wordsBegin = int64_t(blockIdx.y) * sliceWords;
  const int64_t words = wordsBegin + sliceWords < allWords ? wordsBegin + sliceWords : allWords;
  // The trips along k start at a different place for every set of rows and
  // wrap round: rows a power of two apart begin in the same memory channel,
  // and sets that all walked from k = 0 would queue on it.
  const int64_t tripWords = int64_t(G) * U;
  const int64_t trips = words > wordsBegin ? (words - wordsBegin + tripWords - 1) / tripWords : 0;
  const int64_t firstTrip = trips ? (set * 5) % trips : 0;
  for (int64_t trip = 0; trip < trips; ++trip) {
    const int64_t turned = trip + firstTrip < trips ? trip + firstTrip : trip + firstTrip - trips;
    const int64_t w0 = wordsBegin + turned * tripWords + g;
    T x[U][R][W];
    T p[U][W][NB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t w = w0 + int64_t(u) * G;
      if (w < words) {
#pragma unroll
        for (int r = 0; r < R; ++r)
          ThinWord<T, W>::load(row[r] + w * W, x[u][r]);
        if (PV == 1) {
#pragma unroll
          for (int q = 0; q < W; ++q) {
            const PRow v = *reinterpret_cast<const PRow *>(P + (w * W + q) * pk);
#pragma unroll
            for (int j = 0; j < NB; ++j)
              p[u][q][j] = v[j];
          }
        } else if (PV == 2) {
#pragma unroll
          for (int j = 0; j < NB; ++j)
            if (j < n) {
              const PWord v = *reinterpret_cast<const PWord *>(P + w * W + j * pn);
#pragma unroll
              for (int q = 0; q < W; ++q)
                p[u][q][j] = v[q];
            }
        } else {
#pragma unroll
          for (int q = 0; q < W; ++q)
#pragma unroll
            for (int j = 0; j < NB; ++j)
              if (j < n)
                p[u][q][j] = P[(w * W + q) * pk + j * pn];
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t w = w0 + int64_t(u) * G;
      if (w < words) {
#pragma unroll
        for (int q = 0; q < W; ++q)
#pragma unroll
          for (int j = 0; j < NB; ++j)
            if (j < n) {
#pragma unroll
              for (int r = 0; r < R; ++r)
                acc[r][j] += x[u][r][q] * p[u][q][j];
            }
      }
    }
  }
  if (W > 1 && g == 0 && blockIdx.y == gridDim.y - 1) // the elements behind the last whole word
    for (int64_t k = allWords * W; k < K; ++k)
#pragma unroll
      for (int j = 0; j < NB; ++j)
        if (j < n) {
          const T v = P[k * pk + j * pn];
#pragma unroll
          for (int r = 0; r < R; ++r)
            acc[r][j] += row[r][k] * v;
        }
  const int inWave = G < 64 ? G : 64;
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      T v = acc[r][j];
      for (int step = inWave >> 1; step > 0; step >>= 1)
        v += __shfl_xor(v, step, 64);
      acc[r][j] = v;
    }
  if (wholeBlock) { // (the same for every lane of the launch)
    if (lane == 0)
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          cross[wave][r * NB + j] = acc[r][j];
    __syncthreads();
    if (threadIdx.x == 0)
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[r][j] = ((cross[0][r * NB + j] + cross[1][r * NB + j]) + cross[2][r * NB + j]) +
                      cross[3][r * NB + j];
  }
  if (g == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < NB; ++j)
        if (r0 + r < rows && j < n && part) {
          part[(int64_t(blockIdx.y) * rows + r0 + r) * n + j] = acc[r][j];
        } else if (r0 + r < rows && j < n) {
          T *dst = O + (r0 + r) * orow + j * ocol;
          T v = alpha * acc[r][j];
          if (beta != T(0))
            v += beta * *dst;
          *dst = v;
        }
  }
}

// The value that lane `from` (the same for the whole wave) holds in v.
__device__ __forceinline__ float fromLane(float v, int from) {
  return __builtin_bit_cast(float,
                            __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), from));
}
__device__ __forceinline__ double fromLane(double v, int from) {
  const uint64_t bits = __builtin_bit_cast(uint64_t, v);
  const uint32_t lo = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(bits)), from));
  const uint32_t hi = uint32_t(__builtin_amdgcn_readlane(int(uint32_t(bits >> 32)), from));
  return __builtin_bit_cast(double, (uint64_t(hi) << 32) | lo);
}

// O(i, c) = alpha * sum_k P(i, k) S(k, c) + beta * O(i, c) for a thin P
// (m <= MB rows, any strides) and a long S with unit stride along c (rows
// `ld` apart): a lane owns W adjacent columns, each of the four waves of a
// block takes every fourth k of the block's slice of K (eight loads of S in
// flight a lane) and the four add up through LDS in wave order.  P(i, k) is
// the same for the whole wave: the lanes fetch those of 64 steps at a time,
// one each, and hand them round.  With one slice (part == nullptr) the block stores to O;
// with more, slice z stores its m x cPitch partial sums at part + z m cPitch
// and gemm_thin_fold adds the slices in index order.
template <typename T, int MB, int W>
__global__ __launch_bounds__(256) void
gemm_thin_cols(const T *__restrict__ S, int64_t ld, int64_t C, int64_t K, int64_t sliceK,
               const T *__restrict__ P, int64_t pm, int64_t pk, int m, T *__restrict__ O,
               int64_t oi, int64_t oc, T alpha, T beta, T *__restrict__ part,
               int64_t cPitch) {
  constexpr int U = 8, STRIP = 64 * W;
  __shared__ T sums[4][MB][STRIP];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t strip0 = int64_t(blockIdx.x) * STRIP;
  const int64_t c0 = strip0 + lane * W;
  const bool live = c0 < C; // (W > 1: C is a multiple of W)
  const int64_t sliceBegin = int64_t(blockIdx.y) * sliceK;
  const int64_t sliceEnd = sliceBegin + sliceK < K ? sliceBegin + sliceK : K;
  // this wave's rows of S: every fourth of the slice (the four waves of a
  // block read four adjacent rows at a time)
  const int64_t kBegin = sliceBegin + wave;
  const int64_t steps = kBegin < sliceEnd ? (sliceEnd - kBegin + 3) / 4 : 0;
  T acc[MB][W];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int q = 0; q < W; ++q)
      acc[i][q] = T(0);
  const T *col = S + (live ? c0 : 0);
  for (int64_t t64 = 0; t64 < steps; t64 += 64) {
    T mine[MB]; // P(i, k) of step t64 + lane
#pragma unroll
    for (int i = 0; i < MB; ++i)
      mine[i] = i < m && t64 + lane < steps ? P[i * pm + (kBegin + 4 * (t64 + lane)) * pk]
                                            : T(0);
    const int count = steps - t64 < 64 ? int(steps - t64) : 64;
    for (int t0 = 0; t0 < count; t0 += U) {
      T s[U][W];
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (t0 + u < count)
          ThinWord<T, W>::load(col + (kBegin + 4 * (t64 + t0 + u)) * ld, s[u]);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (t0 + u < count) {
#pragma unroll
          for (int i = 0; i < MB; ++i)
            if (i < m) {
              const T v = fromLane(mine[i], t0 + u);
#pragma unroll
              for (int q = 0; q < W; ++q)
                acc[i][q] += v * s[u][q];
            }
        }
    }
  }
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int q = 0; q < W; ++q)
      sums[wave][i][lane * W + q] = acc[i][q];
  __syncthreads();
  for (int e = threadIdx.x; e < m * STRIP; e += 256) {
    const int i = e / STRIP, cc = e % STRIP;
    const int64_t c = strip0 + cc;
    if (c >= C)
      continue;
    const T sum = ((sums[0][i][cc] + sums[1][i][cc]) + sums[2][i][cc]) + sums[3][i][cc];
    if (part) {
      part[(int64_t(blockIdx.y) * m + i) * cPitch + c] = sum;
    } else {
      T *dst = O + i * oi + c * oc;
      T v = alpha * sum;
      if (beta != T(0))
        v += beta * *dst;
      *dst = v;
    }
  }
}

// A small product of long operands (m, n <= 8: the Gram matrix of a few
// columns, a few columns against a right-hand side): block z takes a slice of
// K, a lane every 256th k of it -- the m values of X and the n of Y at that k,
// any strides, two k in flight -- and keeps all m n sums; they meet through
// lane exchanges and LDS, in a fixed order, and go to part + z m n for
// gemm_thin_fold.  ROWS: the m values of X at a k and the n of Y are adjacent
// and aligned (m == MB, n == NB, rows of the transposed tall operands): read
// as words (8 x 1048576 x 8 float32 73 -> 48 us).
template <typename T, int MB, int NB, bool ROWS>
__global__ __launch_bounds__(256) void
gemm_inner(const T *__restrict__ X, int64_t xm, int64_t xk, const T *__restrict__ Y,
           int64_t yk, int64_t yn, int m, int n, int64_t K, int64_t kSlice,
           T *__restrict__ part) {
  constexpr int U = 2;
  __shared__ T cross[4][MB * NB];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t kBegin = int64_t(blockIdx.x) * kSlice;
  const int64_t kEnd = kBegin + kSlice < K ? kBegin + kSlice : K;
  T acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
      acc[i][j] = T(0);
  for (int64_t k0 = kBegin + threadIdx.x; k0 < kEnd; k0 += 256 * U) {
    T x[U][MB], y[U][NB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t k = k0 + 256 * u;
      if (k < kEnd && ROWS) {
        typedef T XRow __attribute__((ext_vector_type(MB), aligned(MB * sizeof(T) < 16 ? MB * sizeof(T) : 16)));
        typedef T YRow __attribute__((ext_vector_type(NB), aligned(NB * sizeof(T) < 16 ? NB * sizeof(T) : 16)));
        const XRow xv = __builtin_nontemporal_load(reinterpret_cast<const XRow *>(X + k * xk));
        const YRow yv = __builtin_nontemporal_load(reinterpret_cast<const YRow *>(Y + k * yk));
#pragma unroll
        for (int i = 0; i < MB; ++i)
          x[u][i] = xv[i];
#pragma unroll
        for (int j = 0; j < NB; ++j)
          y[u][j] = yv[j];
      } else if (k < kEnd) {
#pragma unroll
        for (int i = 0; i < MB; ++i)
          x[u][i] = i < m ? __builtin_nontemporal_load(X + i * xm + k * xk) : T(0);
#pragma unroll
        for (int j = 0; j < NB; ++j)
          y[u][j] = j < n ? __builtin_nontemporal_load(Y + k * yk + j * yn) : T(0);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (k0 + 256 * u < kEnd) {
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
          for (int j = 0; j < NB; ++j)
            acc[i][j] += x[u][i] * y[u][j];
      }
  }
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      T v = acc[i][j];
#pragma unroll
      for (int step = 32; step > 0; step >>= 1)
        v += __shfl_xor(v, step, 64);
      if (lane == 0)
        cross[wave][i * NB + j] = v;
    }
  __syncthreads();
  if (int(threadIdx.x) < m * n) {
    const int i = threadIdx.x / n, j = threadIdx.x % n, at = i * NB + j;
    part[(int64_t(blockIdx.x) * m + i) * n + j] =
        ((cross[0][at] + cross[1][at]) + cross[2][at]) + cross[3][at];
  }
}

// O(i, c) = alpha * (part[0](i, c) + part[1](i, c) + ...) + beta * O(i, c),
// the slices m cPitch elements apart: a block takes 16 adjacent elements of a
// row; 16 lanes an element each add up every 16th slice (eight loads in
// flight), then one adds the 16 sums in lane order -- a fixed order, so the
// result does not depend on which block finished first, and thousands of
// slices of a small result are not one lane's chain of loads.
template <typename T>
__global__ __launch_bounds__(256) void
gemm_thin_fold(const T *__restrict__ part, int slices, int m, int64_t C, int64_t cPitch,
               T *__restrict__ O, int64_t oi, int64_t oc, T alpha, T beta) {
  __shared__ T sums[16][17];
  const int el = threadIdx.x & 15, zl = threadIdx.x >> 4;
  const int64_t c = int64_t(blockIdx.x) * 16 + el;
  const int i = blockIdx.y;
  T sum = T(0);
  if (c < C) {
    const T *src = part + int64_t(i) * cPitch + c;
    const int64_t stride = int64_t(m) * cPitch;
    for (int z = zl; z < slices; z += 16 * 8) {
      T v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        v[u] = z + 16 * u < slices ? src[(z + 16 * u) * stride] : T(0);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        sum += v[u];
    }
  }
  sums[zl][el] = sum;
  __syncthreads();
  if (zl != 0 || c >= C)
    return;
  sum = sums[0][el];
#pragma unroll
  for (int z = 1; z < 16; ++z)
    sum += sums[z][el];
  T *dst = O + i * oi + c * oc;
  T v = alpha * sum;
  if (beta != T(0))
    v += beta * *dst;
  *dst = v;
}

// ---------------------------------------------------------------------------
// A copy of an operand that the tile kernels can read in 128-bit words: the
// R rows of C elements at src (row stride ld, unit stride along a row) go to
// rows of Cp = C rounded up to whole words, dense, 16-byte aligned, the tail
// of every row filled with zeros, followed by rows of zeros up to Rp rows.
// For operands whose rows do not begin or end on a word (an odd extent or
// leading dimension, a view that starts inside a word), and to pad operands
// to whole tiles.  One thread per destination word.
template <typename T>
__global__ __launch_bounds__(256) void
gemm_pack_rows(const T *__restrict__ src, int64_t ld, int64_t R, int64_t C,
               T *__restrict__ dst, int64_t Cp, int64_t Rp) {
  typedef typename Mfma<T>::Vec Vec;
  constexpr int VEC = Mfma<T>::VEC;
  const int64_t wordsPerRow = Cp / VEC;
  const int64_t word = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (word >= Rp * wordsPerRow)
    return;
  int64_t r, c;
  splitWord(word, wordsPerRow, r, c);
  c *= VEC;
  const T *row = src + r * ld;
  Vec v;
#pragma unroll
  for (int q = 0; q < VEC; ++q)
    v[q] = (r < R && c + q < C) ? row[c + q] : T(0);
  *reinterpret_cast<Vec *>(dst + r * Cp + c) = v;
}

// ---------------------------------------------------------------------------
// Workspace of the split-K path, per device.
//
// mkl_gemm_<dtype>_device keeps one hipMalloc'ed block per device, grown on
// demand and released by nmrtMathRuntimeFinalize.  The *_noalloc entry point
// may not allocate: it uses `scratch`, a fixed array in the code object's own
// device memory (every GPU the library runs on holds a copy until the process
// ends).  In host code the array's name is only a handle; its device address
// is looked up once per device with hipGetSymbolAddress and kept.
// 16 MiB: planSplit never asks for more in float32 (slices x tiles <= 256
// resident blocks, 64 KiB of partial product per 128 x 128 tile).
constexpr size_t kScratchBytes = size_t(16) << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
struct DeviceWorkspace {
  void *fixed = nullptr; // device address of `scratch` on this device
  void *heap = nullptr;
  size_t heapBytes = 0;
  int computeUnits = 0; // of the device (or of its partition), asked once
};
DeviceWorkspace workspaces[kMaxDevices];
std::mutex workspaceMutex;
// Held by a call from the moment it asks for a device's workspace (heap or
// fixed) until its kernels have finished: calls from several host threads,
// on whatever queues, take turns on the one workspace of a device.
std::mutex workspaceInUse[kMaxDevices];

DeviceWorkspace &workspaceOf(int device) {
  if (device < 0 || device >= kMaxDevices)
    fatal("mkl_gemm_device: device ordinal %d out of range\n", device);
  return workspaces[device];
}

// Compute units of the current device: 256 on a whole MI355X, fewer on a
// partition of one.  The launch plans below count resident blocks in them.
int computeUnitsOf(int device) {
  std::lock_guard<std::mutex> lock(workspaceMutex);
  DeviceWorkspace &w = workspaceOf(device);
  if (w.computeUnits <= 0) {
    int n = 0;
    checkHip(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device),
             "hipDeviceGetAttribute(multiprocessor count)");
    w.computeUnits = n > 0 ? n : 1;
  }
  return w.computeUnits;
}

// Grown on demand; nullptr when the device has no room for the larger block
// (the block it has stays as it is: the caller then runs without what it
// asked for).  The device must be current, and the caller holds the
// device's turn, so no kernel of another call reads the block that is freed.
void *heapWorkspace(int device, size_t bytes) {
  std::lock_guard<std::mutex> lock(workspaceMutex);
  DeviceWorkspace &w = workspaceOf(device);
  if (bytes <= w.heapBytes)
    return w.heap;
  const size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes;
  void *p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (w.heap) {
    checkHip(hipDeviceSynchronize(), "hipDeviceSynchronize");
    checkHip(hipFree(w.heap), "hipFree");
  }
  w.heap = p;
  w.heapBytes = want;
  return p;
}

// A call whose repacked operands made the block larger than this gives it
// back when it returns (its stream is idle by then): a device keeps at most
// 1 GiB between calls.
constexpr size_t kHeapKeptBytes = size_t(1) << 30;
void trimHeapWorkspace(int device) {
  std::lock_guard<std::mutex> lock(workspaceMutex);
  DeviceWorkspace &w = workspaceOf(device);
  if (w.heapBytes <= kHeapKeptBytes)
    return;
  checkHip(hipFree(w.heap), "hipFree");
  w.heap = nullptr;
  w.heapBytes = 0;
}

// Device address of the fixed array on the current device (set up on the
// first call per device; allocates nothing).
void *fixedWorkspace(int device) {
  std::lock_guard<std::mutex> lock(workspaceMutex);
  DeviceWorkspace &w = workspaceOf(device);
  if (!w.fixed) {
    void *p = nullptr;
    checkHip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)),
             "hipGetSymbolAddress(scratch)");
    w.fixed = p;
  }
  return w.fixed;
}

void releaseHeapWorkspaces() {
  std::lock_guard<std::mutex> lock(workspaceMutex);
  for (int d = 0; d < kMaxDevices; ++d) {
    DeviceWorkspace &w = workspaces[d];
    if (!w.heap)
      continue;
    if (hipSetDevice(d) == hipSuccess)
      (void)hipFree(w.heap);
    w.heap = nullptr;
    w.heapBytes = 0;
  }
}

// How K is cut for a launch of `tiles` block tiles: 1 slice when the tiles
// fill the GPU by themselves or K is short.
struct SplitPlan {
  int slices = 1;
  int sliceK = 0;
};
SplitPlan planSplit(int64_t tiles, int64_t K, int BK, int64_t slots /* resident blocks */) {
  SplitPlan plan;
  if (tiles <= 0 || tiles * 2 > slots)
    return plan;
  // (at most 16 slices, or more of 512 elements each where K is that long:
  // 128 x 262144 x 128 float32 1122 us in 16 slices)
  int64_t slices = slots / tiles;
  const int64_t most = K / 512 > 16 ? K / 512 : 16;
  if (slices > most)
    slices = most;
  const int64_t minSlice = int64_t(8) * BK; // at least eight slabs a slice
  if (slices > K / minSlice)
    slices = K / minSlice;
  if (slices < 2)
    return plan;
  int64_t sliceK = (K + slices - 1) / slices;
  sliceK = (sliceK + BK - 1) / BK * BK;
  plan.sliceK = int(sliceK);
  plan.slices = int((K + sliceK - 1) / sliceK);
  if (plan.slices < 2) {
    plan.slices = 1;
    plan.sliceK = 0;
  }
  return plan;
}

// Blocks of an even-shares launch over `tiles` block tiles of `slabs` K slabs
// each on `slots` resident blocks, or 0 when whole tiles do as well: they
// fill their rounds to nine tenths or more, or a block's share would be under
// eight slabs (the pieces' trip through the workspace would cost more than
// the idle CUs).
int planEvenShares(int64_t tiles, int64_t slabs, int64_t slots) {
  if (tiles <= 0 || slabs <= 0)
    return 0;
  const int64_t rounds = (tiles + slots - 1) / slots;
  if (tiles * 10 >= rounds * slots * 9)
    return 0;
  if (tiles * slabs < 8 * slots)
    return 0;
  return int(slots);
}

// Whether cutting K into plan.slices equal slices goes ahead of even shares:
// when the slices fill the resident blocks to 0.86 (measured: from 0.875 up
// the slices are 4-17 % faster than even shares of the same tiles -- their
// partial products are whole tiles that one streaming pass adds up -- at 0.84
// and below the shares win), or when there are so few tiles that shares
// would cut each into more than 16 pieces.
bool splitFills(const SplitPlan &plan, int64_t tiles, int64_t slots) {
  if (plan.slices < 2)
    return false;
  // (two or three slices leave shares few pieces to add up, so the slices
  // must fill more: 225 tiles x 2 fill 0.88 and lose to shares, 149 against
  // 141 us for 1920^3 float32)
  const int64_t pct = plan.slices >= 4 ? 86 : 93;
  return tiles * plan.slices * 100 >= slots * pct || plan.slices >= 16;
}

enum WorkspaceKind { WORKSPACE_HEAP, WORKSPACE_FIXED };

template <typename T> struct MemrefOf;
template <> struct MemrefOf<float> {
  typedef NmhipMemref2F32 type;
};
template <> struct MemrefOf<double> {
  typedef NmhipMemref2F64 type;
};

template <typename T>
void requireUnitStride(const typename MemrefOf<T>::type *arr, char name) {
  if (arr->strides[0] != 1 && arr->strides[1] != 1)
    fatal("mkl gemm suports only arrays contiguous on inner dimension.\n"
          "stride for at least one dimension should be equal to 1.\n"
          "'%c' parameter is not contiguous. '%c' strides are %d and %d.\n",
          name, name, int(arr->strides[0]), int(arr->strides[1]));
}

bool aligned16(const void *p) {
  return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// Grid of gemm_generic for an m x n result: its 32 x 32 tiles along x, then y
// (a dimension of a launch holds 2^32 - 1 work-items, 2^24 - 1 blocks of 256).
dim3 genericGrid(int64_t m, int64_t n) {
  const int64_t tiles = ((m + 31) / 32) * ((n + 31) / 32);
  const int64_t most = int64_t(1) << 23;
  const int64_t gx = tiles < most ? tiles : most;
  const int64_t gy = (tiles + gx - 1) / gx;
  if (gy > 65535)
    fatal("mkl_gemm_device: a %lld x %lld result is more than one launch of the "
          "strided kernel holds\n",
          (long long)m, (long long)n);
  return dim3(unsigned(gx), unsigned(gy), 1);
}

// Returns 0, or (WORKSPACE_FIXED only) 1 when the product would need more
// workspace than the fixed array holds; nothing has been launched then.
template <typename T>
int deviceGemm(void *queueObj, const typename MemrefOf<T>::type *a,
               const typename MemrefOf<T>::type *b,
               typename MemrefOf<T>::type *c, T alpha, T beta,
               WorkspaceKind workspaceKind) {
  if (!queueObj || !a || !b || !c)
    fatal("mkl_gemm_device: null argument\n");
  auto *base = static_cast<numba::GPUQueueInterface *>(queueObj);
  auto *queue = static_cast<numba::HipQueueInterface *>(base);
  if (queue->hipMagic() != numba::HipQueueInterface::kMagic)
    fatal("mkl_gemm_device: queue '%.*s' was not created by the HIP GPU "
          "runtime\n",
          int(base->getDeviceName().size()), base->getDeviceName().data());

  requireUnitStride<T>(a, 'a');
  requireUnitStride<T>(b, 'b');
  requireUnitStride<T>(c, 'c');

  const int64_t M = int64_t(a->dims[0]);
  const int64_t N = int64_t(b->dims[1]);
  const int64_t K = int64_t(a->dims[1]);
  if (int64_t(b->dims[0]) != K || int64_t(c->dims[0]) != M ||
      int64_t(c->dims[1]) != N)
    fatal("mkl_gemm_device: shape mismatch: a [%lld,%lld] b [%lld,%lld] c "
          "[%lld,%lld]\n",
          (long long)a->dims[0], (long long)a->dims[1], (long long)b->dims[0],
          (long long)b->dims[1], (long long)c->dims[0], (long long)c->dims[1]);

  const T *aData = a->data + a->offset;
  const T *bData = b->data + b->offset;
  T *cData = c->data + c->offset;

  const int device = queue->hipDevice();
  checkHip(hipSetDevice(device), "hipSetDevice");
  auto stream = static_cast<hipStream_t>(queue->hipStream());

  // Split-K workspace for `plan` over an [m, ldw] partial product per slice;
  // leaves plan unsplit when the heap has no room, reports the fixed array
  // as too small through tooLarge.
  bool tooLarge = false;
  // Bytes at the start of the heap workspace that hold repacked operands
  // (gemm_pack_rows); the partial products come behind them.
  size_t packBytes = 0;
  std::unique_lock<std::mutex> workspaceTurn; // (released when the call returns)
  auto takeTurn = [&]() {
    (void)workspaceOf(device); // (checks the ordinal)
    if (!workspaceTurn.owns_lock())
      workspaceTurn = std::unique_lock<std::mutex>(workspaceInUse[device]);
  };
  // `required`: the caller cannot run unsplit (the tile kernels' plans count
  // on their slices): the call then returns 1 before anything is launched.
  // The other callers run unsplit on nullptr, whichever workspace was short.
  auto workspaceFor = [&](SplitPlan &plan, int64_t m, int64_t ldw,
                          bool required = false) -> T * {
    if (plan.slices < 2)
      return nullptr;
    takeTurn();
    const size_t bytes = size_t(plan.slices) * size_t(m) * size_t(ldw) * sizeof(T);
    void *p = nullptr;
    if (workspaceKind == WORKSPACE_FIXED) {
      if (bytes > kScratchBytes && !required) {
        plan = SplitPlan();
        return nullptr;
      }
      if (bytes > kScratchBytes) {
        std::fprintf(stderr,
                     "mkl_gemm_device_noalloc: [%lld,%lld] x [%lld,%lld] needs "
                     "%zu bytes of split-K workspace, the fixed workspace "
                     "holds %zu\n",
                     (long long)a->dims[0], (long long)a->dims[1],
                     (long long)b->dims[0], (long long)b->dims[1], bytes,
                     kScratchBytes);
        tooLarge = true;
        return nullptr;
      }
      p = fixedWorkspace(device);
    } else {
      p = heapWorkspace(device, packBytes + bytes);
      if (!p)
        plan = SplitPlan();
      else
        p = static_cast<unsigned char *>(p) + packBytes;
    }
    return static_cast<T *>(p);
  };
  // Workspace of an even-shares launch: two BM x BN slots a block; the
  // shares are given up (0 blocks) when there is no room.
  auto evenWorkspace = [&](int &blocks, int bm, int bn) -> T * {
    if (blocks <= 0)
      return nullptr;
    takeTurn();
    void *p = heapWorkspace(
        device, packBytes + size_t(blocks) * 2 * size_t(bm) * size_t(bn) * sizeof(T));
    if (!p)
      blocks = 0;
    else
      p = static_cast<unsigned char *>(p) + packBytes;
    return static_cast<T *>(p);
  };
  const int64_t cus = computeUnitsOf(device);
  const int64_t slots = 2 * cus; // resident blocks of the 128 x 128 tiles: two a CU
  // Equal slices of K for `tiles` 128 x 128 tiles, and whether they go ahead
  // of even shares.  float64 blocks share a CU in pairs; float32 ones may
  // (186 registers a lane), which pays where one block a CU would not fill
  // the GPU but two do (72 tiles: 3 slices fill 0.84 of 256 blocks, 7 fill
  // 0.98 of 512; 1000 x 1100 x 1200 58 -> 52 us, 1280^3 64 -> 59), and not
  // otherwise (1024^3: 4 slices on 256 blocks 40 us, 8 on 512 43).  The
  // entry point that may not allocate keeps to 256 blocks: the fixed
  // workspace is sized for those.
  auto planSlices = [&](int64_t tiles, int64_t k, bool &fills) {
    if (sizeof(T) == 8) {
      const SplitPlan two = planSplit(tiles, k, Mfma<T>::BK, 2 * cus);
      fills = splitFills(two, tiles, 2 * cus);
      return two;
    }
    const SplitPlan one = planSplit(tiles, k, Mfma<T>::BK, cus);
    fills = splitFills(one, tiles, cus);
    if (fills || workspaceKind != WORKSPACE_HEAP)
      return one;
    const SplitPlan two = planSplit(tiles, k, Mfma<T>::BK, 2 * cus);
    if (splitFills(two, tiles, 2 * cus)) {
      fills = true;
      return two;
    }
    return one;
  };
  auto fold = [&](const SplitPlan &plan, const T *W, int64_t m, int64_t n,
                  int64_t ldw, int64_t ldz, T *Z) {
    const int64_t words = m * ((n + Mfma<T>::VEC - 1) / Mfma<T>::VEC);
    hipLaunchKernelGGL(gemm_splitk_fold<T>, dim3(unsigned((words + 255) / 256)),
                       dim3(256), 0, stream, W, plan.slices, m * ldw, ldw, Z,
                       int(m), int(n), ldz, alpha, beta);
  };

  auto evenFold = [&](const T *W, int blocks, int slabs, int64_t tilesM, int64_t tilesN,
                      int tile, int64_t m, int64_t n, int64_t ldz, T *Z) {
    const int64_t units = tilesM * tilesN * slabs;
    dim3 grid(unsigned(tilesM * tilesN), unsigned(tile * tile / Mfma<T>::VEC / 256));
    if (tile == 256)
      hipLaunchKernelGGL((gemm_even_fold<T, 256, 256>), grid, dim3(256), 0, stream, W,
                         int64_t(blocks), slabs, int(tilesN), units, Z, int(m), int(n),
                         ldz, alpha, beta);
    else
      hipLaunchKernelGGL((gemm_even_fold<T, 128, 128>), grid, dim3(256), 0, stream, W,
                         int64_t(blocks), slabs, int(tilesN), units, Z, int(m), int(n),
                         ldz, alpha, beta);
  };

  lastPacked = false;
  if (M > 0 && N > 0) {
    bool launched = false;
    {
      // Operands as the kernel sees them: X(m,k), Y(k,n), Z row-major.  A
      // column-major C is computed as C^T = B^T A^T (swap and transpose the
      // inputs); which dimension of each input is contiguous follows from
      // its unit stride (NumpyLinalg.cpp:87-102).
      const bool cRow = c->strides[1] == 1;
      const T *X = cRow ? aData : bData;
      const T *Y = cRow ? bData : aData;
      // strides of X over (m, k) and Y over (k, n)
      const int64_t xm = cRow ? a->strides[0] : b->strides[1];
      const int64_t xk = cRow ? a->strides[1] : b->strides[0];
      const int64_t yk = cRow ? b->strides[0] : a->strides[1];
      const int64_t yn = cRow ? b->strides[1] : a->strides[0];
      const int64_t Mz = cRow ? M : N, Nz = cRow ? N : M;
      const int64_t ldz = cRow ? c->strides[0] : c->strides[1];
      const bool xKc = xk == 1, yNc = yn == 1;
      const int64_t ldx = xKc ? xm : xk, ldy = yNc ? yk : yn;
      constexpr int VEC = Mfma<T>::VEC, BK = Mfma<T>::BK;
      // Tall times small: gemm_skinny.
      if (xKc && K >= 1 && K <= 32 && Nz <= 32 && Mz >= 4096 && ldx > 0) {
        const int64_t rows = 128 * 33 / (K + 1); // of a tile (gemm_skinny)
        const int64_t tiles = (Mz + rows - 1) / rows;
        const unsigned blocks = unsigned(tiles < 2048 ? tiles : 2048);
        // (whole rows of four-element words: one store a lane)
        const int wordStores =
            Nz % 4 == 0 && ldz % 4 == 0 &&
            reinterpret_cast<uintptr_t>(cData) % (4 * sizeof(T)) == 0;
        hipLaunchKernelGGL(gemm_skinny<T>, dim3(blocks), dim3(256), 0, stream, X, ldx, Y, yk,
                           yn, cData, ldz, Mz, int(Nz), int(K), alpha, beta, wordStores);
        lastKernel = sizeof(T) == 4 ? "sgemm_skinny" : "dgemm_skinny";
        launched = true;
      }
      // Small times long: gemm_wide.
      if (!launched && yNc && K >= 1 && K <= 32 && Mz <= 32 && Nz >= 4096 && ldy > 0) {
        const dim3 grid(unsigned((Nz + 255) / 256));
#define NMHIP_GEMM_WIDE(MB)                                                    \
  hipLaunchKernelGGL((gemm_wide<T, MB>), grid, dim3(256), 0, stream, X, xm, xk, \
                     Y, ldy, cData, ldz, int(Mz), Nz, int(K), alpha, beta)
        if (Mz <= 4)
          NMHIP_GEMM_WIDE(4);
        else if (Mz <= 8)
          NMHIP_GEMM_WIDE(8);
        else if (Mz <= 16)
          NMHIP_GEMM_WIDE(16);
        else
          NMHIP_GEMM_WIDE(32);
#undef NMHIP_GEMM_WIDE
        lastKernel = sizeof(T) == 4 ? "sgemm_wide" : "dgemm_wide";
        launched = true;
      }
      // A small product of long operands: gemm_inner, K in slices of 2048
      // or more over at most 1024 blocks.
      if (!launched && Mz <= 8 && Nz <= 8 && K >= 4096) {
        SplitPlan plan;
        plan.slices = int(K / 2048 < 1024 ? K / 2048 : 1024);
        const int64_t kSlice = (K + plan.slices - 1) / plan.slices;
        plan.slices = int((K + kSlice - 1) / kSlice);
        if (T *part = workspaceFor(plan, Mz, Nz)) {
          const dim3 grid{unsigned(plan.slices)};
          auto rowsOf = [](const T *base, int64_t unit, int64_t step, int64_t extent) {
            const size_t bytes = size_t(extent) * sizeof(T) < 16 ? size_t(extent) * sizeof(T) : 16;
            return unit == 1 && (extent == 4 || extent == 8) &&
                   reinterpret_cast<uintptr_t>(base) % bytes == 0 &&
                   size_t(step) * sizeof(T) % bytes == 0;
          };
          const bool rowsXY = rowsOf(X, xm, xk, Mz) && rowsOf(Y, yn, yk, Nz);
#define NMHIP_GEMM_INNER(MB, NB)                                               \
  do {                                                                         \
    if (rowsXY)                                                                \
      hipLaunchKernelGGL((gemm_inner<T, MB, NB, true>), grid, dim3(256), 0,    \
                         stream, X, xm, xk, Y, yk, yn, int(Mz), int(Nz), K,    \
                         kSlice, part);                                        \
    else                                                                       \
      hipLaunchKernelGGL((gemm_inner<T, MB, NB, false>), grid, dim3(256), 0,   \
                         stream, X, xm, xk, Y, yk, yn, int(Mz), int(Nz), K,    \
                         kSlice, part);                                        \
  } while (0)
          if (Mz <= 4 && Nz <= 4)
            NMHIP_GEMM_INNER(4, 4);
          else if (Mz <= 4)
            NMHIP_GEMM_INNER(4, 8);
          else if (Nz <= 4)
            NMHIP_GEMM_INNER(8, 4);
          else
            NMHIP_GEMM_INNER(8, 8);
#undef NMHIP_GEMM_INNER
          hipLaunchKernelGGL(gemm_thin_fold<T>, dim3(unsigned((Nz + 15) / 16), unsigned(Mz)),
                             dim3(256), 0, stream, part, plan.slices, int(Mz), Nz, Nz, cData,
                             ldz, int64_t(1), alpha, beta);
          lastKernel = sizeof(T) == 4 ? "sgemm_inner" : "dgemm_inner";
          launched = true;
        }
      }
      // A long matrix times a thin one (a few columns, or rows):
      // gemm_thin_rows when the long one has unit stride along k,
      // gemm_thin_cols when along its other dimension.
      if (!launched && K > 32) {
        // (by columns up to 16 of them: 16 x 16384 x 16384 float32 701 us on the
        // tiles, 372 here; by rows the thin operand's reads cost more than
        // the tiles' idle rows beyond 8)
        constexpr int64_t kLong = 1024, kThinRows = 8, kThinCols = 16;
        auto wordsOk = [&](const T *S, int64_t ld) { return aligned16(S) && ld % VEC == 0; };
        auto thinRows = [&](const T *S, int64_t ld, int64_t rows, const T *P, int64_t pk,
                            int64_t pn, int n, int64_t orow, int64_t ocol) {
          const bool vec = wordsOk(S, ld);
          const int64_t words = vec ? K / VEC : K;
          int G = 64, gShift = 6;
          while (G > 1 && 2 * G > words)
            G >>= 1, --gShift;
          const int NB = n <= 1 ? 1 : n <= 2 ? 2 : n <= 4 ? 4 : 8;
          auto wavesWith = [&](int R) { return ((rows + R - 1) / R * G + 63) / 64; };
          // Four rows a group where that leaves 2048 waves or more, and for
          // more than one column of P always (fewer reads of P: as many
          // elements of P as of S at most); the four
          // waves of a block on one set of rows where there are few rows.
          const int R = NB == 8 ? 8 : NB > 1 || wavesWith(4) >= 2048 ? 4 : 1;
          if (wavesWith(R) < 2048 && words >= 512)
            G = 256, gShift = 8;
          const int64_t sets = (rows + R - 1) / R;
          const int64_t perBlock = G == 256 ? 1 : 4 * (64 / G);
          const int64_t blocks = (sets + perBlock - 1) / perBlock;
          if (blocks >= (int64_t(1) << 24))
            return false;
          // Few rows of a long K: slices of K (four trips of a block or more
          // each) bring the launch to some 2048 blocks; their sums are
          // added in index order by gemm_thin_fold.
          SplitPlan plan;
          int64_t sliceWords = words > 0 ? words : 1;
          if (G == 256 && blocks < 1024) {
            const int64_t trip = int64_t(256) * (R < 8 ? 8 / R : 1);
            int64_t slices = 2048 / blocks;
            if (slices > words / (4 * trip))
              slices = words / (4 * trip);
            if (slices > 1) {
              sliceWords = ((words + slices - 1) / slices + trip - 1) / trip * trip;
              plan.slices = int((words + sliceWords - 1) / sliceWords);
            }
          }
          T *part = workspaceFor(plan, rows, n);
          if (!part)
            plan.slices = 1, sliceWords = words > 0 ? words : 1;
          // How P is read (gemm_thin_rows).
          const size_t rowBytes = size_t(NB) * sizeof(T) < 16 ? size_t(NB) * sizeof(T) : 16;
          int PV = 0;
          if (NB > 1 && n == NB && pn == 1 &&
              reinterpret_cast<uintptr_t>(P) % rowBytes == 0 &&
              size_t(pk) * sizeof(T) % rowBytes == 0)
            PV = 1;
          else if (vec && pk == 1 && aligned16(P) && (n == 1 || pn % VEC == 0))
            PV = 2;
          const dim3 grid(unsigned(blocks), unsigned(plan.slices));
#define NMHIP_THIN_ROWS(NB_, R_, W_, PV_)                                      \
  hipLaunchKernelGGL((gemm_thin_rows<T, NB_, R_, W_, PV_>), grid, dim3(256), 0, \
                     stream, S, ld, rows, K, P, pk, pn, n, cData, orow, ocol,  \
                     alpha, beta, G, gShift, sliceWords, part)
#define NMHIP_THIN_ROWS_P(NB_, R_)                                             \
  do {                                                                         \
    if (vec && PV == 2)                                                        \
      NMHIP_THIN_ROWS(NB_, R_, VEC, 2);                                        \
    else if (vec && PV == 1)                                                   \
      NMHIP_THIN_ROWS(NB_, R_, VEC, (NB_ > 1 ? 1 : 0));                          \
    else if (vec)                                                              \
      NMHIP_THIN_ROWS(NB_, R_, VEC, 0);                                        \
    else if (PV == 1)                                                          \
      NMHIP_THIN_ROWS(NB_, R_, 1, (NB_ > 1 ? 1 : 0));                            \
    else                                                                       \
      NMHIP_THIN_ROWS(NB_, R_, 1, 0);                                          \
  } while (0)
          if (NB == 1) {
            if (R == 4)
              NMHIP_THIN_ROWS_P(1, 4);
            else
              NMHIP_THIN_ROWS_P(1, 1);
          } else if (NB == 2) {
            NMHIP_THIN_ROWS_P(2, 4);
          } else if (NB == 4) {
            NMHIP_THIN_ROWS_P(4, 4);
          } else {
            NMHIP_THIN_ROWS_P(8, 8);
          }
#undef NMHIP_THIN_ROWS_P
#undef NMHIP_THIN_ROWS
          if (part)
            hipLaunchKernelGGL(gemm_thin_fold<T>, dim3(unsigned((n + 15) / 16), unsigned(rows)),
                               dim3(256), 0, stream, part, plan.slices, int(rows), int64_t(n),
                               int64_t(n), cData, orow, ocol, alpha, beta);
          lastKernel = sizeof(T) == 4 ? "sgemm_thin_rows" : "dgemm_thin_rows";
          return true;
        };
        auto thinCols = [&](const T *S, int64_t ld, int64_t C, const T *P, int64_t pm,
                            int64_t pk, int m, int64_t oi, int64_t oc) {
          const bool vec = wordsOk(S, ld) && C % VEC == 0;
          const int64_t strip = vec ? 64 * VEC : 64;
          const int64_t strips = (C + strip - 1) / strip;
          if (strips >= (int64_t(1) << 24))
            return false;
          // Slices of K so that some 2048 blocks are at work, each wave with
          // sixteen rows of S or more; the partial sums within the fixed
          // workspace's size whichever workspace serves.
          const int64_t cPitch = strips * strip;
          int64_t slices = 2048 / strips;
          if (slices > K / 64)
            slices = K / 64;
          if (slices > 1024)
            slices = 1024;
          while (slices > 1 &&
                 size_t(slices) * size_t(m) * size_t(cPitch) * sizeof(T) > kScratchBytes)
            --slices;
          int64_t sliceK = K;
          if (slices > 1) {
            sliceK = ((K + slices - 1) / slices + 3) / 4 * 4;
            slices = (K + sliceK - 1) / sliceK;
          }
          SplitPlan plan;
          plan.slices = int(slices < 1 ? 1 : slices);
          T *part = workspaceFor(plan, m, cPitch);
          if (!part)
            plan.slices = 1, sliceK = K;
          const dim3 grid(unsigned(strips), unsigned(plan.slices));
#define NMHIP_THIN_COLS(MB, W)                                                 \
  hipLaunchKernelGGL((gemm_thin_cols<T, MB, W>), grid, dim3(256), 0, stream, S, \
                     ld, C, K, sliceK, P, pm, pk, m, cData, oi, oc, alpha,     \
                     beta, part, cPitch)
#define NMHIP_THIN_COLS_W(MB)                                                  \
  do {                                                                         \
    if (vec)                                                                   \
      NMHIP_THIN_COLS(MB, VEC);                                                \
    else                                                                       \
      NMHIP_THIN_COLS(MB, 1);                                                  \
  } while (0)
          if (m <= 1)
            NMHIP_THIN_COLS_W(1);
          else if (m <= 2)
            NMHIP_THIN_COLS_W(2);
          else if (m <= 4)
            NMHIP_THIN_COLS_W(4);
          else if (m <= 8)
            NMHIP_THIN_COLS_W(8);
          else
            NMHIP_THIN_COLS_W(16);
#undef NMHIP_THIN_COLS_W
#undef NMHIP_THIN_COLS
          if (part)
            hipLaunchKernelGGL(gemm_thin_fold<T>, dim3(unsigned((C + 15) / 16), unsigned(m)),
                               dim3(256), 0, stream, part, plan.slices, m, C, cPitch, cData,
                               oi, oc, alpha, beta);
          lastKernel = sizeof(T) == 4 ? "sgemm_thin_cols" : "dgemm_thin_cols";
          return true;
        };
        // (a long extent of 64 to 1023 too where K is long: slices of K fill the GPU)
        const int64_t longEnough = K >= 8192 ? 64 : kLong;
        if (Nz <= kThinCols && Mz >= longEnough)
          launched = xKc && Nz <= kThinRows ? thinRows(X, xm, Mz, Y, yk, yn, int(Nz), ldz, 1)
                     : !xKc && xm == 1      ? thinCols(X, xk, Mz, Y, yn, yk, int(Nz), 1, ldz)
                                            : false;
        else if (Mz <= kThinCols && Nz >= longEnough)
          launched = yNc                         ? thinCols(Y, yk, Nz, X, xm, xk, int(Mz), ldz, 1)
                     : yk == 1 && Mz <= kThinRows ? thinRows(Y, yn, Nz, X, xk, xm, int(Mz), 1, ldz)
                                                  : false;
      }
      // The matrix-core kernel takes the part of the problem that is whole
      // tiles, Z[0:Mt, 0:Nt] over k in [0, Kt); the strided kernel adds the
      // rest of K to that block and computes the rows and columns beyond it
      // (4000^3: 3968 x 3968 x 4000 on the matrix cores, 26 -> 65 TFLOP/s).
      // float32: 256 x 256 block tiles (one block per CU on a 4096^2
      // problem) when the shape allows and there are enough tiles to fill the
      // 256 CUs, 128 x 128 otherwise (measured within 3 % of each other; the
      // larger tile halves the operand traffic).  float64: 128 x 128.  The
      // large tile advances K in slabs of 2 BK where K allows (half the
      // barriers; 144 against 142 TFLOP/s on 4096^3).
      const int64_t Mt = Mz - Mz % 128, Nt = Nz - Nz % 128, Kt = K - K % BK;
      // Where whole tiles would leave CUs idle (too few of them, or a last
      // round that is mostly empty) and K is long enough, the blocks take
      // even shares of the K slabs of all tiles instead (planEvenShares).
      const bool bigFits = sizeof(T) == 4 && Mt % 256 == 0 && Nt % 256 == 0;
      const int64_t bigTiles = (Mt / 256) * (Nt / 256);
      const int bigSlab = Kt % (2 * BK) == 0 ? 2 * BK : BK;
      const int bigEven = bigFits && workspaceKind == WORKSPACE_HEAP
                              ? planEvenShares(bigTiles, Kt / bigSlab, cus)
                              : 0;
      // (from 64 large tiles on: below, the 128 x 128 tiles in slices or
      // shares are as fast or faster -- 1792^3 120 against 131 us, 1024 x
      // 1024 x 4096 92 against 99 -- and from 121 on the large tile wins,
      // 3072^3 456 against 474)
      // (the tile counts below are a quarter and three quarters of the CUs)
      bool big = bigFits && bigTiles * 4 >= cus && (bigEven > 0 || bigTiles * 4 >= 3 * cus);
      if (big && bigTiles * 4 < 3 * cus) {
        // (fewer large tiles than CUs only pay in even shares: without room
        // for those, the 128 x 128 tiles take the shape.  Slices of K on the
        // large tile were measured and gain nothing over its even shares:
        // 2048^3 160 against 158 us.)
        int blocks = bigEven;
        (void)evenWorkspace(blocks, 256, 256);
        big = blocks > 0;
      }
      const int BM = big ? 256 : 128, BN = BM;
      const bool unitOk = (xk == 1 || xm == 1) && (yk == 1 || yn == 1);
      // worth it when the tiled part is most of the work and fills at least
      // half the CUs (1000^3 is 49 tiles: the strided kernel alone, on 1024
      // blocks, takes half the time of tiles plus three edge launches)
      const bool whole = Mt == Mz && Nt == Nz && Kt == K;
      const bool mostly = whole ||
                          (double(Mt) * double(Nt) * double(Kt) >=
                               0.5 * double(Mz) * double(Nz) * double(K) &&
                           (Mt / 128) * (Nt / 128) >= 128);
      // Ragged shapes whose 128-bit words are whole (the extent along each
      // operand's contiguous dimension a multiple of the word): one launch
      // of 128 x 128 tiles that read zeros beyond the operands and store
      // only inside Z.
      const bool wordsWhole = (xKc ? K : Mz) % VEC == 0 && (yNc ? Nz : K) % VEC == 0;
      const int64_t tilesM = (Mz + 127) / 128, tilesN = (Nz + 127) / 128;
      // (only K ragged: the tiles as they are plus the rest of K on the
      // strided kernel is faster, 116 against 106 TFLOP/s on 4096 x 4096 x 4100)
      const bool onlyK = Mt == Mz && Nt == Nz && mostly;
      // An operand whose rows do not begin and end on 128-bit words (an odd
      // extent or leading dimension, a base inside a word) is copied once
      // into word-aligned rows padded with zeros (gemm_pack_rows) and the same
      // guarded tiles run on the copy: reading and writing each operand once
      // more is small beside the product (4094^3 float32: 27 -> 110 TFLOP/s).
      // Needs the heap workspace.
      const int64_t xC = xKc ? K : Mz, xR = xKc ? Mz : K; // X: contiguous extent, rows
      const int64_t yC = yNc ? Nz : K, yR = yNc ? K : Nz;
      auto offWords = [&](const T *base, int64_t ld, int64_t C) {
        return ld % VEC != 0 || !aligned16(base) || C % VEC != 0;
      };
      const bool canPack = workspaceKind == WORKSPACE_HEAP && unitOk && ldx > 0 && ldy > 0;
      const bool packX = canPack && offWords(X, ldx, xC);
      const bool packY = canPack && offWords(Y, ldy, yC);
      const bool wordsOk = (packX || !offWords(X, ldx, xC)) && (packY || !offWords(Y, ldy, yC));
      (void)wordsWhole;
      // Large shapes that are not whole tiles of whole words (256 x 256 for
      // float32, 128 x 128 for float64), where padding them to such tiles
      // costs under a tenth more arithmetic: both operands are copied into
      // zero-padded rows (whole tiles, whole K slabs) and the tiles run on the
      // copies with only their stores guarded.  float32 4000^3: 117 -> 126
      // TFLOP/s, 4094^3: 117 -> 131; float64 4000^3: 56 -> 62, 7000 x 7500 x
      // 8000: 61 -> 65.  From 192 padded tiles on in float32 (below that the
      // guarded 128 x 128 tiles in even shares are as fast or faster, 3000^3:
      // 107 against 104), from 256 in float64 (the same tile either way: the
      // copies have to be won back from the guards on the loads alone).
      bool paddedBig = false;
      {
        // float32: 256 x 256 tiles, K slabs of 32; float64: 128 x 128, slabs of 16
        constexpr int PT = sizeof(T) == 4 ? 256 : 128;
        constexpr int PSLAB = sizeof(T) == 4 ? 2 * BK : BK;
        const int64_t padSlots = sizeof(T) == 4 ? cus : slots;
        const int64_t minTiles = sizeof(T) == 4 ? 3 * cus / 4 : cus;
        auto roundUp = [](int64_t v, int64_t to) { return (v + to - 1) / to * to; };
        const int64_t Mp = roundUp(Mz, PT), Np = roundUp(Nz, PT), Kp = roundUp(K, PSLAB);
        const bool fitsAsIs = Mz == Mp && Nz == Np && K % BK == 0 && !offWords(X, ldx, xC) &&
                              !offWords(Y, ldy, yC);
        const int64_t padTiles = (Mp / PT) * (Np / PT);
        const int slabs = int(Kp / PSLAB);
        int evenBlocks = planEvenShares(padTiles, slabs, padSlots);
        if (!launched && canPack && !fitsAsIs && (!whole || packX || packY) && K >= 256 &&
            padTiles >= minTiles &&
            Mp / PT <= 65535 && Mz <= 0x7fffffff - 256 &&
            Nz <= 0x7fffffff - 256 && K <= 0x7fffffff - 64 &&
            double(Mp) * double(Np) * double(Kp) <= 1.10 * double(Mz) * double(Nz) * double(K)) {
          // X as [rows x contiguous extent], padded; the same for Y
          const int64_t xRp = xKc ? Mp : Kp, xCp = xKc ? Kp : Mp;
          const int64_t yRp = yNc ? Kp : Np, yCp = yNc ? Np : Kp;
          const size_t xBytes = size_t(roundUp(xRp * xCp * int64_t(sizeof(T)), 256));
          const size_t yBytes = size_t(roundUp(yRp * yCp * int64_t(sizeof(T)), 256));
          packBytes = xBytes + yBytes;
          T *W = evenWorkspace(evenBlocks, PT, PT);
          unsigned char *base = W ? reinterpret_cast<unsigned char *>(W) - packBytes : nullptr;
          if (!base) {
            evenBlocks = 0;
            takeTurn();
            base = static_cast<unsigned char *>(heapWorkspace(device, packBytes));
          }
          if (base) {
            auto pack = [&](const T *src, int64_t ld, int64_t R, int64_t C, int64_t Rp,
                            int64_t Cp, T *dst) {
              const int64_t words = Rp * (Cp / VEC);
              hipLaunchKernelGGL(gemm_pack_rows<T>, dim3(unsigned((words + 255) / 256)),
                                 dim3(256), 0, stream, src, ld, R, C, dst, Cp, Rp);
            };
            T *Xp = reinterpret_cast<T *>(base), *Yp = reinterpret_cast<T *>(base + xBytes);
            pack(X, ldx, xR, xC, xRp, xCp, Xp);
            pack(Y, ldy, yR, yC, yRp, yCp, Yp);
            const EvenShares even{evenBlocks ? slabs : 0, int(Np / PT)};
            dim3 grid(unsigned(Np / PT), unsigned(Mp / PT), 1);
            if (evenBlocks)
              grid = dim3(unsigned(evenBlocks), 1, 1);
#define NMHIP_GEMM_PADDED(XKC, YNC)                                            \
  hipLaunchKernelGGL((gemm_mfma<T, PSLAB, 4, 4, XKC, YNC, 2>), grid,          \
                     dim3(256), 0, stream, Xp, Yp, cData, int(Mz), int(Nz),    \
                     int(Kp), xCp, yCp, ldz, alpha, beta, 0, W, int64_t(0),    \
                     even)
            if (xKc && yNc)
              NMHIP_GEMM_PADDED(true, true);
            else if (xKc)
              NMHIP_GEMM_PADDED(true, false);
            else if (yNc)
              NMHIP_GEMM_PADDED(false, true);
            else
              NMHIP_GEMM_PADDED(false, false);
#undef NMHIP_GEMM_PADDED
            if (evenBlocks)
              evenFold(W, evenBlocks, slabs, Mp / PT, Np / PT, PT, Mz, Nz, ldz, cData);
            lastKernel = sizeof(T) == 4
                             ? (evenBlocks ? "sgemm_mfma_256x256_even" : "sgemm_mfma_256x256")
                             : (evenBlocks ? "dgemm_mfma_128x128_even" : "dgemm_mfma_128x128");
            lastPacked = true;
            launched = paddedBig = true;
          } else {
            packBytes = 0;
          }
        }
      }
      // (the guarded tiles below need every operand on the word grid: copies
      // of those that are not, or none of this when there is no room for them)
      size_t packXBytes = 0, packYBytes = 0;
      bool copiesFit = true;
      if (!launched && !paddedBig && (packX || packY)) {
        auto roundUp = [](int64_t v, int64_t to) { return (v + to - 1) / to * to; };
        packXBytes = packX ? size_t(roundUp(xR * roundUp(xC, VEC) * int64_t(sizeof(T)), 256)) : 0;
        packYBytes = packY ? size_t(roundUp(yR * roundUp(yC, VEC) * int64_t(sizeof(T)), 256)) : 0;
        takeTurn();
        copiesFit = heapWorkspace(device, packXBytes + packYBytes) != nullptr;
      }
      // (fewer than 16 tiles go to the strided kernel's 32 x 32 tiles, unless
      // K is long and the result a quarter of a tile or more: slices of K fill
      // the GPU then -- 300 x 65536 x 300 float32 15 -> 60 TFLOP/s)
      if (paddedBig || launched) {
        // (done)
      } else if (((!whole && !onlyK) || packX || packY) && copiesFit && unitOk && wordsOk && K > 0 &&
          ldx > 0 && ldy > 0 && M <= 0x7fffffff &&
          N <= 0x7fffffff && K <= 0x7fffffff - 64 && tilesM <= 65535 &&
          (tilesM * tilesN >= 16 || (K >= 2048 && Mz * Nz >= 4096))) {
        auto roundUp = [](int64_t v, int64_t to) { return (v + to - 1) / to * to; };
        const int64_t xCp = roundUp(xC, VEC), yCp = roundUp(yC, VEC);
        const size_t xBytes = packXBytes;
        packBytes = packXBytes + packYBytes;
        const int slabs = int((K + BK - 1) / BK);
        bool slicesFill = false;
        SplitPlan plan = planSlices(tilesM * tilesN, K, slicesFill);
        int evenBlocks = workspaceKind == WORKSPACE_HEAP && !slicesFill
                             ? planEvenShares(tilesM * tilesN, slabs, slots)
                             : 0;
        T *W = evenWorkspace(evenBlocks, 128, 128);
        if (evenBlocks)
          plan = SplitPlan();
        const int64_t ldw = (Nz + VEC - 1) / VEC * VEC;
        if (!evenBlocks)
          W = workspaceFor(plan, Mz, ldw, true);
        if (tooLarge)
          return 1;
        if (packBytes) {
          // (one block for the copies and the partial products: asked for
          // once, before anything is launched into it)
          // (a workspace request that found no room left the block as it
          // was: the copies still fit, as checked above)
          unsigned char *base = W ? reinterpret_cast<unsigned char *>(W) - packBytes
                                  : static_cast<unsigned char *>(heapWorkspace(device, packBytes));
          auto pack = [&](const T *src, int64_t ld, int64_t R, int64_t C, int64_t Cp, T *dst) {
            const int64_t words = R * (Cp / VEC);
            hipLaunchKernelGGL(gemm_pack_rows<T>, dim3(unsigned((words + 255) / 256)),
                               dim3(256), 0, stream, src, ld, R, C, dst, Cp, R);
          };
          if (packX) {
            T *dst = reinterpret_cast<T *>(base);
            pack(X, ldx, xR, xC, xCp, dst);
            X = dst;
          }
          if (packY) {
            T *dst = reinterpret_cast<T *>(base + xBytes);
            pack(Y, ldy, yR, yC, yCp, dst);
            Y = dst;
          }
        }
        const int64_t ldxk = packX ? xCp : ldx, ldyk = packY ? yCp : ldy;
        const EvenShares even{evenBlocks ? slabs : 0, int(tilesN)};
        dim3 grid(unsigned(tilesN), unsigned(tilesM), unsigned(plan.slices));
        if (evenBlocks)
          grid = dim3(unsigned(evenBlocks), 1, 1);
#define NMHIP_GEMM_RAGGED(TM, TN, XKC, YNC)                                    \
  hipLaunchKernelGGL((gemm_mfma<T, BK, TM, TN, XKC, YNC, 1>), grid,            \
                     dim3(256), 0, stream, X, Y, cData, int(Mz), int(Nz),      \
                     int(K), ldxk, ldyk, ldz, alpha, beta, plan.sliceK, W, ldw,\
                     even)
#define NMHIP_GEMM_RAGGED_LAYOUTS(TM, TN)                                      \
  do {                                                                         \
    if (xKc && yNc)                                                            \
      NMHIP_GEMM_RAGGED(TM, TN, true, true);                                   \
    else if (xKc)                                                              \
      NMHIP_GEMM_RAGGED(TM, TN, true, false);                                  \
    else if (yNc)                                                              \
      NMHIP_GEMM_RAGGED(TM, TN, false, true);                                  \
    else                                                                       \
      NMHIP_GEMM_RAGGED(TM, TN, false, false);                                 \
  } while (0)
        if constexpr (sizeof(T) == 4) {
          NMHIP_GEMM_RAGGED_LAYOUTS(2, 2);
          lastKernel = evenBlocks        ? "sgemm_mfma_128x128_ragged_even"
                       : plan.slices > 1 ? "sgemm_mfma_128x128_ragged_splitk"
                                         : "sgemm_mfma_128x128_ragged";
        } else {
          NMHIP_GEMM_RAGGED_LAYOUTS(4, 4);
          lastKernel = evenBlocks        ? "dgemm_mfma_128x128_ragged_even"
                       : plan.slices > 1 ? "dgemm_mfma_128x128_ragged_splitk"
                                         : "dgemm_mfma_128x128_ragged";
        }
        lastPacked = packBytes != 0;
        if (evenBlocks)
          evenFold(W, evenBlocks, slabs, tilesM, tilesN, 128, Mz, Nz, ldz, cData);
        else if (plan.slices > 1)
          fold(plan, W, Mz, Nz, ldw, ldz, cData);
#undef NMHIP_GEMM_RAGGED_LAYOUTS
#undef NMHIP_GEMM_RAGGED
        launched = true;
      } else if (unitOk && mostly && Mt > 0 && Nt > 0 && Kt > 0 &&
          ldx % VEC == 0 && ldy % VEC == 0 && ldx > 0 && ldy > 0 &&
          aligned16(X) && aligned16(Y) && M <= 0x7fffffff && N <= 0x7fffffff &&
          K <= 0x7fffffff && Mz <= 65535 * 32) {
        const int slabK = big ? bigSlab : BK;
        const int slabs = int(Kt / slabK);
        SplitPlan plan;
        bool slicesFill = false;
        if (!big)
          plan = planSlices((Mt / BM) * (Nt / BN), Kt, slicesFill);
        int evenBlocks = big ? bigEven
                         : workspaceKind == WORKSPACE_HEAP && !slicesFill
                             ? planEvenShares((Mt / BM) * (Nt / BN), slabs, slots)
                             : 0;
        T *W = evenWorkspace(evenBlocks, BM, BN);
        if (evenBlocks)
          plan = SplitPlan();
        else if (!big)
          W = workspaceFor(plan, Mt, Nt, true);
        if (tooLarge)
          return 1;
        const EvenShares even{evenBlocks ? slabs : 0, int(Nt / BN)};
        dim3 grid(unsigned(Nt / BN), unsigned(Mt / BM), unsigned(plan.slices));
        if (evenBlocks)
          grid = dim3(unsigned(evenBlocks), 1, 1);
#define NMHIP_GEMM_LAUNCH(SLAB, TM, TN, XKC, YNC)                              \
  hipLaunchKernelGGL((gemm_mfma<T, SLAB, TM, TN, XKC, YNC>), grid, dim3(256),  \
                     0, stream, X, Y, cData, int(Mt), int(Nt), int(Kt), ldx,   \
                     ldy, ldz, alpha, beta, plan.sliceK, W, int64_t(Nt), even)
#define NMHIP_GEMM_LAYOUTS(SLAB, TM, TN)                                       \
  do {                                                                         \
    if (xKc && yNc)                                                            \
      NMHIP_GEMM_LAUNCH(SLAB, TM, TN, true, true);                             \
    else if (xKc)                                                              \
      NMHIP_GEMM_LAUNCH(SLAB, TM, TN, true, false);                            \
    else if (yNc)                                                              \
      NMHIP_GEMM_LAUNCH(SLAB, TM, TN, false, true);                            \
    else                                                                       \
      NMHIP_GEMM_LAUNCH(SLAB, TM, TN, false, false);                           \
  } while (0)
        if constexpr (sizeof(T) == 4) {
          if (big && bigSlab == 2 * BK)
            NMHIP_GEMM_LAYOUTS(2 * BK, 4, 4);
          else if (big)
            NMHIP_GEMM_LAYOUTS(BK, 4, 4);
          else
            NMHIP_GEMM_LAYOUTS(BK, 2, 2);
          static const char *const names[2][4][2] = {
              {{"sgemm_mfma_128x128", "sgemm_mfma_128x128+edges"},
               {"sgemm_mfma_128x128_splitk", "sgemm_mfma_128x128_splitk+edges"},
               {"sgemm_mfma_128x128_even", "sgemm_mfma_128x128_even+edges"},
               {"", ""}},
              {{"sgemm_mfma_256x256", "sgemm_mfma_256x256+edges"},
               {"", ""},
               {"sgemm_mfma_256x256_even", "sgemm_mfma_256x256_even+edges"},
               {"", ""}}};
          lastKernel = names[big ? 1 : 0][evenBlocks ? 2 : plan.slices > 1 ? 1 : 0][whole ? 0 : 1];
        } else {
          NMHIP_GEMM_LAYOUTS(BK, 4, 4);
          lastKernel = evenBlocks ? (whole ? "dgemm_mfma_128x128_even"
                                           : "dgemm_mfma_128x128_even+edges")
                       : plan.slices > 1
                           ? (whole ? "dgemm_mfma_128x128_splitk"
                                    : "dgemm_mfma_128x128_splitk+edges")
                           : (whole ? "dgemm_mfma_128x128"
                                    : "dgemm_mfma_128x128+edges");
        }
        if (evenBlocks)
          evenFold(W, evenBlocks, slabs, Mt / BM, Nt / BN, BM, Mt, Nt, ldz, cData);
        else if (plan.slices > 1)
          fold(plan, W, Mt, Nt, Nt, ldz, cData);
#undef NMHIP_GEMM_LAYOUTS
#undef NMHIP_GEMM_LAUNCH
        // Z[m0:m0+m, n0:n0+n] = alpha X[m0.., k0:k0+k] Y[k0.., n0..] + bz Z
        auto edge = [&](int64_t m0, int64_t m, int64_t n0, int64_t n, int64_t k0,
                        int64_t k, T bz) {
          if (m <= 0 || n <= 0)
            return;
          const dim3 g = genericGrid(m, n);
          hipLaunchKernelGGL(gemm_generic<T>, g, dim3(256), 0, stream,
                             X + m0 * xm + k0 * xk, Y + k0 * yk + n0 * yn,
                             cData + m0 * ldz + n0, m, n, k, xm, xk, yk, yn, ldz,
                             int64_t(1), alpha, bz, k, static_cast<T *>(nullptr));
        };
        if (Kt < K)
          edge(0, Mt, 0, Nt, Kt, K - Kt, T(1)); // the rest of K, on top
        edge(Mt, Mz - Mt, 0, Nz, 0, K, beta);   // rows below the tiles
        edge(0, Mt, Nt, Nz - Nt, 0, K, beta);   // columns right of them
        launched = true;
      }
    }
    if (!launched) {
      dim3 grid = genericGrid(M, N);
      // A small product of long operands (a Gram matrix of a few columns):
      // K in slices over some 2048 blocks, of 512 elements or more each;
      // the partial sums (at most 16 MiB: a tile's are 8 KiB) are added in
      // index order by gemm_thin_fold.
      const int64_t tiles = int64_t(grid.x) * grid.y;
      SplitPlan plan;
      int64_t kSlice = K;
      if (tiles <= cus && K >= 2048) {
        int64_t slices = 2048 / tiles;
        if (slices > K / 512)
          slices = K / 512;
        kSlice = ((K + slices - 1) / slices + 31) / 32 * 32;
        plan.slices = int((K + kSlice - 1) / kSlice);
      }
      T *part = workspaceFor(plan, M, N);
      if (!part)
        plan.slices = 1, kSlice = K;
      grid.z = unsigned(plan.slices);
      hipLaunchKernelGGL(gemm_generic<T>, grid, dim3(256), 0, stream, aData,
                         bData, cData, M, N, K, int64_t(a->strides[0]),
                         int64_t(a->strides[1]), int64_t(b->strides[0]),
                         int64_t(b->strides[1]), int64_t(c->strides[0]),
                         int64_t(c->strides[1]), alpha, beta, kSlice, part);
      if (part)
        hipLaunchKernelGGL(gemm_thin_fold<T>, dim3(unsigned((N + 15) / 16), unsigned(M)),
                           dim3(256), 0, stream, part, plan.slices, int(M), N, N, cData,
                           int64_t(c->strides[0]), int64_t(c->strides[1]), alpha, beta);
      lastKernel = part ? (sizeof(T) == 4 ? "sgemm_generic_splitk" : "dgemm_generic_splitk")
                        : (sizeof(T) == 4 ? "sgemm_generic" : "dgemm_generic");
    }
    checkHip(hipGetLastError(), "gemm launch");
  }
  // The reference call returns only when C is complete (.wait(), 127/145).
  checkHip(hipStreamSynchronize(stream), "hipStreamSynchronize");
  if (workspaceTurn.owns_lock() && workspaceKind == WORKSPACE_HEAP)
    trimHeapWorkspace(device);
  return 0;
}

} // namespace

#define NMHIP_MATH_EXPORT extern "C" __attribute__((visibility("default")))

NMHIP_MATH_EXPORT void mkl_gemm_float32_device(void *queue,
                                               const NmhipMemref2F32 *a,
                                               const NmhipMemref2F32 *b,
                                               float alpha, float beta,
                                               NmhipMemref2F32 *c) {
  (void)deviceGemm<float>(queue, a, b, c, alpha, beta, WORKSPACE_HEAP);
}

NMHIP_MATH_EXPORT void mkl_gemm_float64_device(void *queue,
                                               const NmhipMemref2F64 *a,
                                               const NmhipMemref2F64 *b,
                                               double alpha, double beta,
                                               NmhipMemref2F64 *c) {
  (void)deviceGemm<double>(queue, a, b, c, alpha, beta, WORKSPACE_HEAP);
}

NMHIP_MATH_EXPORT int mkl_gemm_float32_device_noalloc(
    void *queue, const NmhipMemref2F32 *a, const NmhipMemref2F32 *b,
    float alpha, float beta, NmhipMemref2F32 *c) {
  return deviceGemm<float>(queue, a, b, c, alpha, beta, WORKSPACE_FIXED);
}

NMHIP_MATH_EXPORT void nmrtMathRuntimeInit(void) {}
NMHIP_MATH_EXPORT void nmrtMathRuntimeFinalize(void) {
  releaseHeapWorkspaces();
}

NMHIP_MATH_EXPORT const char *nmhipMathLastKernel(void) {
  if (!lastPacked)
    return lastKernel;
  thread_local char name[96];
  std::snprintf(name, sizeof(name), "%s+packed", lastKernel);
  return name;
}
