/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * CPU restatement of the reference's @njit(parallel=True) CPU path for the
 * offloaded hot path.  Only tests/, __graft_entry__.smoke() and bench.py's
 * cpu_baseline leg may build, load or call this file; nothing under
 * numba_mlir_amd/ does.
 *
 * The reference's CPU path cannot be built here (it needs numba 0.60, LLVM/
 * MLIR at a pinned commit, oneTBB and MKL), so each function restates the
 * algorithm of the reference file:line it cites:
 *
 *  - loop partitioning: nmrtParallelFor splits every parallel dimension into
 *    blocks with grain max(1, min(count / threads / 2, 64))
 *    (numba_mlir_runtime/lib/TbbParallel.cpp:98-217, grain 129-132).  TBB
 *    hands blocks to threads dynamically; here block c goes to thread
 *    c % threads so results are reproducible.
 *  - reductions: one accumulator per thread, initialised to the neutral
 *    element, combined serially in thread order after the loop
 *    (mlir_compiler/lib/pipelines/ParallelToTbb.cpp:50-198).
 *  - transcendentals: host libm (math.* lowered to libm calls,
 *    mlir_compiler/lib/pipelines/LowerToLlvm.cpp:1835-1838).
 *  - no fma contraction (needs fastmath in the reference); build with
 *    -ffp-contract=off.
 *
 * What pins each function is listed next to it ("pinned by").
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int64_t orc_grain(int64_t count, int threads) {
  int64_t g = count / threads / 2;
  if (g > 64)
    g = 64;
  if (g < 1)
    g = 1;
  return g;
}

static int orc_threads(int threads) {
  if (threads > 0)
    return threads;
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

int orc_max_threads(void) { return orc_threads(0); }

/* ------------------------------------------------------------------------ */
/* Elementwise add with broadcasting, float64 and int64.
 * out[i,j] = a[i*sa0 + j*sa1] + b[i*sb0 + j*sb1]; a broadcast dimension has
 * stride 0 (numba_mlir/numba_mlir/mlir/numpy/funcs.py:457-462 -> eltwise,
 * linalg_builder.py:297-325; broadcast NtensorToLinalg.cpp:487-557).
 * Pinned by: one IEEE add per element == numpy a + b bit for bit
 * (tests/test_numpy.py:483-514 fixtures). */
#define ORC_DEFINE_ADD(NAME, T)                                                \
  void NAME(const T *a, int64_t sa0, int64_t sa1, const T *b, int64_t sb0,     \
            int64_t sb1, T *out, int64_t n0, int64_t n1, int threads) {        \
    threads = orc_threads(threads);                                            \
    const int64_t g0 = orc_grain(n0, threads);                                 \
    const int64_t blocks = (n0 + g0 - 1) / g0;                                 \
    _Pragma("omp parallel for num_threads(threads) schedule(static, 1)")       \
    for (int64_t blk = 0; blk < blocks; ++blk) {                               \
      int64_t lo = blk * g0, hi = lo + g0 > n0 ? n0 : lo + g0;                 \
      for (int64_t i = lo; i < hi; ++i)                                        \
        for (int64_t j = 0; j < n1; ++j)                                       \
          out[i * n1 + j] = a[i * sa0 + j * sa1] + b[i * sb0 + j * sb1];       \
    }                                                                          \
  }

ORC_DEFINE_ADD(orc_add_f64, double)
ORC_DEFINE_ADD(orc_add_f32, float)
ORC_DEFINE_ADD(orc_add_i64, int64_t)
ORC_DEFINE_ADD(orc_add_i32, int32_t)

/* ------------------------------------------------------------------------ */
/* Black-Scholes, the fused body of tests/test_numpy.py:2827-2852.
 *
 * Typing (wide != 0, the reference's): a Python float/int literal is
 * float64/int64 (linalg_builder.py:278-291) and mixed operands promote with
 * numpy.promote_types (261-275), so
 *   mr = -rate                               float32
 *   sig_sig_two = volatility*volatility*2    float32*float32 -> *int64: float64
 *   a = log(P / S); b = T * mr               float32
 *   z = T * sig_sig_two; c = 0.25 * z        float64
 *   y = 1.0 / sqrt(z)                        float64
 *   w1 = (a - b + c) * y; w2 = (a - b - c)*y (a - b) float32, rest float64
 *   d1 = 0.5 + 0.5 * erf(w1); d2 likewise    float64
 *   Se = exp(b) * S                          float32
 *   r = P * d1 - Se * d2                     float64
 *   call = r; put = r - P + Se               float64, stored as float32
 * wide == 0 evaluates the same tree in float32 (NumPy's own result for this
 * source under weak Python scalars).
 * Pinned by: float64 evaluation of the closed-form Black-Scholes price with
 * scipy's normal CDF, put-call parity, and the reference's own atol 1e-3
 * agreement between the two typings (test_numpy.py:2862-2863). */
void orc_black_scholes_f32(const float *price, const float *strike,
                           const float *t, float rate, float volatility,
                           float *call, float *put, int64_t n, int wide,
                           int threads) {
  threads = orc_threads(threads);
  const float mr = -rate;
  const int64_t g = orc_grain(n, threads);
  const int64_t blocks = (n + g - 1) / g;
  if (wide) {
    const double sig_sig_two = (double)(volatility * volatility) * 2.0;
#pragma omp parallel for num_threads(threads) schedule(static, 64)
    for (int64_t blk = 0; blk < blocks; ++blk) {
      int64_t lo = blk * g, hi = lo + g > n ? n : lo + g;
      for (int64_t i = lo; i < hi; ++i) {
        const float P = price[i], S = strike[i], T = t[i];
        const float a = logf(P / S);
        const float b = T * mr;
        const double z = (double)T * sig_sig_two;
        const double c = 0.25 * z;
        const double y = 1.0 / sqrt(z);
        const float amb = a - b;
        const double w1 = ((double)amb + c) * y;
        const double w2 = ((double)amb - c) * y;
        const double d1 = 0.5 + 0.5 * erf(w1);
        const double d2 = 0.5 + 0.5 * erf(w2);
        const float Se = expf(b) * S;
        const double r = (double)P * d1 - (double)Se * d2;
        call[i] = (float)r;
        put[i] = (float)(r - (double)P + (double)Se);
      }
    }
  } else {
    const float sig_sig_two = volatility * volatility * 2.0f;
#pragma omp parallel for num_threads(threads) schedule(static, 64)
    for (int64_t blk = 0; blk < blocks; ++blk) {
      int64_t lo = blk * g, hi = lo + g > n ? n : lo + g;
      for (int64_t i = lo; i < hi; ++i) {
        const float P = price[i], S = strike[i], T = t[i];
        const float a = logf(P / S);
        const float b = T * mr;
        const float z = T * sig_sig_two;
        const float c = 0.25f * z;
        const float y = 1.0f / sqrtf(z);
        const float amb = a - b;
        const float w1 = (amb + c) * y;
        const float w2 = (amb - c) * y;
        const float d1 = 0.5f + 0.5f * erff(w1);
        const float d2 = 0.5f + 0.5f * erff(w2);
        const float Se = expf(b) * S;
        const float r = P * d1 - Se * d2;
        call[i] = r;
        put[i] = r - P + Se;
      }
    }
  }
}

/* ------------------------------------------------------------------------ */
/* sum(axis=1), float32 -> float32: rows are the parallel loop, the reduction
 * is the row's inner loop accumulating in float32 from 0
 * (numpy/funcs.py:186-214, 222-227).
 * Pinned by: exact on small-integer inputs (test_numpy.py:760-793,
 * test_gpu.py:2068-2098 use arange); float64 ground truth within rounding
 * bounds on random data. */
void orc_sum_axis1_f32(const float *x, int64_t n0, int64_t n1, int64_t s0,
                       int64_t s1, float *out, int threads) {
  threads = orc_threads(threads);
  const int64_t g = orc_grain(n0, threads);
  const int64_t blocks = (n0 + g - 1) / g;
#pragma omp parallel for num_threads(threads) schedule(static, 1)
  for (int64_t blk = 0; blk < blocks; ++blk) {
    int64_t lo = blk * g, hi = lo + g > n0 ? n0 : lo + g;
    for (int64_t i = lo; i < hi; ++i) {
      float acc = 0.0f;
      for (int64_t j = 0; j < n1; ++j)
        acc += x[i * s0 + j * s1];
      out[i] = acc;
    }
  }
}

/* sum(axis=0), int32 -> int64 (promote_int, numpy/funcs.py:120-123, 210):
 * columns are the parallel loop (the reduction dimension is moved innermost,
 * mlir_compiler/lib/pipelines/PlierToLinalg.cpp:4212-4276).
 * Pinned by: exact integer arithmetic == x.sum(axis=0, dtype=int64). */
void orc_sum_axis0_i32(const int32_t *x, int64_t n0, int64_t n1, int64_t s0,
                       int64_t s1, int64_t *out, int threads) {
  threads = orc_threads(threads);
  const int64_t g = orc_grain(n1, threads);
  const int64_t blocks = (n1 + g - 1) / g;
#pragma omp parallel for num_threads(threads) schedule(static, 1)
  for (int64_t blk = 0; blk < blocks; ++blk) {
    int64_t lo = blk * g, hi = lo + g > n1 ? n1 : lo + g;
    for (int64_t j = lo; j < hi; ++j)
      out[j] = 0;
    /* row-by-row walk of the block keeps the host's cache lines whole; the
     * integer sum does not depend on the order. */
    for (int64_t i = 0; i < n0; ++i)
      for (int64_t j = lo; j < hi; ++j)
        out[j] += (int64_t)x[i * s0 + j * s1];
  }
}

/* sqrt(sum(x * x)) over n float32 values: full reduction with per-thread
 * float32 accumulators and a serial combine in thread order
 * (ParallelToTbb.cpp:124-194), then sqrtf of the 0-d result
 * (numpy/funcs.py:364-368).
 * Pinned by: float64 ground truth within a forward error bound; exact on
 * small-integer inputs (3-4-5 style). */
float orc_norm2_f32(const float *x, int64_t n, int threads) {
  threads = orc_threads(threads);
  float *acc = (float *)calloc((size_t)threads, sizeof(float));
  const int64_t g = orc_grain(n, threads);
  const int64_t blocks = (n + g - 1) / g;
#pragma omp parallel num_threads(threads)
  {
#ifdef _OPENMP
    const int tid = omp_get_thread_num();
    const int nth = omp_get_num_threads();
#else
    const int tid = 0, nth = 1;
#endif
    float local = 0.0f;
    /* block c -> thread c % threads, blocks visited in increasing order */
    for (int64_t blk = tid; blk < blocks; blk += nth) {
      int64_t lo = blk * g, hi = lo + g > n ? n : lo + g;
      for (int64_t i = lo; i < hi; ++i)
        local += x[i] * x[i];
    }
    acc[tid] = local;
  }
  float total = 0.0f;
  for (int i = 0; i < threads; ++i)
    total += acc[i];
  free(acc);
  return sqrtf(total);
}

/* ------------------------------------------------------------------------ */
/* Pairwise distance @kernel body (tests/test_gpu.py:1397-1408):
 *   d = 0.0; for k: tmp = X1[i,k] - X2[j,k]; d += tmp * tmp; D[i,j] = sqrt(d)
 * `tmp` has the array dtype, `d` is float64.  Work-items are independent, so
 * the launch geometry does not affect D.
 * Pinned by: closed form sqrt(3)*|3(i-j)-5| on the reference's arange fixture
 * (test_gpu.py:1413-1418), brute force, scipy cdist. */
void orc_pairwise_f64(const double *X1, const double *X2, double *D, int64_t n1,
                      int64_t n2, int64_t dims, int threads) {
  threads = orc_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static, 16)
  for (int64_t i = 0; i < n1; ++i)
    for (int64_t j = 0; j < n2; ++j) {
      double d = 0.0;
      for (int64_t k = 0; k < dims; ++k) {
        double tmp = X1[i * dims + k] - X2[j * dims + k];
        d += tmp * tmp;
      }
      D[i * n2 + j] = sqrt(d);
    }
}

void orc_pairwise_f32(const float *X1, const float *X2, float *D, int64_t n1,
                      int64_t n2, int64_t dims, int threads) {
  threads = orc_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static, 16)
  for (int64_t i = 0; i < n1; ++i)
    for (int64_t j = 0; j < n2; ++j) {
      double d = 0.0;
      for (int64_t k = 0; k < dims; ++k) {
        float tmp = X1[i * dims + k] - X2[j * dims + k];
        d += (double)(tmp * tmp);
      }
      D[i * n2 + j] = (float)sqrt(d);
    }
}

/* ------------------------------------------------------------------------ */
/* Matmul c = alpha * a @ b + beta * c with arbitrary element strides.
 * The reference routes np.dot to MKL's sgemm when MKL is present
 * (numpy/funcs.py:759-785, math_runtime/lib/NumpyLinalg.cpp:61-107; MKL is a
 * third-party binary not under the reference tree) and otherwise to the
 * generic (d0,d1,d2) a*b+c contraction in float32, k innermost
 * (numpy/funcs.py:788-801).  This is the latter: float32 products and
 * float32 accumulation in k order, then __internal_gemm's
 * beta * c + alpha * dot (866-876).
 * Pinned by: exact integer-valued fixtures (test_gpu.py:2101-2193,
 * linalg_gemmf.mlir:8-19) and a float64 ground truth on random data. */
void orc_gemm_f32(const float *a, int64_t as0, int64_t as1, const float *b,
                  int64_t bs0, int64_t bs1, float *c, int64_t cs0, int64_t cs1,
                  int64_t m, int64_t n, int64_t k, float alpha, float beta,
                  int threads) {
  threads = orc_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static, 4)
  for (int64_t i = 0; i < m; ++i)
    for (int64_t j = 0; j < n; ++j) {
      float acc = 0.0f;
      for (int64_t p = 0; p < k; ++p)
        acc = a[i * as0 + p * as1] * b[p * bs0 + j * bs1] + acc;
      float *dst = c + i * cs0 + j * cs1;
      *dst = beta == 0.0f ? alpha * acc : beta * *dst + alpha * acc;
    }
}

/* Same contraction with float64 accumulation: ground truth for tolerance
 * checks of float32 matmul. */
void orc_gemm_f32_acc64(const float *a, int64_t as0, int64_t as1,
                        const float *b, int64_t bs0, int64_t bs1, double *c,
                        int64_t m, int64_t n, int64_t k, int threads) {
  threads = orc_threads(threads);
#pragma omp parallel for num_threads(threads) schedule(static, 4)
  for (int64_t i = 0; i < m; ++i)
    for (int64_t j = 0; j < n; ++j) {
      double acc = 0.0;
      for (int64_t p = 0; p < k; ++p)
        acc += (double)a[i * as0 + p * as1] * (double)b[p * bs0 + j * bs1];
      c[i * n + j] = acc;
    }
}

/* ------------------------------------------------------------------------ */
/* Block-size suggestion fallback (numba_mlir_gpu_runtime_sycl/lib/
 * GpuModule.cpp:453-509): maxWg = downPow2(max workgroup size); per dim
 * l = g > 1 ? min(g, maxWg) : 1; maxWg /= upPow2(l).
 * Pinned by: hand-computed table in tests. */
static uint32_t orc_down_pow2(uint32_t x) {
  x |= (x >> 1);
  x |= (x >> 2);
  x |= (x >> 4);
  x |= (x >> 8);
  x |= (x >> 16);
  return x - (x >> 1);
}

static uint32_t orc_up_pow2(uint32_t x) {
  x--;
  x |= (x >> 1);
  x |= (x >> 2);
  x |= (x >> 4);
  x |= (x >> 8);
  x |= (x >> 16);
  x++;
  return x;
}

void orc_suggest_block_size(uint32_t max_wg, const uint32_t *global,
                            uint32_t *block, size_t ndims) {
  uint32_t wg = orc_down_pow2(max_wg);
  for (size_t i = 0; i < ndims; ++i) {
    uint32_t g = global[i];
    if (g > 1) {
      uint32_t l = g < wg ? g : wg;
      block[i] = l;
      wg /= orc_up_pow2(l);
    } else {
      block[i] = 1;
    }
  }
}
