/*
 * scorch_oracle.c -- CPU restatement of Scorch's prebuilt CSR sparse x dense
 * kernels.  TEST INFRASTRUCTURE ONLY: this file is the checker the HIP path
 * is compared against (tests/, the smoke check and the cpu_baseline leg of
 * bench.py).  Nothing in the shipped package may call it.
 *
 * Every routine takes flat pointers (the reference takes pybind-wrapped
 * torch tensors; the arrays underneath are the same: int32 pos/crd, flat
 * row-major values) and writes into caller-provided output unless it says
 * otherwise.  Each routine names the reference lines whose algorithm it
 * restates.  Parallel structure (OpenMP schedule, chunk formula, per-thread
 * workspace) follows the reference so that timing it is a fair stand-in for
 * timing the reference itself.
 *
 * Pinned against the reference's own outputs (golden fixtures and, where it
 * is built, its compiled module): every routine here except
 * oracle_softmax_csr_f32, which is PARITY UNPINNED -- the reference has no
 * native row softmax and no test vector for one; that routine is pinned by
 * mathematics only (scipy's softmax, shift invariance, rows summing to one).
 *
 * Build: see oracle/Makefile (flags follow the reference's setup.py:9-14,50:
 * -O3 -ffast-math -funroll-loops -fopenmp).
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <float.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

static int oracle_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

ORACLE_API int oracle_num_threads(void) { return oracle_threads(); }

/* chunk = clamp(total / (threads * 128), 16, 256): the work-stealing grain of
 * csrc/spmm.h:2032-2034 and csrc/kernels.h:531-532. */
static int steal_chunk(int64_t total, int threads) {
  int64_t c = total / ((int64_t)threads * 128);
  if (c > 256) c = 256;
  if (c < 16) c = 16;
  return (int)c;
}

/* ------------------------------------------------------------------------
 * SpMM fp32, the symbol fp32 scorch.matmul dispatches to.
 * Restates spmm_csr_float_v2, csrc/spmm.h:2007-2089:
 *   - C is zero-filled first (2024-2025); rows with no entries are skipped
 *     and keep that zero (2053);
 *   - column tile kTile = tile rounded up to 16 (2028);
 *   - threads take `chunk` consecutive rows at a time from a shared atomic
 *     counter (2035-2047);
 *   - per row and column tile: clear a private 64-byte aligned workspace,
 *     ws[k] += a * B[j, k0 + k] with the next B row prefetched, then copy the
 *     workspace to C (2056-2075).
 * `zero_fill` = 1 reproduces the reference call exactly (memset inside);
 * 0 lets a caller time the loop alone on a pre-zeroed C.
 * ---------------------------------------------------------------------- */
ORACLE_API void oracle_spmm_csr_f32_v2(int M, int N, const int32_t *pos,
                                       const int32_t *crd, const float *aval,
                                       const float *B, float *C, int tile,
                                       int zero_fill) {
  const size_t total = (size_t)M * (size_t)N;
  if (zero_fill) memset(C, 0, total * sizeof(float));
  const int ktile = (tile + 15) & ~15;
  const int threads = oracle_threads();
  const int chunk = steal_chunk(M > 0 ? pos[M] : 0, threads);
  int next_row = 0;

#pragma omp parallel
  {
    float *ws = (float *)aligned_alloc(64, (size_t)ktile * sizeof(float));
    for (;;) {
      const int first = __atomic_fetch_add(&next_row, chunk, __ATOMIC_RELAXED);
      if (first >= M) break;
      const int last = first + chunk < M ? first + chunk : M;
      for (int i = first; i < last; ++i) {
        const int lo = pos[i], hi = pos[i + 1];
        if (lo == hi) continue;
        float *crow = C + (size_t)i * (size_t)N;
        for (int k0 = 0; k0 < N; k0 += ktile) {
          const int w = N - k0 < ktile ? N - k0 : ktile;
          memset(ws, 0, (size_t)w * sizeof(float));
          for (int p = lo; p < hi; ++p) {
            const float a = aval[p];
            const float *brow = B + (size_t)crd[p] * (size_t)N + k0;
            if (p + 1 < hi)
              __builtin_prefetch(B + (size_t)crd[p + 1] * (size_t)N + k0, 0, 1);
            for (int k = 0; k < w; ++k) ws[k] += a * brow[k];
          }
          memcpy(crow + k0, ws, (size_t)w * sizeof(float));
        }
      }
    }
    free(ws);
  }
}

/* ------------------------------------------------------------------------
 * SpMM for the four dtypes, accumulating straight into a zeroed C.
 * Restates spmm_csr_typed<T>, csrc/spmm.h:91-150 (bound as
 * prebuilt_spmm_csr_{f32,f64,i32,i64}, csrc/ops.cpp:30-39,92-98):
 * C zero-filled (114), rows in parallel with schedule(dynamic,16) (121),
 * C[i,k] += a * B[j,k] in nonzero order (124-137).  Integer types wrap:
 * the arithmetic is done unsigned so that the wrap is defined here.
 * ---------------------------------------------------------------------- */
#define DEFINE_SPMM_TYPED(NAME, T, ACC)                                        \
  ORACLE_API void NAME(int M, int N, const int32_t *pos, const int32_t *crd,   \
                       const T *aval, const T *B, T *C) {                      \
    memset(C, 0, (size_t)M * (size_t)N * sizeof(T));                           \
    _Pragma("omp parallel for schedule(dynamic, 16)")                          \
    for (int i = 0; i < M; ++i) {                                              \
      T *crow = C + (size_t)i * (size_t)N;                                     \
      const int hi = pos[i + 1];                                               \
      for (int p = pos[i]; p < hi; ++p) {                                      \
        if (p + 1 < hi)                                                        \
          __builtin_prefetch(B + (size_t)crd[p + 1] * (size_t)N, 0, 1);        \
        const ACC a = (ACC)aval[p];                                            \
        const T *brow = B + (size_t)crd[p] * (size_t)N;                        \
        for (int k = 0; k < N; ++k)                                            \
          crow[k] = (T)((ACC)crow[k] + a * (ACC)brow[k]);                      \
      }                                                                        \
    }                                                                          \
  }

DEFINE_SPMM_TYPED(oracle_spmm_csr_f32, float, float)
DEFINE_SPMM_TYPED(oracle_spmm_csr_f64, double, double)
DEFINE_SPMM_TYPED(oracle_spmm_csr_i32, int32_t, uint32_t)
DEFINE_SPMM_TYPED(oracle_spmm_csr_i64, int64_t, uint64_t)

/* ------------------------------------------------------------------------
 * Fused SpMM + bias (+ ReLU), fp32.
 * Restates spmm_csr_bias_act<float, relu>, csrc/spmm.h:28-89 (bound as
 * spmm_csr_bias_float / spmm_csr_bias_relu_float, csrc/ops.cpp:167-208):
 * each row starts as the bias vector (55-57), accumulates its nonzeros
 * (60-71), then is clamped at zero in place when relu is set (74-79).
 * No zero fill: every row is written.
 * ---------------------------------------------------------------------- */
ORACLE_API void oracle_spmm_csr_bias_act_f32(int M, int N, const int32_t *pos,
                                             const int32_t *crd,
                                             const float *aval, const float *B,
                                             const float *bias, float *C,
                                             int relu) {
#pragma omp parallel for schedule(dynamic, 16)
  for (int i = 0; i < M; ++i) {
    float *crow = C + (size_t)i * (size_t)N;
    const int hi = pos[i + 1];
    for (int k = 0; k < N; ++k) crow[k] = bias[k];
    for (int p = pos[i]; p < hi; ++p) {
      if (p + 1 < hi)
        __builtin_prefetch(B + (size_t)crd[p + 1] * (size_t)N, 0, 1);
      const float a = aval[p];
      const float *brow = B + (size_t)crd[p] * (size_t)N;
      for (int k = 0; k < N; ++k) crow[k] += a * brow[k];
    }
    if (relu)
      for (int k = 0; k < N; ++k) crow[k] = crow[k] > 0.0f ? crow[k] : 0.0f;
  }
}

/* ------------------------------------------------------------------------
 * SDDMM fp32 with a COO mask: out[p] = s[p] * <A[row[p], :], B[col[p], :]>.
 * Restates sddmm_coo_float_prebuilt, csrc/kernels.h:508-570: B is indexed
 * [j, k] (548), i.e. the product is A * B^T sampled at the mask; threads take
 * `chunk` consecutive nonzeros from an atomic counter (531-540); the output
 * keeps the mask's index arrays untouched (567), so only values are produced.
 * ---------------------------------------------------------------------- */
ORACLE_API void oracle_sddmm_coo_f32(int64_t nnz, int K, const int32_t *row,
                                     const int32_t *col, const float *sval,
                                     const float *A, const float *B,
                                     float *out) {
  const int threads = oracle_threads();
  const int chunk = steal_chunk(nnz, threads);
  int64_t next = 0;
#pragma omp parallel
  {
    for (;;) {
      const int64_t first = __atomic_fetch_add(&next, (int64_t)chunk, __ATOMIC_RELAXED);
      if (first >= nnz) break;
      const int64_t last = first + chunk < nnz ? first + chunk : nnz;
      for (int64_t p = first; p < last; ++p) {
        const float *arow = A + (size_t)row[p] * (size_t)K;
        const float *brow = B + (size_t)col[p] * (size_t)K;
        if (p + 1 < last) {
          __builtin_prefetch(A + (size_t)row[p + 1] * (size_t)K, 0, 1);
          __builtin_prefetch(B + (size_t)col[p + 1] * (size_t)K, 0, 1);
        }
        float dot = 0.0f;
        for (int k = 0; k < K; ++k) dot += arow[k] * brow[k];
        out[p] = sval[p] * dot;
      }
    }
  }
}

/* ------------------------------------------------------------------------
 * SDDMM fp32 with a CSR mask.  The reference has no native kernel for this
 * form: einsum("ij,ik,jk->ij") with a "d,s" mask goes through its code
 * generator, which infers an all-coordinate output (src/scorch/ops.py:638-666)
 * and emits a scalar-accumulator loop nest (compiler/iter_lattice.py:1011-1098)
 * that appends one output entry per mask entry, in mask order, without
 * dropping zeros (compiler/cin_lowerer.py:2286-2326).  This routine restates
 * that result: out_row/out_col are the coordinate arrays of the output
 * (row of each entry, copy of crd), out_val[p] = s[p] * <A[i,:], B[j,:]>.
 * The row loop is serial in the generated code; here rows are independent and
 * run under a static schedule, which does not change any value.
 * ---------------------------------------------------------------------- */
ORACLE_API void oracle_sddmm_csr_f32(int M, int K, const int32_t *pos,
                                     const int32_t *crd, const float *sval,
                                     const float *A, const float *B,
                                     int32_t *out_row, int32_t *out_col,
                                     float *out_val) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < M; ++i) {
    const float *arow = A + (size_t)i * (size_t)K;
    for (int p = pos[i]; p < pos[i + 1]; ++p) {
      const float *brow = B + (size_t)crd[p] * (size_t)K;
      float acc = 0.0f;
      for (int k = 0; k < K; ++k) acc += arow[k] * brow[k];
      if (out_row) out_row[p] = i;
      if (out_col) out_col[p] = crd[p];
      out_val[p] = sval[p] * acc;
    }
  }
}

/* ------------------------------------------------------------------------
 * SpMV for the four dtypes: y[i] = sum_p a[p] * x[crd[p]].
 * Restates spmv_csr<T>, csrc/kernels.h:13-49 (bound as
 * prebuilt_spmv_csr_{f32,f64,i32,i64}, csrc/ops.cpp:52-61,100-101):
 * scalar accumulator per row, rows under schedule(static) (31-39).
 * ---------------------------------------------------------------------- */
#define DEFINE_SPMV_TYPED(NAME, T, ACC)                                        \
  ORACLE_API void NAME(int M, const int32_t *pos, const int32_t *crd,          \
                       const T *aval, const T *x, T *y) {                      \
    _Pragma("omp parallel for schedule(static)")                               \
    for (int i = 0; i < M; ++i) {                                              \
      ACC acc = (ACC)0;                                                        \
      for (int p = pos[i]; p < pos[i + 1]; ++p)                                \
        acc += (ACC)aval[p] * (ACC)x[crd[p]];                                  \
      y[i] = (T)acc;                                                           \
    }                                                                          \
  }

DEFINE_SPMV_TYPED(oracle_spmv_csr_f32, float, float)
DEFINE_SPMV_TYPED(oracle_spmv_csr_f64, double, double)
DEFINE_SPMV_TYPED(oracle_spmv_csr_i32, int32_t, uint32_t)
DEFINE_SPMV_TYPED(oracle_spmv_csr_i64, int64_t, uint64_t)

/* ------------------------------------------------------------------------
 * Row softmax over the stored values of a CSR matrix, fp32:
 * out[p] = exp(scale*v[p] - max_row) / sum_row exp(scale*v[q] - max_row).
 * Restates _sparse_softmax_csr_vectorized, bench/bench_sparse_transformer.py:
 * 277-297, applied to `scores * scale` as at 362-368 of the same file.  The
 * reference composes this from torch scatter ops; the arithmetic per row is
 * the textbook max-shifted softmax.  Empty rows produce nothing.
 * ---------------------------------------------------------------------- */
ORACLE_API void oracle_softmax_csr_f32(int M, const int32_t *pos,
                                       const float *val, float scale,
                                       float *out) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < M; ++i) {
    const int lo = pos[i], hi = pos[i + 1];
    if (lo == hi) continue;
    float mx = -FLT_MAX; /* finite: the file is built with -ffast-math */
    for (int p = lo; p < hi; ++p) {
      const float s = val[p] * scale;
      mx = s > mx ? s : mx;
    }
    float sum = 0.0f;
    for (int p = lo; p < hi; ++p) {
      const float e = expf(val[p] * scale - mx);
      out[p] = e;
      sum += e;
    }
    for (int p = lo; p < hi; ++p) out[p] = out[p] / sum;
  }
}

/* ------------------------------------------------------------------------
 * SpGEMM: C = A * B, all three CSR, for the four dtypes.
 * Restates spmspm_csr<T>, csrc/kernels.h:52-202 (bound as
 * prebuilt_spmspm_csr_{f32,f64,i32,i64}, csrc/ops.cpp:41-50,99, and
 * spmspm_csr_float, :113):
 *   phase 1 (73-104)  per row, the number of distinct columns reached through
 *                     A's entries, with a per-thread "next" array used as a
 *                     linked list of touched columns;
 *   phase 2 (107-113) prefix sum -> row pointer;
 *   phase 3 (119-186) per row, sums[k] += a * b in traversal order, then the
 *                     touched columns are collected and sorted ascending.
 * Every structurally reachable column is stored, also when its sum is zero.
 * Two calls, like any two-phase SpGEMM: `oracle_spgemm_csr_count` fills
 * c_pos[M + 1]; the typed call fills c_crd / c_val, which the caller sized
 * from c_pos[M].
 * ---------------------------------------------------------------------- */
ORACLE_API void oracle_spgemm_csr_count(int M, int N, const int32_t *a_pos, const int32_t *a_crd,
                                        const int32_t *b_pos, const int32_t *b_crd, int32_t *c_pos) {
  c_pos[0] = 0;
#pragma omp parallel
  {
    int *next = (int *)malloc((size_t)(N > 0 ? N : 1) * sizeof(int));
    for (int k = 0; k < N; ++k) next[k] = -1;
#pragma omp for schedule(dynamic, 64)
    for (int i = 0; i < M; ++i) {
      int head = -2, length = 0;
      for (int p = a_pos[i]; p < a_pos[i + 1]; ++p) {
        const int j = a_crd[p];
        for (int q = b_pos[j]; q < b_pos[j + 1]; ++q) {
          const int k = b_crd[q];
          if (next[k] == -1) { next[k] = head; head = k; ++length; }
        }
      }
      c_pos[i + 1] = length;
      while (head >= 0) { const int t = head; head = next[head]; next[t] = -1; }
    }
    free(next);
  }
  for (int i = 0; i < M; ++i) c_pos[i + 1] += c_pos[i];
}

static int cmp_int32(const void *x, const void *y) {
  const int32_t a = *(const int32_t *)x, b = *(const int32_t *)y;
  return (a > b) - (a < b);
}

#define DEFINE_SPGEMM_TYPED(NAME, T, ACC)                                                          \
  ORACLE_API void NAME(int M, int N, const int32_t *a_pos, const int32_t *a_crd, const T *a_val,   \
                       const int32_t *b_pos, const int32_t *b_crd, const T *b_val,                 \
                       const int32_t *c_pos, int32_t *c_crd, T *c_val) {                           \
    _Pragma("omp parallel")                                                                        \
    {                                                                                              \
      int *next = (int *)malloc((size_t)(N > 0 ? N : 1) * sizeof(int));                            \
      ACC *sums = (ACC *)calloc((size_t)(N > 0 ? N : 1), sizeof(ACC));                             \
      for (int k = 0; k < N; ++k) next[k] = -1;                                                    \
      _Pragma("omp for schedule(dynamic, 64)")                                                     \
      for (int i = 0; i < M; ++i) {                                                                \
        int head = -2, length = 0;                                                                 \
        for (int p = a_pos[i]; p < a_pos[i + 1]; ++p) {                                            \
          const int j = a_crd[p];                                                                  \
          const ACC v = (ACC)a_val[p];                                                             \
          for (int q = b_pos[j]; q < b_pos[j + 1]; ++q) {                                          \
            const int k = b_crd[q];                                                                \
            sums[k] += v * (ACC)b_val[q];                                                          \
            if (next[k] == -1) { next[k] = head; head = k; ++length; }                             \
          }                                                                                        \
        }                                                                                          \
        int32_t *crd = c_crd + c_pos[i];                                                           \
        int n = 0;                                                                                 \
        while (head >= 0) { crd[n++] = head; const int t = head; head = next[head]; next[t] = -1; } \
        qsort(crd, (size_t)n, sizeof(int32_t), cmp_int32);                                         \
        for (int e = 0; e < n; ++e) { c_val[c_pos[i] + e] = (T)sums[crd[e]]; sums[crd[e]] = 0; }   \
        (void)length;                                                                              \
      }                                                                                            \
      free(next);                                                                                  \
      free(sums);                                                                                  \
    }                                                                                              \
  }

DEFINE_SPGEMM_TYPED(oracle_spgemm_csr_f32, float, float)
DEFINE_SPGEMM_TYPED(oracle_spgemm_csr_f64, double, double)
DEFINE_SPGEMM_TYPED(oracle_spgemm_csr_i32, int32_t, uint32_t)
DEFINE_SPGEMM_TYPED(oracle_spgemm_csr_i64, int64_t, uint64_t)
