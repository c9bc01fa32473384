// Row-split CSR x dense SpMM for matrices whose rows are all short, and the
// inspection pass that tells a caller whether a matrix is one.
//
// The merge-path kernels of spmm.hip bound the work of a wavefront whatever the
// row lengths, at the price of two searches of row_ptr per wavefront and a
// second launch that folds the carries of rows cut by chunk boundaries.  When
// no row is long, none of that is needed: here a row belongs to one team of
// lanes, which reads its two row pointers, walks its entries and stores the
// row of C.  One launch, no workspace, no carries; every row of C is written
// exactly once (empty rows as zeros), and the summation order is fixed, so
// results are bit-reproducible.
//
// Lanes.  LPR lanes cover one column tile of B (LPR * VEC columns); a wavefront
// holds G = 64 / LPR such lane groups.  `team` groups (a power of two, at most
// G) share one row: group `sub` of the team takes the row's entries sub,
// sub + team, ...; their partial sums are combined with shuffles in a fixed
// order.  The launcher picks `team` so that a row of mean length is covered by
// one or two batches of loads and a small matrix still starts thousands of
// wavefronts.  The column indices and values of the next batch are requested
// while the current batch's rows of B are in flight, so a batch costs one
// memory round trip, not two.
//
// The kernel is correct for rows of any length; a long row only makes it slow
// (one team walks it alone).  The callers that know the longest row (the
// inspection pass below reports it) choose between this kernel and the
// merge-path one.
#include "spmm.hpp"

namespace scorch {

constexpr int kRowsBatch = 8;  // B-row loads in flight per lane group

template <typename T, int VEC, int LPR>
__global__ __launch_bounds__(kBlockThreads) void spmm_rows_kernel(
    int M, int N, const int *__restrict__ row_ptr, const int *__restrict__ col_idx,
    const T *__restrict__ vals, const T *__restrict__ B, T *__restrict__ C,
    const T *__restrict__ bias, int relu, int team_shift, int n_tiles, int64_t blocks_per_tile,
    int64_t batch_nnz, int64_t batch_b, int64_t batch_c) {
  using A = typename Acc<T>::type;
  // grid.y > 1: several products over one pattern, each with its own values, B and C
  vals += blockIdx.y * batch_nnz;
  B += blockIdx.y * batch_b;
  C += blockIdx.y * batch_c;
  using VecT = Vec<T, VEC>;
  constexpr int G = kWaveSize / LPR;

  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  const int g = lane / LPR;
  const int t = lane % LPR;
  const int team = 1 << team_shift;
  const int rows_per_wave = G >> team_shift;
  const int member = g >> team_shift;     // which of the wavefront's rows
  const int sub = g & (team - 1);         // which share of that row
  const TileMap where = map_workgroup(blockIdx.x, n_tiles, blocks_per_tile);
  const int64_t row64 = (where.block * kWavesPerBlock + w) * rows_per_wave + member;
  const bool live = row64 < M;
  const int row = live ? (int)row64 : 0;
  const int col0 = (where.tile * LPR + t) * VEC;
  const bool active = col0 < N;

  int begin = 0, end = 0;
  if (live) {
    begin = row_ptr[row];
    end = row_ptr[row + 1];
  }

  A acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = (A)0;

  // batch of kRowsBatch entries of this group's share: k, k + team, ...
  int c[kRowsBatch];
  T a[kRowsBatch];
  auto load_entries = [&](int k) {
#pragma unroll
    for (int u = 0; u < kRowsBatch; ++u) {
      const int p = k + (u << team_shift);
      const bool ok = p < end;
      c[u] = ok ? col_idx[p] : -1;
      a[u] = ok ? vals[p] : (T)0;
    }
  };

  int k = begin + sub;
  if (k < end) load_entries(k);
  while (k < end) {
    VecT b[kRowsBatch];
    A av[kRowsBatch];
#pragma unroll
    for (int u = 0; u < kRowsBatch; ++u) {
      av[u] = (A)a[u];
      if (c[u] >= 0 && active) {
        b[u] = *reinterpret_cast<const VecT *>(B + (size_t)c[u] * (size_t)N + col0);
      } else {
#pragma unroll
        for (int v = 0; v < VEC; ++v) b[u].v[v] = (T)0;
      }
    }
    k += kRowsBatch << team_shift;
    if (k < end) load_entries(k);  // in flight together with the rows of B above
#pragma unroll
    for (int u = 0; u < kRowsBatch; ++u)
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] += av[u] * (A)b[u].v[v];
  }

  // combine the team's shares: groups sub ^ 1, sub ^ 2, ... in a fixed order
  for (int off = LPR; off < (LPR << team_shift); off <<= 1)
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] += (A)__shfl_xor((T)acc[v], off);

  if (live && active && sub == 0) {
    VecT o;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      T r = (T)acc[v];
      if (bias) r = r + bias[col0 + v];
      if (relu) r = r > (T)0 ? r : (T)0;
      o.v[v] = r;
    }
    store_streaming(C + (size_t)row * (size_t)N + col0, o);
  }
}

template <typename T, int VEC, int LPR>
int launch_spmm_rows(int M, int N, int64_t nnz, const int *row_ptr, const int *col_idx, const T *vals,
                     const T *B, const T *bias, int relu, T *C, hipStream_t stream, int batch, int64_t K) {
  constexpr int G = kWaveSize / LPR;
  const int tile = LPR * VEC;
  const int n_tiles = (N + tile - 1) / tile;
  // Groups per row: enough that a row of mean length is one batch of loads per group, and more
  // while that leaves fewer than 8192 wavefronts (256 CUs x 32) for a small matrix.
  const int64_t mean = (nnz + M - 1) / M;
  int team_shift = 0;
  while ((1 << team_shift) < G && (int64_t)(kRowsBatch << team_shift) < mean) ++team_shift;
  while ((1 << team_shift) < G && mean > (2 << team_shift) &&
         ((int64_t)M * n_tiles << team_shift) / G < 8192)
    ++team_shift;
  const int rows_per_wave = G >> team_shift;
  const int64_t waves = ((int64_t)M + rows_per_wave - 1) / rows_per_wave;
  const int64_t blocks_per_tile = round_up_8((waves + kWavesPerBlock - 1) / kWavesPerBlock);
  if (blocks_per_tile * n_tiles > INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED, "SpMM (row split): %lld workgroups exceed the launch limit",
                (long long)(blocks_per_tile * n_tiles));
  mark_launch(stream);
  spmm_rows_kernel<T, VEC, LPR><<<dim3((unsigned)(blocks_per_tile * n_tiles), (unsigned)batch), kBlockThreads, 0,
                                 stream>>>(M, N, row_ptr, col_idx, vals, B, C, bias, relu, team_shift, n_tiles,
                                           blocks_per_tile, nnz, K * N, (int64_t)M * N);
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(stream);
  return SCORCH_HIP_OK;
}

template <typename T>
int spmm_rows_entry(const char *fn, int64_t M, int64_t K, int64_t N, int64_t nnz, const int32_t *row_ptr,
                    const int32_t *col_idx, const T *vals, const T *B, const T *bias, int act, T *C,
                    void *stream, int64_t batch = 1) {
  if (batch < 0 || batch > 65535)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: batch=%lld is outside [0, 65535]", fn, (long long)batch);
  if (batch == 0) return SCORCH_HIP_OK;
  if (int rc = check_csr_args(fn, M, K, nnz, row_ptr, col_idx, vals)) return rc;
  SCORCH_REQUIRE(N >= 0, "%s: negative N=%lld", fn, (long long)N);
  if (N > INT32_MAX - kWaveSize * 4)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: N=%lld is too large", fn, (long long)N);
  SCORCH_REQUIRE(act == SCORCH_HIP_ACT_NONE || act == SCORCH_HIP_ACT_RELU, "%s: unknown activation %d", fn, act);
  SCORCH_REQUIRE(act == SCORCH_HIP_ACT_NONE || bias != nullptr, "%s: an activation needs a bias", fn);
  if (M == 0 || N == 0) return SCORCH_HIP_OK;  // nothing to write
  SCORCH_REQUIRE(C != nullptr, "%s: C is NULL", fn);
  SCORCH_REQUIRE(K == 0 || B != nullptr, "%s: B is NULL", fn);
  SCORCH_REQUIRE(aligned_to(B, sizeof(T)) && aligned_to(C, sizeof(T)) && aligned_to(vals, sizeof(T)) &&
                     aligned_to(bias, sizeof(T)),
                 "%s: value arrays must be aligned to their element size", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int m = (int)M, n = (int)N;
  const int relu = act == SCORCH_HIP_ACT_RELU;

  // widest vector (at most 16 bytes) that divides N and is aligned
  constexpr int kMaxVec = (int)(16 / sizeof(T));
  int vec = kMaxVec;
  while (vec > 1 && !(N % vec == 0 && aligned_to(B, sizeof(T) * vec) && aligned_to(C, sizeof(T) * vec)))
    vec /= 2;
  // lanes that cover a row of B (at most a wavefront: wider rows take several column tiles)
  const int64_t lanes = (N + vec - 1) / vec;
#define SCORCH_ROWS(VEC, LPR) \
  return launch_spmm_rows<T, VEC, LPR>(m, n, nnz, row_ptr, col_idx, vals, B, bias, relu, C, s, (int)batch, K)
#define SCORCH_ROWS_LANES(VEC)              \
  do {                                      \
    if (lanes <= 8) SCORCH_ROWS(VEC, 8);    \
    if (lanes <= 16) SCORCH_ROWS(VEC, 16);  \
    if (lanes <= 32) SCORCH_ROWS(VEC, 32);  \
    SCORCH_ROWS(VEC, 64);                   \
  } while (0)
  if constexpr (sizeof(T) == 4) {
    if (vec == 4) SCORCH_ROWS_LANES(4);
  }
  if (vec == 2) SCORCH_ROWS_LANES(2);
  SCORCH_ROWS_LANES(1);
#undef SCORCH_ROWS_LANES
#undef SCORCH_ROWS
}

// ---- inspection of a CSR index ------------------------------------------------------------
// report[0]  1 if row_ptr is malformed: row_ptr[0] != 0, row_ptr[M] != nnz, or a
//            row pointer below its predecessor
// report[1]  1 if a column index lies outside [0, K)
// report[2]  the longest row
// report[3]  the number of empty rows
// report[4]  the number of entries that do not exceed the entry before them in the same row
//            (0: every row's columns increase strictly)
// report[5]  the number of runs: maximal stretches of a row's entries that lie in one aligned
//            group of 64 columns and increase.  nnz / (64 runs) bounds from above the share of
//            stored positions in the 64 x 64 blocks the pattern touches (a block's row holds one
//            run at least when it holds anything), so a graph is told from a mask made of blocks
//            without looking at blocks
// report[6], report[7]  0 (reserved)
// Only row_ptr[0 .. M] and col_idx[0 .. nnz) are read, whatever they contain; [4] and [5] mean
// what they say only when [0] is 0.
constexpr int kInspectReportInts = 8;

__global__ void csr_inspect_clear_kernel(int *__restrict__ report) {
  if (threadIdx.x < kInspectReportInts) report[threadIdx.x] = 0;
}

__global__ __launch_bounds__(kBlockThreads) void csr_inspect_kernel(int M, int K, int64_t nnz,
                                                                    const int *__restrict__ row_ptr,
                                                                    const int *__restrict__ col_idx,
                                                                    int *__restrict__ report) {
  const int64_t stride = (int64_t)gridDim.x * kBlockThreads;
  const int64_t first = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  int bad_rows = 0, bad_cols = 0, longest = 0, empty = 0;
  // The entry loop below does not know where rows begin: it counts an entry as a descent when it
  // does not exceed its predecessor, and as the head of a run when it is a descent or lies in
  // another group of 64 columns than its predecessor.  Every row's first entry is the head of a
  // run and never a descent, whatever its predecessor: the row loop corrects both counts.
  int descents = 0, runs = 0;
  if (first == 0) {
    if (row_ptr[0] != 0 || (int64_t)row_ptr[M] != nnz) bad_rows = 1;
    if (nnz > 0) runs = 1;  // entry 0
  }
  for (int64_t i = first; i < M; i += stride) {
    const int begin = row_ptr[i], len = row_ptr[i + 1] - begin;
    bad_rows |= len < 0;
    longest = len > longest ? len : longest;
    empty += len == 0;
    if (len > 0 && begin > 0 && (int64_t)begin < nnz) {
      const int before = col_idx[begin - 1], here = col_idx[begin];
      const bool descent = here <= before;
      const bool head = descent || ((unsigned)here >> 6) != ((unsigned)before >> 6);
      descents -= descent;
      runs += !head;
    }
  }
  {
    // four column indices per thread in flight, each with its predecessor (the same cache line
    // another lane reads, except for the wavefront's first lane)
    auto look = [&](int64_t p) {
      const int here = col_idx[p];
      bad_cols |= (unsigned)here >= (unsigned)K;
      if (p > 0) {
        const int before = col_idx[p - 1];
        const bool descent = here <= before;
        descents += descent;
        runs += descent || ((unsigned)here >> 6) != ((unsigned)before >> 6);
      }
    };
    int64_t p = first;
    for (; p + 3 * stride < nnz; p += 4 * stride) {
      look(p);
      look(p + stride);
      look(p + 2 * stride);
      look(p + 3 * stride);
    }
    for (; p < nnz; p += stride) look(p);
  }
  // one atomic of each kind per workgroup that has something to say
#pragma unroll
  for (int off = kWaveSize / 2; off > 0; off >>= 1) {
    const int other = __shfl_xor(longest, off);
    longest = other > longest ? other : longest;
    empty += __shfl_xor(empty, off);
    descents += __shfl_xor(descents, off);
    runs += __shfl_xor(runs, off);
  }
  __shared__ int s_bad_rows, s_bad_cols, s_longest[kWavesPerBlock], s_empty[kWavesPerBlock];
  __shared__ int s_descents[kWavesPerBlock], s_runs[kWavesPerBlock];
  if (threadIdx.x == 0) s_bad_rows = s_bad_cols = 0;
  __syncthreads();
  const bool any_bad_rows = __any(bad_rows), any_bad_cols = __any(bad_cols);
  if (wave_lane() == 0) {
    if (any_bad_rows) s_bad_rows = 1;
    if (any_bad_cols) s_bad_cols = 1;
    s_longest[threadIdx.x / kWaveSize] = longest;
    s_empty[threadIdx.x / kWaveSize] = empty;
    s_descents[threadIdx.x / kWaveSize] = descents;
    s_runs[threadIdx.x / kWaveSize] = runs;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    longest = empty = descents = runs = 0;
    for (int w = 0; w < kWavesPerBlock; ++w) {
      longest = s_longest[w] > longest ? s_longest[w] : longest;
      empty += s_empty[w];
      descents += s_descents[w];
      runs += s_runs[w];
    }
    if (s_bad_rows) atomicOr(&report[0], 1);
    if (s_bad_cols) atomicOr(&report[1], 1);
    if (longest > 0) atomicMax(&report[2], longest);
    if (empty > 0) atomicAdd(&report[3], empty);  // at most M < 2^31 in all
    // partial sums may be negative (the row loop's corrections); the totals lie in [0, nnz]
    if (descents != 0) atomicAdd(&report[4], descents);
    if (runs != 0) atomicAdd(&report[5], runs);
  }
}

}  // namespace scorch

extern "C" {

#define SCORCH_DEFINE_SPMM_ROWS(SUFFIX, T)                                                              \
  int scorch_hip_spmm_csr_rows_##SUFFIX(int64_t M, int64_t K, int64_t N, int64_t nnz,                    \
                                        const int32_t *row_ptr, const int32_t *col_idx, const T *vals,   \
                                        const T *B, const T *bias, int act, T *C, void *stream) {        \
    return scorch::spmm_rows_entry<T>("scorch_hip_spmm_csr_rows_" #SUFFIX, M, K, N, nnz, row_ptr,        \
                                      col_idx, vals, B, bias, act, C, stream);                           \
  }

int scorch_hip_spmm_csr_rows_batched_f32(int64_t batch, int64_t M, int64_t K, int64_t N, int64_t nnz,
                                         const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                                         const float *B, float *C, void *stream) {
  return scorch::spmm_rows_entry<float>("scorch_hip_spmm_csr_rows_batched_f32", M, K, N, nnz, row_ptr, col_idx,
                                        vals, B, nullptr, SCORCH_HIP_ACT_NONE, C, stream, batch);
}

SCORCH_DEFINE_SPMM_ROWS(f32, float)
SCORCH_DEFINE_SPMM_ROWS(f64, double)
SCORCH_DEFINE_SPMM_ROWS(i32, int32_t)
SCORCH_DEFINE_SPMM_ROWS(i64, int64_t)

int scorch_hip_csr_inspect(int64_t M, int64_t K, int64_t nnz, const int32_t *row_ptr,
                           const int32_t *col_idx, int32_t *report, void *stream) {
  const char *fn = "scorch_hip_csr_inspect";
  if (M < 0 || K < 0 || nnz < 0)
    return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size (M=%lld K=%lld nnz=%lld)", fn, (long long)M,
                        (long long)K, (long long)nnz);
  if (M >= INT32_MAX || K > INT32_MAX || nnz > INT32_MAX)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: M, K and nnz must fit the int32 index arrays", fn);
  SCORCH_REQUIRE(row_ptr != nullptr && report != nullptr, "%s: row_ptr or report is NULL", fn);
  SCORCH_REQUIRE(nnz == 0 || col_idx != nullptr, "%s: col_idx is NULL with nnz=%lld", fn, (long long)nnz);
  SCORCH_REQUIRE(scorch::aligned_to(row_ptr, 4) && scorch::aligned_to(col_idx, 4) &&
                     scorch::aligned_to(report, 4),
                 "%s: arrays must be 4-byte aligned", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  scorch::csr_inspect_clear_kernel<<<1, 64, 0, s>>>(report);
  SCORCH_HIP_CHECK(hipGetLastError());
  const int64_t work = (M > nnz ? M : nnz) + 1;
  int64_t blocks = (work + scorch::kBlockThreads - 1) / scorch::kBlockThreads;
  if (blocks > 2048) blocks = 2048;
  scorch::csr_inspect_kernel<<<dim3((unsigned)blocks), scorch::kBlockThreads, 0, s>>>((int)M, (int)K, nnz, row_ptr,
                                                                                    col_idx, report);
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

}  // extern "C"

SCORCH_DEFINE_PRELOAD(spmm_rows)
