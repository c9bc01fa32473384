// SDDMM for gfx950: out[p] = mask[p] * <A[row_p, :], B[col_p, :]>.
//
// A wavefront owns kEntriesPerWave consecutive mask entries and handles them
// 64 at a time.  For each batch of 64, lane L first fetches the coordinates and
// mask value of entry L (coalesced).  The wavefront is then split into 64/GS
// groups of GS lanes; in step s, group g computes the dot product of entry
// g * GS + s: its GS lanes read the two K-vectors with one vector load each
// (GS * VEC elements per load, so a K = 64 fp32 row is one dwordx4 access by
// 16 lanes), multiply, and reduce with GS-wide butterfly shuffles.  After GS
// steps lane L keeps the result of entry L and the batch is written with one
// coalesced store.  Consecutive entries mostly share their A row, which a group
// keeps in registers until the row changes (K up to GS * VEC).
//
// With a CSR mask the row of each entry is found by bisection of row_ptr; the
// wavefront first narrows the range to the rows its entries span, so the
// per-lane search is a few steps.  The same pass can write the row of every
// entry (the coordinate array of the result).
#include "common.hpp"

namespace scorch {

constexpr int kEntriesPerWave = 256;

// LONG: K exceeds what the group's lanes cover with one load each (GS * VEC
// elements); the vectors are then read four such pieces at a time, all eight
// loads requested before the first product.
template <int GS, int VEC, bool COO, bool LONG>
__global__ __launch_bounds__(kBlockThreads) void sddmm_kernel(
    int M, int K, int64_t nnz, const int *__restrict__ rows /* row_idx (COO) or row_ptr (CSR) */,
    const int *__restrict__ col_idx, const float *__restrict__ mask_vals,
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ out_vals,
    int *__restrict__ out_row_idx, int64_t batch_stride_a, int64_t batch_stride_b) {
  using VecT = Vec<float, VEC>;
  const int lane = wave_lane();
  // grid.y > 1: several products over one mask (one per attention head); problem h has its own A,
  // B and result values, the mask's values are shared and the row coordinates are written once
  if (blockIdx.y > 0) {
    A += blockIdx.y * batch_stride_a;
    B += blockIdx.y * batch_stride_b;
    out_vals += blockIdx.y * nnz;
    out_row_idx = nullptr;
  }
  // the grid is a multiple of 8 workgroups; every XCD takes a contiguous eighth of the entries
  const int64_t wave = xcd_contiguous(blockIdx.x, gridDim.x) * kWavesPerBlock + threadIdx.x / kWaveSize;
  const int64_t first = wave * kEntriesPerWave;
  if (first >= nnz) return;
  const int64_t last = first + kEntriesPerWave < nnz ? first + kEntriesPerWave : nnz;

  // Rows spanned by this wavefront's entries: row(p) = #{i : row_ptr[i+1] <= p}.
  int row_lo = 0, row_hi = 0;
  if (!COO) {
    auto end_key = [&](int i) { return (int64_t)rows[i + 1]; };
    row_lo = wave_count_below(M, first + 1, end_key);
    row_hi = wave_count_below(M, last, end_key);  // row of entry last - 1
  }

  const int t = lane % GS;  // position inside the group
  const int g = lane / GS;  // group

  for (int64_t base = first; base < last; base += kWaveSize) {
    const int64_t p = base + lane;
    const bool valid = p < last;
    int row = 0, col = 0;
    float scale = 0.0f;
    if (valid) {
      col = col_idx[p];
      scale = mask_vals ? mask_vals[p] : 1.0f;  // (no value array: every stored entry is 1)
      if (COO) {
        row = rows[p];
      } else {
        int lo = row_lo, hi = row_hi;  // answer in [lo, hi]
        while (lo < hi) {
          const int mid = (lo + hi) >> 1;
          if ((int64_t)rows[mid + 1] <= p) lo = mid + 1; else hi = mid;
        }
        row = lo;
      }
    }

    float mine = 0.0f;
    // !LONG: a group's piece of its current row of A stays in registers; a group's 16 or more
    // consecutive entries mostly share a row, and a mask of long rows (an attention pattern)
    // would otherwise ask the vector cache for the same line once per entry
    int held_row = -1;
    VecT held;
#pragma unroll 4
    for (int s = 0; s < GS; ++s) {
      const int src = g * GS + s;
      const int r = __shfl(row, src);
      const int c = __shfl(col, src);
      const float *a = A + (size_t)r * (size_t)K;
      const float *b = B + (size_t)c * (size_t)K;
      float dot = 0.0f;
      if (!LONG) {
        const int k = t * VEC;
        if (k < K) {
          const VecT bv = *reinterpret_cast<const VecT *>(b + k);
          if (r != held_row) {
            held = *reinterpret_cast<const VecT *>(a + k);
            held_row = r;
          }
#pragma unroll
          for (int v = 0; v < VEC; ++v) dot += held.v[v] * bv.v[v];
        }
      } else {
        constexpr int kPieces = 4;
        for (int k0 = t * VEC; k0 < K; k0 += kPieces * GS * VEC) {
          VecT av[kPieces], bv[kPieces];
#pragma unroll
          for (int u = 0; u < kPieces; ++u) {
            const int k = k0 + u * GS * VEC;
            if (k < K) {
              av[u] = *reinterpret_cast<const VecT *>(a + k);
              bv[u] = *reinterpret_cast<const VecT *>(b + k);
            } else {
#pragma unroll
              for (int v = 0; v < VEC; ++v) av[u].v[v] = bv[u].v[v] = 0.0f;
            }
          }
#pragma unroll
          for (int u = 0; u < kPieces; ++u)
#pragma unroll
            for (int v = 0; v < VEC; ++v) dot += av[u].v[v] * bv[u].v[v];
        }
      }
      dot = group_sum<GS>(dot);
      if (t == s) mine = dot;
    }

    if (valid) {
      out_vals[p] = scale * mine;
      if (!COO && out_row_idx) out_row_idx[p] = row;
    }
  }
}

// ---- a mask that is used again and again: its entries listed per XCD ------------------------
// With B larger than one L2 (4 MB per XCD) most of the gathered B rows come over
// the fabric, although all of B would fit the eight L2s together.  For a mask
// whose pattern stays (an attention mask serves every head, layer and step) the
// entries are therefore listed once by the column range they fall in, one range
// per XCD: XCD x then only ever gathers rows of B from its eighth of B, which
// stays in its L2, at the price of every XCD streaming all of A once.
//
// sddmm_bucket_count_kernel / sddmm_bucket_fill_kernel build the lists: each
// wavefront takes kEntriesPerWave consecutive entries (so that a row's entries
// stay together in the lists and its row of A is reused from the vector cache),
// counts them per range (sddmm_bucket_count_kernel), a scan over the wavefronts'
// counts gives every wavefront its place in every list (sddmm_bucket_scan_kernel),
// and the wavefront writes (entry number, row, column) there
// (sddmm_bucket_fill_kernel).  No atomics: the lists come out in entry order, the
// same on every build.
constexpr int kBuckets = 8;  // one per XCD
// Workgroups per XCD of the kernel that walks the lists: a grid that is resident as a whole,
// workgroup id & 7 being the XCD it runs on (checked against the hardware's XCC_ID register: no
// workgroup of 102,400 was elsewhere, also with 256 per XCD).  65,536^2 mask, 64 per row, K = 64:
// 64 per XCD 0.222 ms, 128 0.136, 192 0.105, 256 0.098 (fewer wavefronts hide less latency); more
// than the 256 a XCD holds change nothing.
constexpr int kListedWorkgroupsPerXcd = 256;

__device__ __forceinline__ int sddmm_entry_row(const int *__restrict__ row_ptr, int row_lo, int row_hi, int64_t p) {
  int lo = row_lo, hi = row_hi;  // answer in [lo, hi]
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)row_ptr[mid + 1] <= p) lo = mid + 1; else hi = mid;
  }
  return lo;
}

// wave_counts[wave][b] = entries of the wavefront's piece whose column lies in range b; columns
// outside [0, n_cols) count for no range
__global__ __launch_bounds__(kBlockThreads) void sddmm_bucket_count_kernel(int64_t nnz, int cols_per_bucket,
                                                                           const int *__restrict__ col_idx,
                                                                           int *__restrict__ wave_counts) {
  const int lane = wave_lane();
  const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWaveSize;
  const int64_t first = wave * kEntriesPerWave;
  if (first >= nnz) return;
  const int64_t last = first + kEntriesPerWave < nnz ? first + kEntriesPerWave : nnz;
  int mine[kBuckets] = {0};
  for (int64_t p = first + lane; p < last; p += kWaveSize) {
    const unsigned b = (unsigned)col_idx[p] / (unsigned)cols_per_bucket;
#pragma unroll
    for (int k = 0; k < kBuckets; ++k) mine[k] += b == (unsigned)k;
  }
  int total = 0;  // lane k < kBuckets ends up with range k's count
#pragma unroll
  for (int k = 0; k < kBuckets; ++k) {
    int sum = mine[k];
#pragma unroll
    for (int off = kWaveSize / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == k) total = sum;
  }
  if (lane < kBuckets) wave_counts[wave * kBuckets + lane] = total;
}

// One workgroup: wave_counts[wave][b] becomes the number of range-b entries in the pieces before
// `wave`, and list_ptr[b] the start of range b's list (list_ptr[kBuckets] = entries listed).
constexpr int kScanThreads = 1024;

__global__ __launch_bounds__(kScanThreads) void sddmm_bucket_scan_kernel(int64_t n_waves, int *__restrict__ wave_counts,
                                                                        int *__restrict__ list_ptr) {
  constexpr int kScanWaves = kScanThreads / kWaveSize;
  __shared__ int s_wave_total[kBuckets][kScanWaves];
  __shared__ int s_running[kBuckets];
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  if (threadIdx.x < kBuckets) s_running[threadIdx.x] = 0;
  __syncthreads();
  for (int64_t base = 0; base < n_waves; base += kScanThreads) {
    const int64_t i = base + threadIdx.x;
    int count[kBuckets], upto[kBuckets];
#pragma unroll
    for (int k = 0; k < kBuckets; ++k) {
      count[k] = i < n_waves ? wave_counts[i * kBuckets + k] : 0;
      int v = count[k];
#pragma unroll
      for (int off = 1; off < kWaveSize; off <<= 1) {
        const int from_below = __shfl_up(v, off);
        if (lane >= off) v += from_below;
      }
      upto[k] = v;
      if (lane == kWaveSize - 1) s_wave_total[k][w] = v;
    }
    __syncthreads();
    if (i < n_waves) {
#pragma unroll
      for (int k = 0; k < kBuckets; ++k) {
        int before = s_running[k];
        for (int j = 0; j < w; ++j) before += s_wave_total[k][j];
        wave_counts[i * kBuckets + k] = before + upto[k] - count[k];
      }
    }
    __syncthreads();
    if (threadIdx.x < kBuckets) {
      int total = 0;
      for (int j = 0; j < kScanWaves; ++j) total += s_wave_total[threadIdx.x][j];
      s_running[threadIdx.x] += total;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    int at = 0;
    for (int k = 0; k < kBuckets; ++k) {
      list_ptr[k] = at;
      at += s_running[k];
    }
    list_ptr[kBuckets] = at;
  }
}

// The entries of every piece go to their places in the lists: range b's part of piece `wave`
// starts at list_ptr[b] + wave_offsets[wave][b] (from the scan above).
__global__ __launch_bounds__(kBlockThreads) void sddmm_bucket_fill_kernel(
    int M, int64_t nnz, int cols_per_bucket, const int *__restrict__ row_ptr, const int *__restrict__ col_idx,
    const int *__restrict__ wave_offsets, const int *__restrict__ list_ptr, int *__restrict__ entry_pos,
    int *__restrict__ entry_row, int *__restrict__ entry_col) {
  const int lane = wave_lane();
  const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWaveSize;
  const int64_t first = wave * kEntriesPerWave;
  if (first >= nnz) return;
  const int64_t last = first + kEntriesPerWave < nnz ? first + kEntriesPerWave : nnz;
  auto end_key = [&](int i) { return (int64_t)row_ptr[i + 1]; };
  const int row_lo = wave_count_below(M, first + 1, end_key);
  const int row_hi = wave_count_below(M, last, end_key);

  constexpr int kRounds = kEntriesPerWave / kWaveSize;
  int col[kRounds], row[kRounds];
  unsigned bucket[kRounds];
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
    const int64_t p = first + r * kWaveSize + lane;
    bucket[r] = ~0u;
    col[r] = row[r] = 0;
    if (p < last) {
      col[r] = col_idx[p];
      row[r] = sddmm_entry_row(row_ptr, row_lo, row_hi, p);
      bucket[r] = (unsigned)col[r] / (unsigned)cols_per_bucket;
    }
  }
  // every entry's slot: the wavefront's entries keep their order inside a list, so that a row's
  // entries stay next to each other there (its row of A is then kept in registers, and the
  // entry's mask value and result lie next to its neighbours')
  int base[kBuckets];
#pragma unroll
  for (int k = 0; k < kBuckets; ++k) base[k] = list_ptr[k] + wave_offsets[wave * kBuckets + k];
  const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (kWaveSize - lane));
#pragma unroll
  for (int r = 0; r < kRounds; ++r) {
#pragma unroll
    for (int k = 0; k < kBuckets; ++k) {
      const unsigned long long members = __ballot(bucket[r] == (unsigned)k);
      if (bucket[r] == (unsigned)k) {
        const int at = base[k] + __popcll(members & below);
        entry_pos[at] = (int)(first + r * kWaveSize + lane);
        entry_row[at] = row[r];
        entry_col[at] = col[r];
      }
      base[k] += __popcll(members);
    }
  }
}

// The SDDMM proper over such lists.  Workgroup ids are dealt to the XCDs round robin, so
// workgroup id & 7 is the XCD and the range; the XCD's workgroups share out its list in
// pieces of kEntriesPerWave entries.  Everything else as in sddmm_kernel.
template <int GS, int VEC>
__global__ __launch_bounds__(kBlockThreads) void sddmm_listed_kernel(
    int K, const int *__restrict__ list_ptr, const int *__restrict__ entry_pos,
    const int *__restrict__ entry_row, const int *__restrict__ entry_col,
    const float *__restrict__ mask_vals, const float *__restrict__ listed_vals, const float *__restrict__ A,
    const float *__restrict__ B, float *__restrict__ out_vals, int *__restrict__ out_row_idx, int64_t nnz,
    int64_t batch_stride_a, int64_t batch_stride_b) {
  using VecT = Vec<float, VEC>;
  if (blockIdx.y > 0) {  // problem blockIdx.y of a batch over one mask
    A += blockIdx.y * batch_stride_a;
    B += blockIdx.y * batch_stride_b;
    out_vals += blockIdx.y * nnz;
    out_row_idx = nullptr;
  }
  const int lane = wave_lane();
  const int xcd = blockIdx.x & 7;
  const int64_t begin = list_ptr[xcd], end = list_ptr[xcd + 1];
  const int64_t waves_per_xcd = (int64_t)(gridDim.x >> 3) * kWavesPerBlock;
  const int t = lane % GS;
  const int g = lane / GS;
  for (int64_t first = begin + ((int64_t)(blockIdx.x >> 3) * kWavesPerBlock + threadIdx.x / kWaveSize) * kEntriesPerWave;
       first < end; first += waves_per_xcd * kEntriesPerWave) {
    const int64_t last = first + kEntriesPerWave < end ? first + kEntriesPerWave : end;
    // the piece's list entries and mask values are requested for all of its batches of 64 at
    // once: two round trips to memory per piece instead of two per batch
    constexpr int kBatches = kEntriesPerWave / kWaveSize;
    int rows_of[kBatches], cols_of[kBatches], pos_of[kBatches];
    float scale_of[kBatches];
#pragma unroll
    for (int b = 0; b < kBatches; ++b) {
      const int64_t e = first + b * kWaveSize + lane;
      const bool valid = e < last;
      pos_of[b] = valid ? entry_pos[e] : -1;
      rows_of[b] = valid ? entry_row[e] : 0;
      cols_of[b] = valid ? entry_col[e] : 0;
    }
#pragma unroll
    for (int b = 0; b < kBatches; ++b) {
      // the mask's values: in list order if the caller keeps such a copy (read with the entries,
      // coalesced), else from their places in the mask (one scattered load per entry); no value
      // array at all: every stored entry is 1
      const int64_t e = first + b * kWaveSize + lane;
      scale_of[b] = pos_of[b] < 0 ? 0.0f : listed_vals ? listed_vals[e] : mask_vals ? mask_vals[pos_of[b]] : 1.0f;
    }
#pragma unroll
    for (int b = 0; b < kBatches; ++b) {
      if (first + b * kWaveSize >= last) break;
      const int row = rows_of[b], col = cols_of[b], pos = pos_of[b];
      const float scale = scale_of[b];
      const bool valid = pos >= 0;
      float mine = 0.0f;
      if (K <= GS * VEC) {
        // One load per lane covers a row.  Consecutive entries of a list mostly share their row
        // of A (a row's entries of one column range lie together): the group keeps that row in
        // registers and reloads it only when the row changes.
        const int k = t * VEC;
        const bool in_row = k < K;
        VecT av;
#pragma unroll
        for (int v = 0; v < VEC; ++v) av.v[v] = 0.0f;
        int held = -1;
#pragma unroll 4
        for (int s = 0; s < GS; ++s) {
          const int src = g * GS + s;
          const int r = __shfl(row, src);
          const int c = __shfl(col, src);
          if (r != held && in_row) av = *reinterpret_cast<const VecT *>(A + (size_t)r * (size_t)K + k);
          held = r;
          float dot = 0.0f;
          if (in_row) {
            const VecT bv = *reinterpret_cast<const VecT *>(B + (size_t)c * (size_t)K + k);
#pragma unroll
            for (int v = 0; v < VEC; ++v) dot += av.v[v] * bv.v[v];
          }
          dot = group_sum<GS>(dot);
          if (t == s) mine = dot;
        }
      } else {
#pragma unroll 4
        for (int s = 0; s < GS; ++s) {
          const int src = g * GS + s;
          const int r = __shfl(row, src);
          const int c = __shfl(col, src);
          const float *a = A + (size_t)r * (size_t)K;
          const float *b = B + (size_t)c * (size_t)K;
          float dot = 0.0f;
          for (int k = t * VEC; k < K; k += GS * VEC) {
            const VecT av = *reinterpret_cast<const VecT *>(a + k);
            const VecT bv = *reinterpret_cast<const VecT *>(b + k);
#pragma unroll
            for (int v = 0; v < VEC; ++v) dot += av.v[v] * bv.v[v];
          }
          dot = group_sum<GS>(dot);
          if (t == s) mine = dot;
        }
      }
      if (valid) {
        // The results are scattered 4-byte writes that nothing reads again: marked as streaming
        // they do not take L2 lines from the XCD's part of B (8 % faster at 65,536^2; the same
        // mark on the loads of the lists or of A made the kernel slower).
        store_streaming(out_vals + pos, scale * mine);
        if (out_row_idx) store_streaming(out_row_idx + pos, row);
      }
    }
  }
}

template <bool COO>
int launch_sddmm(int M, int K, int64_t nnz, const int *rows, const int *col_idx,
                 const float *mask_vals, const float *A, const float *B, float *out_vals,
                 int *out_row_idx, hipStream_t stream, int batch = 1, int64_t batch_stride_a = 0,
                 int64_t batch_stride_b = 0) {
  const int64_t waves = (nnz + kEntriesPerWave - 1) / kEntriesPerWave;
  const dim3 grid((unsigned)round_up_8((waves + kWavesPerBlock - 1) / kWavesPerBlock), (unsigned)batch);
  const bool vec4 = K % 4 == 0 && aligned_to(A, 16) && aligned_to(B, 16);
  const int per_lane = vec4 ? 4 : 1;
  const int64_t lanes_needed = (K + per_lane - 1) / per_lane;

  mark_launch(stream);
#define SCORCH_SDDMM_LAUNCH(GS, VEC, LONG)                                                         \
  sddmm_kernel<GS, VEC, COO, LONG><<<grid, kBlockThreads, 0, stream>>>(M, K, nnz, rows, col_idx,   \
                                                                      mask_vals, A, B, out_vals,  \
                                                                      out_row_idx, batch_stride_a,  \
                                                                      batch_stride_b)
#define SCORCH_SDDMM_PICK(VEC)                                              \
  do {                                                                      \
    if (lanes_needed <= 4) SCORCH_SDDMM_LAUNCH(4, VEC, false);              \
    else if (lanes_needed <= 8) SCORCH_SDDMM_LAUNCH(8, VEC, false);         \
    else if (lanes_needed <= 16) SCORCH_SDDMM_LAUNCH(16, VEC, false);       \
    else if (lanes_needed <= 32) SCORCH_SDDMM_LAUNCH(32, VEC, false);       \
    else if (lanes_needed <= 64) SCORCH_SDDMM_LAUNCH(64, VEC, false);       \
    else SCORCH_SDDMM_LAUNCH(64, VEC, true);                                \
  } while (0)

  if (vec4) SCORCH_SDDMM_PICK(4); else SCORCH_SDDMM_PICK(1);
#undef SCORCH_SDDMM_PICK
#undef SCORCH_SDDMM_LAUNCH
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(stream);
  return SCORCH_HIP_OK;
}

template <bool COO>
int sddmm_entry(const char *fn, int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                const int32_t *rows, const int32_t *col_idx, const float *mask_vals,
                const float *A, const float *B, float *out_vals, int32_t *out_row_idx,
                void *stream, int64_t batch = 1) {
  if (batch < 0 || batch > 65535)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: batch=%lld is outside [0, 65535]", fn, (long long)batch);
  if (batch == 0) return SCORCH_HIP_OK;
  if (M < 0 || n_cols < 0 || K < 0 || nnz < 0)
    return fail(SCORCH_HIP_EINVAL, "%s: negative size (M=%lld n_cols=%lld K=%lld nnz=%lld)", fn,
                (long long)M, (long long)n_cols, (long long)K, (long long)nnz);
  if (M >= INT32_MAX || n_cols > INT32_MAX || K > INT32_MAX || nnz > INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  SCORCH_REQUIRE(COO || rows != nullptr, "%s: row_ptr is NULL", fn);
  if (nnz == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(M > 0 && n_cols > 0, "%s: nnz=%lld in an empty mask", fn, (long long)nnz);
  SCORCH_REQUIRE(rows && col_idx && out_vals, "%s: NULL index/value array", fn);
  SCORCH_REQUIRE(K == 0 || (A && B), "%s: NULL dense operand", fn);
  SCORCH_REQUIRE(aligned_to(rows, 4) && aligned_to(col_idx, 4) && aligned_to(mask_vals, 4) &&
                     aligned_to(out_vals, 4) && aligned_to(A, 4) && aligned_to(B, 4) &&
                     aligned_to(out_row_idx, 4),
                 "%s: arrays must be 4-byte aligned", fn);
  return launch_sddmm<COO>((int)M, (int)K, nnz, rows, col_idx, mask_vals, A, B, out_vals,
                           out_row_idx, static_cast<hipStream_t>(stream), (int)batch, M * K, n_cols * K);
}

inline size_t align_up_256(size_t v) { return (v + 255) / 256 * 256; }

// Layout of the per-XCD entry lists inside the caller's buffer.
struct SddmmLists {
  int *list_ptr;   // [9]
  int *entry_pos, *entry_row, *entry_col;  // [nnz] each
  int *wave_offsets;  // [pieces][kBuckets]: used while the lists are built
};

inline int64_t sddmm_pieces(int64_t nnz) { return (nnz + kEntriesPerWave - 1) / kEntriesPerWave; }

inline SddmmLists sddmm_lists(void *buffer, int64_t nnz) {
  char *base = static_cast<char *>(buffer);
  const size_t array = align_up_256((size_t)nnz * sizeof(int32_t));
  SddmmLists l;
  l.list_ptr = reinterpret_cast<int *>(base) + 16;
  l.entry_pos = reinterpret_cast<int *>(base + 256);
  l.entry_row = reinterpret_cast<int *>(base + 256 + array);
  l.entry_col = reinterpret_cast<int *>(base + 256 + 2 * array);
  l.wave_offsets = reinterpret_cast<int *>(base + 256 + 3 * array);
  return l;
}

// listed_vals[e] = vals[entry_pos[e]]: the mask's values in the order of the lists.
__global__ __launch_bounds__(kBlockThreads) void sddmm_list_values_kernel(int64_t nnz, const int *__restrict__ entry_pos,
                                                                           const float *__restrict__ vals,
                                                                           float *__restrict__ listed_vals) {
  const int64_t stride = (int64_t)gridDim.x * kBlockThreads;
  for (int64_t e = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x; e < nnz; e += stride)
    listed_vals[e] = vals[entry_pos[e]];
}

__global__ void sddmm_lists_clear_kernel(int *list_ptr) {
  if (threadIdx.x <= kBuckets) list_ptr[threadIdx.x] = 0;
}

}  // namespace scorch

extern "C" {

int scorch_hip_sddmm_coo_f32(int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                             const int32_t *row_idx, const int32_t *col_idx,
                             const float *mask_vals, const float *A, const float *B,
                             float *out_vals, void *stream) {
  return scorch::sddmm_entry<true>("scorch_hip_sddmm_coo_f32", M, n_cols, K, nnz, row_idx, col_idx,
                                   mask_vals, A, B, out_vals, nullptr, stream);
}

int scorch_hip_sddmm_csr_f32(int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                             const int32_t *row_ptr, const int32_t *col_idx,
                             const float *mask_vals, const float *A, const float *B,
                             float *out_vals, int32_t *out_row_idx, void *stream) {
  return scorch::sddmm_entry<false>("scorch_hip_sddmm_csr_f32", M, n_cols, K, nnz, row_ptr,
                                    col_idx, mask_vals, A, B, out_vals, out_row_idx, stream);
}

int scorch_hip_sddmm_csr_batched_f32(int64_t batch, int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                                     const int32_t *row_ptr, const int32_t *col_idx, const float *mask_vals,
                                     const float *A, const float *B, float *out_vals, int32_t *out_row_idx,
                                     void *stream) {
  return scorch::sddmm_entry<false>("scorch_hip_sddmm_csr_batched_f32", M, n_cols, K, nnz, row_ptr, col_idx,
                                    mask_vals, A, B, out_vals, out_row_idx, stream, batch);
}

size_t scorch_hip_sddmm_csr_lists_bytes(int64_t nnz) {
  if (nnz < 0) return 0;
  // the 9 list starts (256 bytes), entry numbers, rows and columns, and the per-piece offsets the
  // build works with
  return 256 + 3 * scorch::align_up_256((size_t)nnz * sizeof(int32_t)) +
         scorch::align_up_256((size_t)scorch::sddmm_pieces(nnz) * scorch::kBuckets * sizeof(int32_t));
}

int scorch_hip_sddmm_csr_lists(int64_t M, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                               const int32_t *col_idx, void *lists, size_t lists_bytes, void *stream) {
  const char *fn = "scorch_hip_sddmm_csr_lists";
  if (M < 0 || n_cols < 0 || nnz < 0)
    return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size (M=%lld n_cols=%lld nnz=%lld)", fn, (long long)M,
                        (long long)n_cols, (long long)nnz);
  if (M >= INT32_MAX || n_cols > INT32_MAX || nnz > INT32_MAX)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  SCORCH_REQUIRE(row_ptr != nullptr && lists != nullptr, "%s: row_ptr or lists is NULL", fn);
  SCORCH_REQUIRE(nnz == 0 || col_idx != nullptr, "%s: col_idx is NULL", fn);
  SCORCH_REQUIRE(scorch::aligned_to(row_ptr, 4) && scorch::aligned_to(col_idx, 4) && scorch::aligned_to(lists, 256),
                 "%s: index arrays must be 4-byte and lists 256-byte aligned", fn);
  if (lists_bytes < scorch_hip_sddmm_csr_lists_bytes(nnz))
    return scorch::fail(SCORCH_HIP_EWORKSPACE, "%s: %zu bytes needed for the lists, %zu given", fn,
                        scorch_hip_sddmm_csr_lists_bytes(nnz), lists_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  scorch::SddmmLists l = scorch::sddmm_lists(lists, nnz);
  if (nnz == 0 || n_cols == 0) {
    scorch::sddmm_lists_clear_kernel<<<1, 64, 0, s>>>(l.list_ptr);
    SCORCH_HIP_CHECK(hipGetLastError());
    return SCORCH_HIP_OK;
  }
  const int cols_per_bucket = (int)((n_cols + scorch::kBuckets - 1) / scorch::kBuckets);
  const int64_t waves = scorch::sddmm_pieces(nnz);
  const dim3 grid((unsigned)((waves + scorch::kWavesPerBlock - 1) / scorch::kWavesPerBlock));
  scorch::sddmm_bucket_count_kernel<<<grid, scorch::kBlockThreads, 0, s>>>(nnz, cols_per_bucket, col_idx,
                                                                          l.wave_offsets);
  SCORCH_HIP_CHECK(hipGetLastError());
  scorch::sddmm_bucket_scan_kernel<<<1, scorch::kScanThreads, 0, s>>>(waves, l.wave_offsets, l.list_ptr);
  SCORCH_HIP_CHECK(hipGetLastError());
  scorch::sddmm_bucket_fill_kernel<<<grid, scorch::kBlockThreads, 0, s>>>((int)M, nnz, cols_per_bucket, row_ptr,
                                                                         col_idx, l.wave_offsets, l.list_ptr,
                                                                         l.entry_pos, l.entry_row, l.entry_col);
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

int scorch_hip_sddmm_csr_list_values_f32(int64_t nnz, const void *lists, size_t lists_bytes, const float *vals,
                                         float *listed_vals, void *stream) {
  const char *fn = "scorch_hip_sddmm_csr_list_values_f32";
  if (nnz < 0) return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size", fn);
  if (nnz > INT32_MAX) return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  if (nnz == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(lists && vals && listed_vals, "%s: NULL array", fn);
  SCORCH_REQUIRE(scorch::aligned_to(lists, 256) && scorch::aligned_to(vals, 4) && scorch::aligned_to(listed_vals, 4),
                 "%s: lists must be 256-byte aligned, the value arrays 4-byte", fn);
  if (lists_bytes < scorch_hip_sddmm_csr_lists_bytes(nnz))
    return scorch::fail(SCORCH_HIP_EWORKSPACE, "%s: the lists of %lld entries take %zu bytes, %zu given", fn,
                        (long long)nnz, scorch_hip_sddmm_csr_lists_bytes(nnz), lists_bytes);
  const scorch::SddmmLists l = scorch::sddmm_lists(const_cast<void *>(lists), nnz);
  int64_t blocks = (nnz + scorch::kBlockThreads * 4 - 1) / (scorch::kBlockThreads * 4);
  if (blocks > 8192) blocks = 8192;  // the kernel strides
  scorch::sddmm_list_values_kernel<<<dim3((unsigned)blocks), scorch::kBlockThreads, 0,
                                     static_cast<hipStream_t>(stream)>>>(nnz, l.entry_pos, vals, listed_vals);
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

int scorch_hip_sddmm_csr_listed_f32(int64_t batch, int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                                    const void *lists, size_t lists_bytes, const float *mask_vals,
                                    const float *listed_vals, const float *A, const float *B, float *out_vals,
                                    int32_t *out_row_idx, void *stream) {
  const char *fn = "scorch_hip_sddmm_csr_listed_f32";
  if (batch < 0 || batch > 65535)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: batch=%lld is outside [0, 65535]", fn, (long long)batch);
  if (M < 0 || n_cols < 0 || K < 0 || nnz < 0)
    return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size (M=%lld n_cols=%lld K=%lld nnz=%lld)", fn,
                        (long long)M, (long long)n_cols, (long long)K, (long long)nnz);
  if (M >= INT32_MAX || n_cols > INT32_MAX || K > INT32_MAX || nnz > INT32_MAX)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  if (batch == 0 || nnz == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(lists && out_vals, "%s: NULL lists or value array", fn);
  SCORCH_REQUIRE(K == 0 || (A && B), "%s: NULL dense operand", fn);
  SCORCH_REQUIRE(scorch::aligned_to(lists, 256) && scorch::aligned_to(mask_vals, 4) && scorch::aligned_to(listed_vals, 4) &&
                     scorch::aligned_to(out_vals, 4) &&
                     scorch::aligned_to(A, 4) && scorch::aligned_to(B, 4) && scorch::aligned_to(out_row_idx, 4),
                 "%s: lists must be 256-byte aligned, the other arrays 4-byte", fn);
  if (lists_bytes < scorch_hip_sddmm_csr_lists_bytes(nnz))
    return scorch::fail(SCORCH_HIP_EWORKSPACE, "%s: lists of %zu bytes expected, %zu given", fn,
                        scorch_hip_sddmm_csr_lists_bytes(nnz), lists_bytes);
  if (K > 256)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: K=%lld beyond 256 is served by scorch_hip_sddmm_csr_f32 only", fn,
                        (long long)K);
  const scorch::SddmmLists l = scorch::sddmm_lists(const_cast<void *>(lists), nnz);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // a resident grid: every XCD's workgroups walk that XCD's list
  const int64_t waves = (nnz / scorch::kBuckets + scorch::kEntriesPerWave - 1) / scorch::kEntriesPerWave + 1;
  int64_t wgs = (waves + scorch::kWavesPerBlock - 1) / scorch::kWavesPerBlock;
  if (wgs > scorch::kListedWorkgroupsPerXcd) wgs = scorch::kListedWorkgroupsPerXcd;
  const dim3 grid((unsigned)(wgs * 8), (unsigned)batch);
  const bool vec4 = K % 4 == 0 && scorch::aligned_to(A, 16) && scorch::aligned_to(B, 16);
  const int64_t lanes_needed = (K + (vec4 ? 4 : 1) - 1) / (vec4 ? 4 : 1);
  scorch::mark_launch(s);
#define SCORCH_LISTED(GS, VEC)                                                                                   \
  scorch::sddmm_listed_kernel<GS, VEC><<<grid, scorch::kBlockThreads, 0, s>>>(                                   \
      (int)K, l.list_ptr, l.entry_pos, l.entry_row, l.entry_col, mask_vals, listed_vals, A, B, out_vals,        \
      out_row_idx, nnz,                                                                                          \
      M * K, n_cols * K)
#define SCORCH_LISTED_PICK(VEC)                          \
  do {                                                   \
    if (lanes_needed <= 4) SCORCH_LISTED(4, VEC);        \
    else if (lanes_needed <= 8) SCORCH_LISTED(8, VEC);   \
    else if (lanes_needed <= 16) SCORCH_LISTED(16, VEC); \
    else if (lanes_needed <= 32) SCORCH_LISTED(32, VEC); \
    else SCORCH_LISTED(64, VEC);                         \
  } while (0)
  if (vec4) SCORCH_LISTED_PICK(4); else SCORCH_LISTED_PICK(1);
#undef SCORCH_LISTED_PICK
#undef SCORCH_LISTED
  SCORCH_HIP_CHECK(hipGetLastError());
  scorch::mark_launch(s);
  return SCORCH_HIP_OK;
}

}  // extern "C"

SCORCH_DEFINE_PRELOAD(sddmm)
