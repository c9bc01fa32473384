// CSR x dense SpMM for a wide dense operand that is multiplied many times (a
// weight matrix): B is stored once by column tiles, and every XCD then keeps
// one tile of B in its L2 while all rows of A gather from it.
//
// Why.  With B row-major and wide (N = 4096 fp32: 16 KB per row), every stored
// entry of A gathers a whole row of B.  When B has far fewer rows than A has
// entries, each row of B is gathered several times, yet almost every gather
// goes to memory: the eight L2s are 4 MB each and B is hundreds of megabytes.
// Cutting the columns into tiles narrow enough that K rows of one tile fit an
// L2 does not help while B is row-major, because the K pieces of a tile then
// lie a full row apart and map onto a fraction of the cache's sets.
//
// Layout.  Bt[tile][k][kTileBytes / sizeof(T) columns]: tile t holds columns
// [t * TC, (t + 1) * TC) of every row of B, contiguous, zero padded past N.
// With 128-byte tile rows, K = 16,384 rows make a 2 MiB slice.  The layout is
// built by dense_to_tiled_kernel (one read and one write of B) and belongs to
// the caller, who keeps it as long as B does not change.
//
// Kernel.  A resident grid: wgs_per_xcd workgroups on each of the 8 XCDs
// (workgroup ids are dealt to XCDs round robin).  XCD x works through tiles x,
// x + 8, ... one after the other; inside a tile its wavefronts share out the
// merge-path chunks of A exactly as spmm_grouped_kernel does (lane groups of 8
// lanes x 16 bytes = one 128-byte tile row; a group per row of A, long rows by
// all groups together; carries for rows cut by chunk boundaries, folded by
// spmm_fixup_kernel).  When every wavefront has a single chunk, its indices
// and values are staged in LDS once and reused for all tiles of the XCD.  No
// workgroup waits for another: with few enough requests in flight per wavefront
// (kTiledBatch) the wavefronts of an XCD, which all have about the same work per
// tile, stay together well enough by themselves.
#include "spmm.hpp"

namespace scorch {

constexpr int kTileBytes = 128;                // bytes of one row of a column tile
constexpr int64_t kTiledSliceMax = 3 << 20;    // K * kTileBytes must fit an L2 beside A
constexpr int kTiledGroupRowMax = 64;          // longer in-chunk rows are shared by all groups
constexpr int kTiledItemsMax = 320;            // most merge items per chunk (the split may exceed the usual 256)
// A chunk stages what lies between its two boundaries, and its end may move forward by up to
// kSnapItems items to a row's end (chunk_boundary), so a wavefront's staging arrays hold this many.
constexpr int kTiledSlots = kTiledItemsMax + kSnapItems;
static_assert(kTiledItemsMax >= kItemsPerWave, "the usual split must fit the staging arrays too");
// Tile rows a lane group requests together.  Decoder shape (4096 x 16384, 32 per row, N = 4096;
// 128 workgroups per XCD, all resident), kernel time: 2: 0.126 ms, 3: 0.110, 4: 0.099, 6: 0.112,
// 8: 0.147 (0.115 with only two workgroups per CU resident): beyond four, the requests of a CU's
// sixteen wavefronts queue up in front of its vector cache faster than the L2 answers them.  With
// eight, keeping an XCD's workgroups within a tile of each other by a bounded wait on a per-XCD
// counter made up for part of it (0.137 ms); with four such a wait only costs (0.127 and more),
// as does walking a tile in two to four stretches of every row's batches (0.100 - 0.105 ms).
constexpr int kTiledBatch = 4;
constexpr int kTiledMaxWorkgroupsPerXcd = 256; // 32 CUs x 8 workgroups

inline int64_t tiled_cols(size_t elem) { return kTileBytes / (int64_t)elem; }
inline int64_t tiled_tiles(int64_t N, size_t elem) { return (N + tiled_cols(elem) - 1) / tiled_cols(elem); }
inline size_t tiled_bytes(int64_t K, int64_t N, size_t elem) {
  return (size_t)tiled_tiles(N, elem) * (size_t)K * kTileBytes;
}

// One thread per 16-byte piece of Bt.
template <typename T>
__global__ __launch_bounds__(kBlockThreads) void dense_to_tiled_kernel(int64_t K, int64_t N, int64_t pieces,
                                                                       const T *__restrict__ B,
                                                                       T *__restrict__ Bt) {
  constexpr int VEC = (int)(16 / sizeof(T));
  constexpr int LPR = kTileBytes / 16;
  const int64_t idx = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  if (idx >= pieces) return;
  const int64_t tile = idx / (K * LPR);
  const int64_t k = (idx / LPR) % K;
  const int64_t col = tile * (LPR * VEC) + (idx % LPR) * VEC;
  Vec<T, VEC> o;
#pragma unroll
  for (int v = 0; v < VEC; ++v) o.v[v] = col + v < N ? B[k * N + col + v] : (T)0;
  *reinterpret_cast<Vec<T, VEC> *>(Bt + idx * VEC) = o;
}

template <typename T, int EPI>
__global__ __launch_bounds__(kBlockThreads) void spmm_tiled_kernel(
    int M, int N, int K, const int *__restrict__ row_ptr, const int *__restrict__ col_idx,
    const T *__restrict__ vals, const T *__restrict__ Bt, T *__restrict__ C,
    const T *__restrict__ bias, int64_t total_items, int items_per_chunk, int snap, int n_tiles,
    int wgs_per_xcd, int64_t spans, int vector_stores, int *__restrict__ carry_row,
    T *__restrict__ carry_val, const Boundary *__restrict__ bounds) {
  using A = typename Acc<T>::type;
  constexpr int VEC = (int)(16 / sizeof(T));
  constexpr int LPR = kTileBytes / 16;
  constexpr int TC = LPR * VEC;
  constexpr int G = kWaveSize / LPR;
  constexpr int kSlots = kTiledSlots;
  using VecT = Vec<T, VEC>;

  __shared__ int s_col[kWavesPerBlock][kSlots];
  __shared__ T s_val[kWavesPerBlock][kSlots];
  __shared__ int s_rp[kWavesPerBlock][kSlots + 2];

  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  const int g = lane / LPR;
  const int t = lane % LPR;
  const int xcd = blockIdx.x & 7;
  const int64_t first_span = (int64_t)(blockIdx.x >> 3) * kWavesPerBlock + w;
  const int64_t span_stride = (int64_t)wgs_per_xcd * kWavesPerBlock;
  const bool single = spans <= span_stride;  // a wavefront has one chunk at most: stage it once

  int x0 = 0, y0 = 0, x1 = 0, y1 = 0, n_nz = 0, n_rows = 0;
  bool carry_in = false, staged = false;
  const bool has_work = first_span < spans;

  for (int tile = xcd; tile < n_tiles; tile += 8) {
    // A gathered row's address is the slice's (the same for the whole wavefront: scalar registers) plus
    // a byte offset of 32 bits (the entry's, staged as such, plus the lane's 16 bytes of the tile row):
    // one vector instruction per load where a 64-bit product and sum took four.
    const char *__restrict__ slice = reinterpret_cast<const char *>(Bt + (size_t)tile * (size_t)K * TC);
    const unsigned lane_bytes = (unsigned)(t * VEC * sizeof(T));
    const int col0 = tile * TC + t * VEC;
    const bool active = col0 < N;
    T bias_v[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) bias_v[v] = (EPI != kEpiNone && col0 + v < N) ? bias[col0 + v] : (T)0;

    for (int64_t span = first_span; has_work && span < spans; span += span_stride) {
      if (!(single && staged)) {
        wave_lds_sync();  // the previous chunk's reads are done
        const int64_t d0 = span * items_per_chunk;
        const Boundary from = bounds ? load_boundary(bounds, span)
                                     : chunk_boundary(d0, M, total_items, row_ptr, snap);
        const Boundary to = bounds ? load_boundary(bounds, span + 1)
                                   : chunk_boundary(d0 + items_per_chunk, M, total_items, row_ptr, snap);
        x0 = from.x, y0 = from.y, x1 = to.x, y1 = to.y;
        n_nz = y1 - y0;
        n_rows = x1 - x0;
        for (int k = lane; k < n_nz; k += kWaveSize) {
          s_col[w][k] = (int)((unsigned)col_idx[y0 + k] * (unsigned)kTileBytes);  // byte offset within a slice
          s_val[w][k] = vals[y0 + k];
        }
        for (int k = lane; k <= n_rows + 1; k += kWaveSize) {
          const int r = x0 + k < M ? x0 + k : M;
          s_rp[w][k] = row_ptr[r];
        }
        wave_lds_sync();
        carry_in = uniform(s_rp[w][0]) < y0;  // row x0 began in an earlier chunk
        staged = true;
      }

      auto add_entry = [&](A (&acc)[VEC], int k) {
        const A a = (A)s_val[w][k];
        const VecT b = *reinterpret_cast<const VecT *>(slice + ((unsigned)s_col[w][k] + lane_bytes));
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += a * (A)b.v[v];
      };

      // Row slot r is row x0 + r; slot n_rows is the row that continues past the chunk.
      for (int base = 0; base <= n_rows; base += G) {
        const int slot = base + g;
        const bool live = slot <= n_rows;
        int lo = 0, hi = 0;
        if (live) {
          const int begin = s_rp[w][slot], end = s_rp[w][slot + 1];
          lo = (begin > y0 ? begin : y0) - y0;
          hi = (end < y1 ? end : y1) - y0;
          if (hi < lo) hi = lo;
        }
        const int len = hi - lo;
        A acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = (A)0;

        if (len <= kTiledGroupRowMax) {
          int k = lo;
          for (; k + kTiledBatch <= hi; k += kTiledBatch) {
            VecT b[kTiledBatch];
            A a[kTiledBatch];
#pragma unroll
            for (int u = 0; u < kTiledBatch; ++u) {
              a[u] = (A)s_val[w][k + u];
              b[u] = *reinterpret_cast<const VecT *>(slice + ((unsigned)s_col[w][k + u] + lane_bytes));
            }
#pragma unroll
            for (int u = 0; u < kTiledBatch; ++u)
#pragma unroll
              for (int v = 0; v < VEC; ++v) acc[v] += a[u] * (A)b[u].v[v];
          }
          for (; k < hi; ++k) add_entry(acc, k);
        }

        // Rows with many entries in the chunk: one at a time, all groups.
        unsigned long long pending = __ballot(len > kTiledGroupRowMax && t == 0);
        while (pending) {
          const int owner_lane = __ffsll(pending) - 1;  // lane 0 of the owning group
          pending &= pending - 1;
          const int olo = __shfl(lo, owner_lane), ohi = __shfl(hi, owner_lane);
          A part[VEC];
#pragma unroll
          for (int v = 0; v < VEC; ++v) part[v] = (A)0;
          for (int k = olo + g; k < ohi; k += G) add_entry(part, k);
#pragma unroll
          for (int off = LPR; off < kWaveSize; off <<= 1)
#pragma unroll
            for (int v = 0; v < VEC; ++v) part[v] += (A)__shfl_xor((T)part[v], off);
          if (g == owner_lane / LPR) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) acc[v] = part[v];
          }
        }

        if (live && active) {
          const bool whole_row = slot < n_rows;
          if (whole_row || len > 0) {
            const bool partial = !whole_row || (carry_in && slot == 0);
            T *dst = whole_row ? C + (size_t)(x0 + slot) * (size_t)N + col0
                               : carry_val + (size_t)span * (size_t)N + col0;
            VecT o;
#pragma unroll
            for (int v = 0; v < VEC; ++v)
              o.v[v] = partial ? (T)acc[v] : apply_epilogue<T, EPI>(acc[v], bias_v[v]);
            if (vector_stores) {
              store_streaming(dst, o);  // C passes through once; the L2 is for the slice of B
            } else {
#pragma unroll
              for (int v = 0; v < VEC; ++v)
                if (col0 + v < N) dst[v] = o.v[v];
            }
          }
        }
        if (live && slot == n_rows && tile == 0 && t == 0) carry_row[span] = len > 0 ? x1 : -1;
      }
    }
  }
}

template <typename T, int EPI>
int spmm_tiled_entry(const char *fn, int64_t M, int64_t K, int64_t N, int64_t nnz, const int32_t *row_ptr,
                     const int32_t *col_idx, const T *vals, const T *Bt, size_t bt_bytes, const T *bias, T *C,
                     const void *bounds_buffer, size_t bounds_bytes, void *workspace, size_t workspace_bytes,
                     int64_t longest_row, void *stream) {
  if (int rc = check_csr_args(fn, M, K, nnz, row_ptr, col_idx, vals)) return rc;
  SCORCH_REQUIRE(N >= 0, "%s: negative N=%lld", fn, (long long)N);
  if (N > INT32_MAX - kWaveSize * 4)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: N=%lld is too large", fn, (long long)N);
  if (M == 0 || N == 0) return SCORCH_HIP_OK;  // nothing to write
  if (K * (int64_t)kTileBytes > (int64_t)UINT32_MAX)  // (the kernel addresses a slice with 32-bit byte offsets)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: K=%lld rows make a slice of more than 4 GiB", fn, (long long)K);
  SCORCH_REQUIRE(C != nullptr, "%s: C is NULL", fn);
  SCORCH_REQUIRE(K == 0 || Bt != nullptr, "%s: the tiled operand is NULL", fn);
  SCORCH_REQUIRE(EPI == kEpiNone || bias != nullptr, "%s: bias is NULL", fn);
  SCORCH_REQUIRE(aligned_to(Bt, kTileBytes), "%s: the tiled operand must be %d-byte aligned", fn, kTileBytes);
  SCORCH_REQUIRE(aligned_to(C, sizeof(T)) && aligned_to(vals, sizeof(T)) && aligned_to(bias, sizeof(T)),
                 "%s: value arrays must be aligned to their element size", fn);
  if (bt_bytes < tiled_bytes(K, N, sizeof(T)))
    return fail(SCORCH_HIP_EINVAL, "%s: the tiled operand has %zu bytes, %zu needed for K=%lld N=%lld", fn,
                bt_bytes, tiled_bytes(K, N, sizeof(T)), (long long)K, (long long)N);
  const size_t need = spmm_workspace_bytes(M, nnz, N, sizeof(T));
  if (!workspace || workspace_bytes < need)
    return fail(SCORCH_HIP_EWORKSPACE, "%s: workspace of %zu bytes needed, %zu given", fn, need,
                workspace ? workspace_bytes : (size_t)0);
  SCORCH_REQUIRE(aligned_to(workspace, 256), "%s: workspace must be 256-byte aligned", fn);
  SpmmSplit split = spmm_split(M, nnz, N, sizeof(T));
  const Boundary *bounds = static_cast<const Boundary *>(bounds_buffer);
  // When every wavefront gets one chunk anyway (the whole grid is resident), cut the work into a
  // multiple of 128 chunks, i.e. the same number of wavefronts for each of an XCD's 128 SIMDs:
  // 528 chunks of 256 items leave some CUs with five workgroups and others with four, and the
  // XCD then waits for the fuller ones in every tile (0.190 against 0.158 ms with 512 chunks of
  // 264 items on the decoder shape).  Boundaries computed for the usual split do not apply then.
  if (split.spans > 128 && split.spans <= (int64_t)kTiledMaxWorkgroupsPerXcd * kWavesPerBlock) {
    const int64_t even = split.spans / 128 * 128;
    const int64_t ipc = (M + nnz + even - 1) / even;
    if (even != split.spans && ipc <= kTiledItemsMax) {
      split.items_per_chunk = (int)ipc;
      split.spans = (M + nnz + ipc - 1) / ipc;
      bounds = nullptr;
    }
  }
  if (split.items_per_chunk + split.snap > kTiledSlots)
    return fail(SCORCH_HIP_ERUNTIME, "%s: chunks of %d + %d items exceed the %d staging slots", fn,
                split.items_per_chunk, split.snap, kTiledSlots);
  if (bounds) {
    const size_t have = (size_t)(split.spans + 1) * sizeof(Boundary);
    if (bounds_bytes < have)
      return fail(SCORCH_HIP_EWORKSPACE, "%s: chunk boundaries of %zu bytes needed, %zu given", fn, have,
                  bounds_bytes);
    SCORCH_REQUIRE(aligned_to(bounds, 8), "%s: the chunk boundaries must be 8-byte aligned", fn);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  int *carry_row = static_cast<int *>(workspace);
  T *carry_val = reinterpret_cast<T *>(static_cast<char *>(workspace) +
                                       align_up((size_t)split.spans * sizeof(int), 256));
  constexpr int VEC = (int)(16 / sizeof(T));
  const int vector_stores = N % VEC == 0 && aligned_to(C, 16) && aligned_to(carry_val, 16);
  int64_t wgs = (split.spans + kWavesPerBlock - 1) / kWavesPerBlock;
  if (wgs > kTiledMaxWorkgroupsPerXcd) wgs = kTiledMaxWorkgroupsPerXcd;
  mark_launch(s);
  spmm_tiled_kernel<T, EPI><<<dim3((unsigned)(wgs * 8)), kBlockThreads, 0, s>>>(
      (int)M, (int)N, (int)K, row_ptr, col_idx, vals, Bt, C, bias, M + nnz, split.items_per_chunk, split.snap,
      (int)tiled_tiles(N, sizeof(T)), (int)wgs, split.spans, vector_stores, carry_row, carry_val, bounds);
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(s);
  // A boundary that falls inside a row moves to the row's end when that is at most `snap` items
  // away (chunk_boundary): with no row longer than that no chunk leaves a carry, and a caller who
  // knows the longest row (the inspection reports it) saves the launch that would look for them.
  if (longest_row > 0 && longest_row <= split.snap) return SCORCH_HIP_OK;
  const int64_t fix_per_block = kWavesPerBlock * kFixupChunks;
  spmm_fixup_kernel<T, 1, EPI><<<dim3((unsigned)((split.spans + fix_per_block - 1) / fix_per_block)),
                                 kBlockThreads, 0, s>>>((int)N, split.spans, carry_row, carry_val, C, bias,
                                                        SpmmBatch{0, 0, 0, 0});
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(s);
  return SCORCH_HIP_OK;
}

}  // namespace scorch

extern "C" {

size_t scorch_hip_dense_tiled_bytes(int64_t K, int64_t N, size_t elem_size) {
  if (K < 0 || N < 0 || (elem_size != 4 && elem_size != 8)) return 0;
  return scorch::tiled_bytes(K, N, elem_size);
}

int scorch_hip_dense_tiled_recommended(int64_t K, int64_t N, int64_t nnz, size_t elem_size) {
  if (K <= 0 || N <= 0 || (elem_size != 4 && elem_size != 8)) return 0;
  // worth it when a row of B spans many tiles, a tile's slice fits an L2, and the rows of B
  // are gathered more than once on average
  return N * (int64_t)elem_size >= 16 * scorch::kTileBytes && K * scorch::kTileBytes <= scorch::kTiledSliceMax &&
         nnz >= 2 * K;
}

int scorch_hip_dense_to_tiled_f32(int64_t K, int64_t N, const float *B, float *Bt, size_t bt_bytes,
                                  void *stream) {
  const char *fn = "scorch_hip_dense_to_tiled_f32";
  SCORCH_REQUIRE(K >= 0 && N >= 0, "%s: negative size (K=%lld N=%lld)", fn, (long long)K, (long long)N);
  if (K == 0 || N == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(B != nullptr && Bt != nullptr, "%s: B or Bt is NULL", fn);
  SCORCH_REQUIRE(scorch::aligned_to(B, 4) && scorch::aligned_to(Bt, scorch::kTileBytes),
                 "%s: B must be 4-byte and Bt %d-byte aligned", fn, scorch::kTileBytes);
  const size_t need = scorch::tiled_bytes(K, N, sizeof(float));
  if (bt_bytes < need)
    return scorch::fail(SCORCH_HIP_EINVAL, "%s: Bt has %zu bytes, %zu needed", fn, bt_bytes, need);
  const int64_t pieces = (int64_t)(need / 16);
  const int64_t blocks = (pieces + scorch::kBlockThreads - 1) / scorch::kBlockThreads;
  if (blocks > INT32_MAX)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: %lld workgroups exceed the launch limit", fn,
                        (long long)blocks);
  scorch::dense_to_tiled_kernel<float><<<dim3((unsigned)blocks), scorch::kBlockThreads, 0,
                                        static_cast<hipStream_t>(stream)>>>(K, N, pieces, B, Bt);
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

int scorch_hip_spmm_csr_tiled_f32(int64_t M, int64_t K, int64_t N, int64_t nnz, const int32_t *row_ptr,
                                  const int32_t *col_idx, const float *vals, const float *Bt, size_t bt_bytes,
                                  const float *bias, int act, float *C, const void *bounds,
                                  size_t bounds_bytes, void *workspace, size_t workspace_bytes,
                                  int64_t longest_row, void *stream) {
  const char *fn = "scorch_hip_spmm_csr_tiled_f32";
  if (!bias && act == SCORCH_HIP_ACT_NONE)
    return scorch::spmm_tiled_entry<float, scorch::kEpiNone>(fn, M, K, N, nnz, row_ptr, col_idx, vals, Bt,
                                                             bt_bytes, nullptr, C, bounds, bounds_bytes,
                                                             workspace, workspace_bytes, longest_row, stream);
  if (bias && act == SCORCH_HIP_ACT_NONE)
    return scorch::spmm_tiled_entry<float, scorch::kEpiBias>(fn, M, K, N, nnz, row_ptr, col_idx, vals, Bt,
                                                             bt_bytes, bias, C, bounds, bounds_bytes, workspace,
                                                             workspace_bytes, longest_row, stream);
  if (bias && act == SCORCH_HIP_ACT_RELU)
    return scorch::spmm_tiled_entry<float, scorch::kEpiBiasRelu>(fn, M, K, N, nnz, row_ptr, col_idx, vals, Bt,
                                                                 bt_bytes, bias, C, bounds, bounds_bytes,
                                                                 workspace, workspace_bytes, longest_row, stream);
  return scorch::fail(SCORCH_HIP_EINVAL, "%s: activation %d (with%s bias) is not supported", fn, act,
                      bias ? "" : "out");
}

}  // extern "C"

SCORCH_DEFINE_PRELOAD(spmm_tiled)
