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
// and values are staged in LDS once and reused for all tiles of the XCD.  The
// workgroups of an XCD are kept within a tile of each other by a bounded wait on
// a per-XCD counter (see "Pacing" in the kernel): left alone they drift apart by
// a tile or two over sixteen tiles, the L2 then holds parts of several slices and
// half of the gathers miss.
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
constexpr int kTiledBatch = 8;                 // tile-row loads in flight per lane group (16 measured slower)
constexpr int kTiledMaxWorkgroupsPerXcd = 256; // 32 CUs x 8 workgroups
constexpr int kPacePolls = 400;                // polls after which a wavefront stops waiting for the others
// Share of an XCD's workgroups that must have finished a tile before the next is begun.  On the
// decoder shape (4096 x 16384, 32 per row, N = 4096), with C written by streaming stores: no
// pacing 0.146 ms; 50 to 80 % 0.135 - 0.137 ms; 90 % 0.141 ms; 95 % 0.150 ms (the slice comes in
// fewer times, but every tile waits for its slowest workgroups).  Of the flat range the upper end
// fetches least.
constexpr int kPacePercent = 80;
constexpr int kTiledPacedWorkgroupsPerXcd = 160;  // 32 CUs x 5 workgroups surely resident together
// The kernel for operands whose rows are all short (spmm_tiled_short_rows_kernel): the most
// workgroups per XCD it is launched with (32 CUs x 5, all resident), and the tile rows a lane group
// requests together.  Decoder shape (4096 x 16384, 32 per row, N = 4096; 128 workgroups per XCD),
// kernel time by that number: 2: 0.126 ms, 3: 0.110, 4: 0.099, 6: 0.112, 8: 0.147 (0.115 with only
// two workgroups per CU resident): beyond four the requests of a CU's sixteen wavefronts queue up
// in front of its vector cache faster than the L2 answers them.
constexpr int kShortRowsWorkgroupsPerXcd = 160;
constexpr int kShortRowsBatch = 4;

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
    T *__restrict__ carry_val, const Boundary *__restrict__ bounds, int *__restrict__ pace, int pace_need,
    int pace_zero) {
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

  // Pacing.  The workgroups of an XCD should all be in the same tile: one that runs ahead pulls
  // the next slice into the L2 and pushes out lines of the current one that the others still need.
  // pace[xcd * kPaceStride] counts the workgroups of this XCD that have finished a tile; before
  // tile number `it` a workgroup waits until pace_need of every earlier tile's finishers are
  // there (fewer than all lets the last few finish while the rest start).  The counter is only
  // touched by workgroups of one XCD, so its updates and polls are atomics that execute in that
  // XCD's L2 (workgroup scope: nothing has to be visible to another XCD; `pace_zero` is 0, added
  // so that a poll is a read-modify-write the L2 performs, not a load a CU's vector cache may answer).
  // The wait is bounded: a workgroup that has polled kPacePolls times goes on regardless and never
  // waits again, so the kernel ends whatever happens to the others; results do not depend on it.
  int *my_pace = pace + xcd * kPaceStride;
  __shared__ int s_gave_up;
  bool paced = pace_need > 0;  // the same in all threads of the workgroup
  int it = 0;

  for (int tile = xcd; tile < n_tiles; tile += 8, ++it) {
    if (pace_need > 0) {
      __syncthreads();  // everybody is done with the previous tile (and has read s_gave_up)
      if (it > 0 && paced) {
        if (threadIdx.x == 0) {
          __hip_atomic_fetch_add(my_pace, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          const int need = it * pace_need;
          int polls = 0, gave_up = 0;
          while (__hip_atomic_fetch_add(my_pace, pace_zero, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) < need) {
            if (++polls > kPacePolls) {
              gave_up = 1;
              break;
            }
            __builtin_amdgcn_s_sleep(16);
          }
          s_gave_up = gave_up;
        }
        __syncthreads();
        paced = s_gave_up == 0;
      }
    }
    const T *__restrict__ slice = Bt + (size_t)tile * (size_t)K * TC + t * VEC;
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
          s_col[w][k] = col_idx[y0 + k];
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
        const VecT b = *reinterpret_cast<const VecT *>(slice + (size_t)s_col[w][k] * TC);
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
              b[u] = *reinterpret_cast<const VecT *>(slice + (size_t)s_col[w][k + u] * TC);
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

// ---- operands whose rows are all short ----------------------------------------------------------
// One batch of a row's entries against the tile's slice: entries k .. k + kShortRowsBatch - 1 of the
// staged chunk (a lane group per row: 8 lanes x 16 bytes cover a tile row), the tile rows
// requested together.  In a row's last batch, which may reach past the row's end `hi`, the
// positions beyond it request the row's last entry again and contribute nothing.
template <typename T, typename A, int VEC>
__device__ __forceinline__ void tiled_gather_batch(A (&acc)[VEC], int k, int hi, const int *s_col, const T *s_val,
                                                   const T *__restrict__ slice, int TC) {
  using VecT = Vec<T, VEC>;
  VecT bv[kShortRowsBatch];
  A av[kShortRowsBatch];
  if (k + kShortRowsBatch <= hi) {
#pragma unroll
    for (int u = 0; u < kShortRowsBatch; ++u) {
      av[u] = (A)s_val[k + u];
      bv[u] = *reinterpret_cast<const VecT *>(slice + (size_t)s_col[k + u] * TC);
    }
#pragma unroll
    for (int u = 0; u < kShortRowsBatch; ++u)
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] += av[u] * (A)bv[u].v[v];
  } else {
#pragma unroll
    for (int u = 0; u < kShortRowsBatch; ++u) {
      const int e = k + u < hi ? k + u : hi - 1;
      av[u] = (A)s_val[e];
      bv[u] = *reinterpret_cast<const VecT *>(slice + (size_t)s_col[e] * TC);
    }
#pragma unroll
    for (int u = 0; u < kShortRowsBatch; ++u)
      if (k + u < hi) {  // (not a zero factor: the stand-in may be infinite)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += av[u] * (A)bv[u].v[v];
      }
  }
}

// The tiled product for an operand of which the caller knows that no row has more than
// kTiledGroupRowMax entries (SCORCH_HIP_HINT_SHORT_ROWS), launched with one chunk per wavefront
// and at most kShortRowsWorkgroupsPerXcd workgroups per XCD, all resident.  Every row is one lane
// group's, whole, in batches of kShortRowsBatch tile rows; no workgroup waits for another: XCD x
// walks tiles x, x + 8, ... and its wavefronts, which all have the same amount of work per tile,
// stay together well enough by themselves.  Results are those of spmm_tiled_kernel bit for bit
// (the same entries in the same order per row).  Decoder shape, same box, same run:
// spmm_tiled_kernel paced 0.137 - 0.140 ms, unpaced 0.148; this kernel 0.099.  Measured and left
// out: a tile walked in two to four stretches of every row's batches with the rows' sums kept in
// registers in between (0.100 - 0.105 ms; by column ranges instead of by batch count 0.122), any
// pacing on top of it (0.127 and more), two batches in flight per lane group (registers spill).
template <typename T, int EPI>
__global__ __launch_bounds__(kBlockThreads) void spmm_tiled_short_rows_kernel(
    int M, int N, int K, const int *__restrict__ row_ptr, const int *__restrict__ col_idx,
    const T *__restrict__ vals, const T *__restrict__ Bt, T *__restrict__ C,
    const T *__restrict__ bias, int64_t total_items, int items_per_chunk, int snap, int n_tiles,
    int64_t spans, int vector_stores, int *__restrict__ carry_row, T *__restrict__ carry_val,
    const Boundary *__restrict__ bounds) {
  using A = typename Acc<T>::type;
  constexpr int VEC = (int)(16 / sizeof(T));
  constexpr int LPR = kTileBytes / 16;
  constexpr int TC = LPR * VEC;
  constexpr int G = kWaveSize / LPR;
  using VecT = Vec<T, VEC>;

  __shared__ int s_col[kWavesPerBlock][kTiledSlots];
  __shared__ T s_val[kWavesPerBlock][kTiledSlots];
  __shared__ int s_rp[kWavesPerBlock][kTiledSlots + 2];

  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  const int g = lane / LPR;
  const int t = lane % LPR;
  const int xcd = blockIdx.x & 7;
  const int64_t span = (int64_t)(blockIdx.x >> 3) * kWavesPerBlock + w;
  if (span >= spans) return;  // (no workgroup barriers below)

  // the wavefront's chunk, staged once for all tiles
  const int64_t d0 = span * items_per_chunk;
  const Boundary from = bounds ? load_boundary(bounds, span) : chunk_boundary(d0, M, total_items, row_ptr, snap);
  const Boundary to = bounds ? load_boundary(bounds, span + 1)
                             : chunk_boundary(d0 + items_per_chunk, M, total_items, row_ptr, snap);
  const int x0 = from.x, y0 = from.y, x1 = to.x, y1 = to.y;
  const int n_nz = y1 - y0, n_rows = x1 - x0;
  for (int k = lane; k < n_nz; k += kWaveSize) {
    s_col[w][k] = col_idx[y0 + k];
    s_val[w][k] = vals[y0 + k];
  }
  for (int k = lane; k <= n_rows + 1; k += kWaveSize) {
    const int r = x0 + k < M ? x0 + k : M;
    s_rp[w][k] = row_ptr[r];
  }
  wave_lds_sync();
  const bool carry_in = uniform(s_rp[w][0]) < y0;  // row x0 began in an earlier chunk
  // entries [lo, hi) of row slot `slot` inside the staged chunk (slot n_rows: the row that continues)
  auto slot_range = [&](int slot, int &lo, int &hi) {
    const int begin = s_rp[w][slot], end = s_rp[w][slot + 1];
    lo = (begin > y0 ? begin : y0) - y0;
    hi = (end < y1 ? end : y1) - y0;
    if (hi < lo) hi = lo;
  };
  // a row's sums go to C, or (the row that continues past the chunk, or began before it) to the carries
  auto store_row = [&](int slot, int len, const A (&acc)[VEC], int col0, const T (&bias_v)[VEC]) {
    const bool whole_row = slot < n_rows;
    if (!whole_row && len == 0) return;
    const bool partial = !whole_row || (carry_in && slot == 0);
    T *dst = whole_row ? C + (size_t)(x0 + slot) * (size_t)N + col0 : carry_val + (size_t)span * (size_t)N + col0;
    VecT o;
#pragma unroll
    for (int v = 0; v < VEC; ++v) o.v[v] = partial ? (T)acc[v] : apply_epilogue<T, EPI>(acc[v], bias_v[v]);
    if (vector_stores) {
      store_streaming(dst, o);  // C passes through once; the L2 is for the slice of B
    } else {
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        if (col0 + v < N) dst[v] = o.v[v];
    }
  };
  for (int tile = xcd; tile < n_tiles; tile += 8) {
    const int col0 = tile * TC + t * VEC;
    const bool active = col0 < N;
    T bias_v[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) bias_v[v] = (EPI != kEpiNone && col0 + v < N) ? bias[col0 + v] : (T)0;
    const T *__restrict__ slice = Bt + (size_t)tile * (size_t)K * TC + t * VEC;
    // eight row slots at a time; slot n_rows is the row that continues past the chunk
    for (int base = 0; base <= n_rows; base += G) {
      const int slot = base + g;
      if (slot <= n_rows) {
        int lo, hi;
        slot_range(slot, lo, hi);
        A acc[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] = (A)0;
        for (int k = lo; k < hi; k += kShortRowsBatch)
          tiled_gather_batch<T, A, VEC>(acc, k, hi, s_col[w], s_val[w], slice, TC);
        if (active) store_row(slot, hi - lo, acc, col0, bias_v);
        if (slot == n_rows && tile == 0 && t == 0) carry_row[span] = hi > lo ? x1 : -1;
      }
    }
  }
}

// pace counters start at zero (a kernel, not a memset, so that the call can be captured in a graph)
__global__ void spmm_tiled_clear_kernel(int *__restrict__ pace) {
  if (threadIdx.x < 8) pace[threadIdx.x * kPaceStride] = 0;
}

template <typename T, int EPI>
int spmm_tiled_entry(const char *fn, int64_t M, int64_t K, int64_t N, int64_t nnz, const int32_t *row_ptr,
                     const int32_t *col_idx, const T *vals, const T *Bt, size_t bt_bytes, const T *bias, T *C,
                     const void *bounds_buffer, size_t bounds_bytes, void *workspace, size_t workspace_bytes,
                     void *stream, bool short_rows) {
  if (int rc = check_csr_args(fn, M, K, nnz, row_ptr, col_idx, vals)) return rc;
  SCORCH_REQUIRE(N >= 0, "%s: negative N=%lld", fn, (long long)N);
  if (N > INT32_MAX - kWaveSize * 4)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: N=%lld is too large", fn, (long long)N);
  if (M == 0 || N == 0) return SCORCH_HIP_OK;  // nothing to write
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
  const size_t carry_bytes = need - kPaceBytes;
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
  const int64_t fix_per_block = kWavesPerBlock * kFixupChunks;
  if (short_rows && split.spans <= wgs * kWavesPerBlock && wgs <= kShortRowsWorkgroupsPerXcd) {
    // every row short, one chunk per wavefront, all of them resident: the kernel that waits for nobody
    mark_launch(s);
    spmm_tiled_short_rows_kernel<T, EPI><<<dim3((unsigned)(wgs * 8)), kBlockThreads, 0, s>>>(
        (int)M, (int)N, (int)K, row_ptr, col_idx, vals, Bt, C, bias, M + nnz, split.items_per_chunk, split.snap,
        (int)tiled_tiles(N, sizeof(T)), split.spans, vector_stores, carry_row, carry_val, bounds);
    SCORCH_HIP_CHECK(hipGetLastError());
    mark_launch(s);
    spmm_fixup_kernel<T, 1, EPI><<<dim3((unsigned)((split.spans + fix_per_block - 1) / fix_per_block)),
                                   kBlockThreads, 0, s>>>((int)N, split.spans, carry_row, carry_val, C, bias,
                                                          SpmmBatch{0, 0, 0, 0});
    SCORCH_HIP_CHECK(hipGetLastError());
    mark_launch(s);
    return SCORCH_HIP_OK;
  }
  // Pacing only when every wavefront with work is resident at once (one chunk per wavefront and
  // the grid within what the chip holds); otherwise waiting for wavefronts that have not started
  // would only run into the poll limit.
  int *pace = reinterpret_cast<int *>(static_cast<char *>(workspace) + carry_bytes);
  int pace_need = 0;
  if (split.spans <= wgs * kWavesPerBlock && wgs <= kTiledPacedWorkgroupsPerXcd) {
    pace_need = (int)(wgs * kPacePercent / 100);
  }
  mark_launch(s);
  spmm_tiled_clear_kernel<<<1, 64, 0, s>>>(pace);
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(s);
  spmm_tiled_kernel<T, EPI><<<dim3((unsigned)(wgs * 8)), kBlockThreads, 0, s>>>(
      (int)M, (int)N, (int)K, row_ptr, col_idx, vals, Bt, C, bias, M + nnz, split.items_per_chunk, split.snap,
      (int)tiled_tiles(N, sizeof(T)), (int)wgs, split.spans, vector_stores, carry_row, carry_val, bounds, pace,
      pace_need, 0);
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(s);
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
                                  size_t bounds_bytes, void *workspace, size_t workspace_bytes, void *stream) {
  const char *fn = "scorch_hip_spmm_csr_tiled_f32";
  const bool short_rows = (act & SCORCH_HIP_HINT_SHORT_ROWS) != 0;
  act &= ~SCORCH_HIP_HINT_SHORT_ROWS;
  if (!bias && act == SCORCH_HIP_ACT_NONE)
    return scorch::spmm_tiled_entry<float, scorch::kEpiNone>(fn, M, K, N, nnz, row_ptr, col_idx, vals, Bt,
                                                             bt_bytes, nullptr, C, bounds, bounds_bytes,
                                                             workspace, workspace_bytes, stream, short_rows);
  if (bias && act == SCORCH_HIP_ACT_NONE)
    return scorch::spmm_tiled_entry<float, scorch::kEpiBias>(fn, M, K, N, nnz, row_ptr, col_idx, vals, Bt,
                                                             bt_bytes, bias, C, bounds, bounds_bytes, workspace,
                                                             workspace_bytes, stream, short_rows);
  if (bias && act == SCORCH_HIP_ACT_RELU)
    return scorch::spmm_tiled_entry<float, scorch::kEpiBiasRelu>(fn, M, K, N, nnz, row_ptr, col_idx, vals, Bt,
                                                                 bt_bytes, bias, C, bounds, bounds_bytes,
                                                                 workspace, workspace_bytes, stream, short_rows);
  return scorch::fail(SCORCH_HIP_EINVAL, "%s: activation %d (with%s bias) is not supported", fn, act,
                      bias ? "" : "out");
}

}  // extern "C"
