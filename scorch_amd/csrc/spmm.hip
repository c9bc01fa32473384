// CSR x dense SpMM for gfx950: merge-path work split, one wavefront per chunk.
//
// Work model.  The rows of A and its nonzeros are merged into one sequence of
// M + nnz items: nonzero p of row i sits at position p + i, the "end of row i"
// marker at row_ptr[i+1] + i.  The sequence is cut into chunks of
// kItemsPerWave items; wavefront c owns chunk c.  A wavefront therefore does a
// bounded amount of work whatever the row-length distribution: a 50 000-entry
// row is spread over ~200 wavefronts, 250 one-entry rows share one.
//
// Within a chunk the wavefront walks its nonzeros in order.  All 64 lanes work
// on the SAME nonzero: lane l holds VEC consecutive output columns, so one B
// row is read with a single coalesced wave-wide load (64 * VEC elements) and
// the column index / value are wave-uniform (scalar registers, scalar address
// arithmetic).  When the walk reaches an end-of-row marker the accumulator is
// stored to C and cleared.  Every row's marker belongs to exactly one chunk,
// so every row of C is stored exactly once (empty rows store zeros) and C
// needs no prior zero fill.
//
// Rows cut by a chunk boundary.  A chunk that ends inside a row has no marker
// for it; it writes its partial sum to carry_val[chunk] and the row number to
// carry_row[chunk].  The chunk holding the marker stores only its own part.
// spmm_fixup_kernel then adds, in chunk order, the carries of each such row
// to C: a fixed summation order, so results are bit-reproducible, and no
// atomics.  A fused bias/ReLU epilogue is applied at the store when the row
// lies wholly inside the chunk, and by the fix-up otherwise.
//
// Columns beyond 64 * VEC are covered by column tiles (each tile walks the same
// chunks again; A's indices are small next to the B rows gathered).  Tiles are
// placed on XCDs so that a tile's slice of B stays in one L2 (map_workgroup).
#include "spmm.hpp"

#include <mutex>

namespace scorch {

// C = 0 in 16-byte pieces with streaming stores (grid-stride).
__global__ __launch_bounds__(kBlockThreads) void zero_fill_kernel(uint4 *__restrict__ out, int64_t pieces) {
  const int64_t stride = (int64_t)gridDim.x * kBlockThreads;
  typedef unsigned Native __attribute__((ext_vector_type(4)));
  for (int64_t i = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x; i < pieces; i += stride)
    __builtin_nontemporal_store(Native{0u, 0u, 0u, 0u}, reinterpret_cast<Native *>(out + i));
}

template <typename T, int VEC, int EPI>
__global__ __launch_bounds__(kBlockThreads) void spmm_merge_kernel(
    int M, int N, const int *__restrict__ row_ptr, const int *__restrict__ col_idx,
    const T *__restrict__ vals, const T *__restrict__ B, T *__restrict__ C,
    const T *__restrict__ bias, int64_t total_items, int items_per_chunk, int snap, int n_tiles,
    int64_t blocks_per_tile, int *__restrict__ carry_row, T *__restrict__ carry_val,
    const Boundary *__restrict__ bounds, SpmmBatch batch, int zero_filled) {
  using A = typename Acc<T>::type;
  using VecT = Vec<T, VEC>;
  constexpr int kSlots = kItemsPerWave + kSnapItems;
  vals += blockIdx.y * batch.vals;  // problem blockIdx.y of a batch over one pattern
  B += blockIdx.y * batch.b;
  C += blockIdx.y * batch.c;
  carry_val += blockIdx.y * batch.carry;

  __shared__ int s_col[kWavesPerBlock][kSlots];
  __shared__ T s_val[kWavesPerBlock][kSlots];
  __shared__ int s_rp[kWavesPerBlock][kSlots + 2];

  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  const TileMap where = map_workgroup(blockIdx.x, n_tiles, blocks_per_tile);
  const int64_t chunk = where.block * kWavesPerBlock + w;
  const int col0 = (where.tile * kWaveSize + lane) * VEC;
  const bool active = col0 < N;

  const int64_t d0 = chunk * items_per_chunk;
  if (d0 >= total_items) return;  // only wave-level synchronisation below
  const Boundary from = bounds ? load_boundary(bounds, chunk) : chunk_boundary(d0, M, total_items, row_ptr, snap);
  const Boundary to = bounds ? load_boundary(bounds, chunk + 1)
                             : chunk_boundary(d0 + items_per_chunk, M, total_items, row_ptr, snap);
  const int x0 = from.x, y0 = from.y, x1 = to.x, y1 = to.y;
  const int n_nz = y1 - y0;
  const int n_rows = x1 - x0;

  // Stage the chunk's slice of A in LDS: coalesced loads now, broadcast reads later.
  for (int k = lane; k < n_nz; k += kWaveSize) {
    s_col[w][k] = col_idx[y0 + k];
    s_val[w][k] = vals[y0 + k];
  }
  // s_rp[k] = row_ptr[x0 + k] for k = 0 .. n_rows + 1 (clamped at M).
  for (int k = lane; k <= n_rows + 1; k += kWaveSize) {
    const int r = x0 + k < M ? x0 + k : M;
    s_rp[w][k] = row_ptr[r];
  }
  wave_lds_sync();  // the slices are private to this wavefront

  // Row x0 began in an earlier chunk iff its first nonzero precedes y0: then
  // its store is a partial sum and its epilogue is the fix-up's.
  const bool carry_in = uniform(s_rp[w][0]) < y0;

  T bias_v[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) bias_v[v] = (EPI != kEpiNone && active) ? bias[col0 + v] : (T)0;

  A acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = (A)0;

  int x = x0;  // next row to finish
  int next_end = uniform(s_rp[w][1]);
  // zero_filled: C holds zeros already (a matrix most of whose rows are empty: one streaming
  // fill and then only the other rows, instead of row-sized zero stores mixed into the gathers);
  // a row none of whose entries this chunk has seen then needs no store
  bool touched = !zero_filled;

  auto flush_row = [&]() {
    if (active && touched) {
      const bool partial = carry_in && x == x0;
      VecT o;
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        o.v[v] = partial ? (T)acc[v] : apply_epilogue<T, EPI>(acc[v], bias_v[v]);
      store_streaming(C + (size_t)x * (size_t)N + col0, o);
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] = (A)0;
    touched = !zero_filled;
    ++x;
    next_end = uniform(s_rp[w][x - x0 + 1]);
  };

  auto gather = [&](int k) -> VecT {
    const int j = uniform(s_col[w][k]);
    VecT b;
    if (active) {
      b = *reinterpret_cast<const VecT *>(B + (size_t)j * (size_t)N + col0);
    } else {
#pragma unroll
      for (int v = 0; v < VEC; ++v) b.v[v] = (T)0;
    }
    return b;
  };

  auto consume = [&](int k, const VecT &b) {
    while (y0 + k == next_end) flush_row();  // markers that precede nonzero y0 + k
    touched = true;
    const A a = (A)s_val[w][k];
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[v] += a * (A)b.v[v];
  };

  int k = 0;
  for (; k + kGather <= n_nz; k += kGather) {
    VecT b[kGather];
#pragma unroll
    for (int u = 0; u < kGather; ++u) b[u] = gather(k + u);
#pragma unroll
    for (int u = 0; u < kGather; ++u) consume(k + u, b[u]);
  }
  for (; k < n_nz; ++k) consume(k, gather(k));
  while (x < x1) flush_row();  // markers after the chunk's last nonzero

  // Whatever is left belongs to row x1, whose marker lies in a later chunk.
  const int row_start = uniform(s_rp[w][n_rows]);  // row_ptr[x1]
  const int tail = y1 - (row_start > y0 ? row_start : y0);
  if (where.tile == 0 && lane == 0 && blockIdx.y == 0) carry_row[chunk] = tail > 0 ? x1 : -1;
  if (tail > 0 && active) {
    VecT o;
#pragma unroll
    for (int v = 0; v < VEC; ++v) o.v[v] = (T)acc[v];
    *reinterpret_cast<VecT *>(carry_val + (size_t)chunk * (size_t)N + col0) = o;
  }
}

// ---- narrow column tiles: one lane group per row --------------------------------------------
// When a column tile is narrower than a wavefront's 64 lanes can cover with
// full vectors, the wavefront is divided into G = 64 / LPR groups of LPR lanes
// and every group works on a different row of the chunk: group g takes the
// chunk's row slots g, g + G, ... and walks each one's nonzeros itself (up to
// four B-row loads in flight per group, so 4 G per wavefront).  No reduction
// between groups is needed, since a row is summed by one group.  A row with many
// nonzeros in the chunk would leave the other groups idle: such rows are summed
// by all groups together (strided over its nonzeros, then combined with
// shuffles in a fixed order).  Used when a row of B is at most 256 bytes (see
// narrow_tile_bytes).
constexpr int kGroupRowMax = 24;  // longer in-chunk rows are shared by all groups

template <typename T, int VEC, int LPR, int EPI>
__global__ __launch_bounds__(kBlockThreads) void spmm_grouped_kernel(
    int M, int N, const int *__restrict__ row_ptr, const int *__restrict__ col_idx,
    const T *__restrict__ vals, const T *__restrict__ B, T *__restrict__ C,
    const T *__restrict__ bias, int64_t total_items, int items_per_chunk, int snap, int n_tiles,
    int64_t blocks_per_tile, int *__restrict__ carry_row, T *__restrict__ carry_val,
    const Boundary *__restrict__ bounds, SpmmBatch batch) {
  using A = typename Acc<T>::type;
  using VecT = Vec<T, VEC>;
  constexpr int G = kWaveSize / LPR;
  constexpr int kSlots = kItemsPerWave + kSnapItems;
  vals += blockIdx.y * batch.vals;  // problem blockIdx.y of a batch over one pattern
  B += blockIdx.y * batch.b;
  C += blockIdx.y * batch.c;
  carry_val += blockIdx.y * batch.carry;

  __shared__ int s_col[kWavesPerBlock][kSlots];
  __shared__ T s_val[kWavesPerBlock][kSlots];
  __shared__ int s_rp[kWavesPerBlock][kSlots + 2];

  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  const int g = lane / LPR;
  const int t = lane % LPR;
  const TileMap where = map_workgroup(blockIdx.x, n_tiles, blocks_per_tile);
  const int64_t span = where.block * kWavesPerBlock + w;
  const int col0 = (where.tile * LPR + t) * VEC;
  const bool active = col0 < N;

  const int64_t d0 = span * items_per_chunk;
  if (d0 >= total_items) return;  // only wave-level synchronisation below
  const Boundary from = bounds ? load_boundary(bounds, span) : chunk_boundary(d0, M, total_items, row_ptr, snap);
  const Boundary to = bounds ? load_boundary(bounds, span + 1)
                             : chunk_boundary(d0 + items_per_chunk, M, total_items, row_ptr, snap);
  const int x0 = from.x, y0 = from.y, x1 = to.x, y1 = to.y;
  const int n_nz = y1 - y0;
  const int n_rows = x1 - x0;

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
  T bias_v[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) bias_v[v] = (EPI != kEpiNone && active) ? bias[col0 + v] : (T)0;

  auto add_entry = [&](A (&acc)[VEC], int k) {
    const A a = (A)s_val[w][k];
    const VecT b = *reinterpret_cast<const VecT *>(B + (size_t)s_col[w][k] * (size_t)N + col0);
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

    if (active && len <= kGroupRowMax) {
      int k = lo;
      for (; k + 4 <= hi; k += 4) {
        VecT b[4];
        A a[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          a[u] = (A)s_val[w][k + u];
          b[u] = *reinterpret_cast<const VecT *>(B + (size_t)s_col[w][k + u] * (size_t)N + col0);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
          for (int v = 0; v < VEC; ++v) acc[v] += a[u] * (A)b[u].v[v];
      }
      for (; k < hi; ++k) add_entry(acc, k);
    }

    // Rows with many nonzeros in the chunk: one at a time, all groups.
    unsigned long long pending = __ballot(len > kGroupRowMax && t == 0);
    while (pending) {
      const int owner_lane = __ffsll(pending) - 1;  // lane 0 of the owning group
      pending &= pending - 1;
      const int olo = __shfl(lo, owner_lane), ohi = __shfl(hi, owner_lane);
      A part[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) part[v] = (A)0;
      if (active)
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
      VecT o;
      if (slot < n_rows) {
        const bool partial = carry_in && slot == 0;
#pragma unroll
        for (int v = 0; v < VEC; ++v)
          o.v[v] = partial ? (T)acc[v] : apply_epilogue<T, EPI>(acc[v], bias_v[v]);
        store_streaming(C + (size_t)(x0 + slot) * (size_t)N + col0, o);
      } else if (len > 0) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) o.v[v] = (T)acc[v];
        *reinterpret_cast<VecT *>(carry_val + (size_t)span * (size_t)N + col0) = o;
      }
    }
    if (live && slot == n_rows && where.tile == 0 && t == 0 && blockIdx.y == 0) carry_row[span] = len > 0 ? x1 : -1;
  }
}


// ---- host side ----------------------------------------------------------------

// ---- chunk boundaries computed once -----------------------------------------------------------
// The boundaries depend on row_ptr and on the split only, not on the values or
// the dense operand: a caller that multiplies by the same sparse matrix again
// and again (a graph's adjacency in every layer and iteration) computes them once
// with spmm_bounds_kernel, one thread per boundary, and hands them to the
// kernels, whose wavefronts then read two records instead of searching row_ptr
// twice.  bounds[c] is what chunk_boundary returns for position c * items.
__global__ __launch_bounds__(kBlockThreads) void spmm_bounds_kernel(int M, int64_t total_items,
                                                                    int items_per_chunk, int snap,
                                                                    int64_t num_bounds,
                                                                    const int *__restrict__ row_ptr,
                                                                    Boundary *__restrict__ bounds) {
  const int64_t c = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  if (c >= num_bounds) return;
  const int64_t d = c * items_per_chunk;
  Boundary b;
  if (d >= total_items) {
    b.x = M;
    b.y = (int)(total_items - M);
  } else {
    // rows whose end marker (position row_ptr[i + 1] + i) lies before d
    int lo = 0, hi = M;
    while (lo < hi) {
      const int mid = lo + (hi - lo) / 2;
      if ((int64_t)row_ptr[mid + 1] + mid < d) lo = mid + 1; else hi = mid;
    }
    b.x = lo;
    b.y = (int)(d - lo);
    if (b.x < M) {
      const int begin = row_ptr[b.x], end = row_ptr[b.x + 1];
      if (begin < b.y && (int64_t)end + b.x + 1 - d <= snap) {  // as in chunk_boundary
        b.x += 1;
        b.y = end;
      }
    }
  }
  bounds[c] = b;
}

inline size_t spmm_bounds_bytes(int64_t M, int64_t nnz, int64_t N, size_t elem) {
  return (size_t)(spmm_split(M, nnz, N, elem).spans + 1) * sizeof(Boundary);
}

// Optional per-kernel timing: events recorded on the launch stream around each
// of the two kernels.
struct KernelTimer {
  hipEvent_t ev[3] = {nullptr, nullptr, nullptr};
  int init() {
    for (auto &e : ev) SCORCH_HIP_CHECK(hipEventCreate(&e));
    return SCORCH_HIP_OK;
  }
  ~KernelTimer() {
    for (auto &e : ev)
      if (e) (void)hipEventDestroy(e);
  }
};

template <typename T, int VEC, int EPI>
int launch_spmm(int M, int N, int64_t nnz, const int *row_ptr, const int *col_idx, const T *vals,
                const T *B, const T *bias, T *C, void *workspace, hipStream_t stream,
                KernelTimer *timer, const Boundary *bounds, int batch, int64_t K, bool zero_fill = false) {
  const SpmmSplit split = spmm_split(M, nnz, N, sizeof(T));
  const int64_t chunks = split.spans;
  const SpmmBatch strides = {nnz, K * N, (int64_t)M * N, chunks * N};
  int *carry_row = static_cast<int *>(workspace);
  T *carry_val = reinterpret_cast<T *>(
      static_cast<char *>(workspace) +
      align_up((size_t)spmm_num_chunks(M, nnz, N, sizeof(T)) * sizeof(int), 256));
  const int tile = kWaveSize * VEC;
  const int n_tiles = (N + tile - 1) / tile;
  // a multiple of 8 (see map_workgroup); workgroups past the last chunk find nothing to do
  const int64_t blocks_per_tile = round_up_8((chunks + kWavesPerBlock - 1) / kWavesPerBlock);
  if (blocks_per_tile * n_tiles > INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED, "SpMM: %lld workgroups exceed the launch limit",
                (long long)(blocks_per_tile * n_tiles));
  const dim3 grid((unsigned)(blocks_per_tile * n_tiles), (unsigned)batch);
  if (timer) SCORCH_HIP_CHECK(hipEventRecord(timer->ev[0], stream));
  mark_launch(stream);
  zero_fill = zero_fill && EPI == kEpiNone && aligned_to(C, 16) && ((int64_t)batch * M * N * (int64_t)sizeof(T)) % 16 == 0;
  if (zero_fill) {
    const int64_t pieces = (int64_t)batch * M * N * (int64_t)sizeof(T) / 16;
    const int64_t fill_blocks = (pieces + kBlockThreads * 8 - 1) / (kBlockThreads * 8);
    zero_fill_kernel<<<dim3((unsigned)(fill_blocks < 65536 ? fill_blocks : 65536)), kBlockThreads, 0, stream>>>(
        reinterpret_cast<uint4 *>(C), pieces);
    SCORCH_HIP_CHECK(hipGetLastError());
    mark_launch(stream);
  }
  spmm_merge_kernel<T, VEC, EPI><<<grid, kBlockThreads, 0, stream>>>(
      M, N, row_ptr, col_idx, vals, B, C, bias, (int64_t)M + nnz, split.items_per_chunk,
      split.snap, n_tiles, blocks_per_tile, carry_row, carry_val, bounds, strides, zero_fill ? 1 : 0);
  SCORCH_HIP_CHECK(hipGetLastError());
  if (timer) SCORCH_HIP_CHECK(hipEventRecord(timer->ev[1], stream));
  mark_launch(stream);
  const int64_t fix_per_block = kWavesPerBlock * kFixupChunks;
  spmm_fixup_kernel<T, VEC, EPI><<<dim3((unsigned)((chunks + fix_per_block - 1) / fix_per_block), (unsigned)batch),
                                   kBlockThreads, 0, stream>>>(N, chunks, carry_row, carry_val, C, bias, strides);
  SCORCH_HIP_CHECK(hipGetLastError());
  if (timer) SCORCH_HIP_CHECK(hipEventRecord(timer->ev[2], stream));
  mark_launch(stream);
  return SCORCH_HIP_OK;
}

// Narrow-tile variant: lane groups of LPR lanes, tiles of LPR * VEC columns, one
// chunk per wavefront.  The fix-up does not care how the main kernel tiled the
// columns; it runs with scalar lanes over ceil(N / 64) tiles.
template <typename T, int VEC, int LPR, int EPI>
int launch_spmm_grouped(int M, int N, int64_t nnz, const int *row_ptr, const int *col_idx,
                        const T *vals, const T *B, const T *bias, T *C, void *workspace,
                        hipStream_t stream, const Boundary *bounds, int batch, int64_t K) {
  const int64_t total = (int64_t)M + nnz;
  const int tile = LPR * VEC;
  const int n_tiles = (N + tile - 1) / tile;
  // as in spmm_split, with the real tile count: fill 8192 wavefront slots, at most 256 items each
  const int64_t per_wave = total * n_tiles / 8192;
  int ipc = kMinItemsPerWave;
  while (ipc < kItemsPerWave && ipc * 2 <= per_wave) ipc *= 2;
  const int wide_ipc = spmm_split(M, nnz, N, sizeof(T)).items_per_chunk;
  if (ipc < wide_ipc) ipc = wide_ipc;  // never more carry records than the workspace holds
  if (bounds && ipc != wide_ipc)
    return fail(SCORCH_HIP_ERUNTIME, "SpMM: the chunk boundaries were built for %d items per chunk, not %d",
                wide_ipc, ipc);
  const int64_t spans = (total + ipc - 1) / ipc;
  if (spans > spmm_num_chunks(M, nnz, N, sizeof(T)))
    return fail(SCORCH_HIP_ERUNTIME, "SpMM: %lld carry records exceed the workspace's %lld",
                (long long)spans, (long long)spmm_num_chunks(M, nnz, N, sizeof(T)));
  int *carry_row = static_cast<int *>(workspace);
  T *carry_val = reinterpret_cast<T *>(
      static_cast<char *>(workspace) +
      align_up((size_t)spmm_num_chunks(M, nnz, N, sizeof(T)) * sizeof(int), 256));
  const int64_t blocks_per_tile = round_up_8((spans + kWavesPerBlock - 1) / kWavesPerBlock);
  if (blocks_per_tile * n_tiles > INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED, "SpMM: %lld workgroups exceed the launch limit",
                (long long)(blocks_per_tile * n_tiles));
  mark_launch(stream);
  const SpmmBatch strides = {nnz, K * N, (int64_t)M * N, spans * N};
  spmm_grouped_kernel<T, VEC, LPR, EPI><<<dim3((unsigned)(blocks_per_tile * n_tiles), (unsigned)batch), kBlockThreads,
                                          0, stream>>>(
      M, N, row_ptr, col_idx, vals, B, C, bias, total, ipc, ipc < kSnapItems ? ipc : kSnapItems, n_tiles,
      blocks_per_tile, carry_row, carry_val, bounds, strides);
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(stream);
  const int64_t fix_per_block = kWavesPerBlock * kFixupChunks;
  spmm_fixup_kernel<T, 1, EPI><<<dim3((unsigned)((spans + fix_per_block - 1) / fix_per_block), (unsigned)batch),
                                 kBlockThreads, 0, stream>>>(N, spans, carry_row, carry_val, C, bias, strides);
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(stream);
  return SCORCH_HIP_OK;
}

// Narrow tiles pay off when N is small: a row of B is at most 256 bytes, so
// full-width tiles would leave lanes idle or fall back to 4-byte loads.  Returns the tile width in
// bytes, or 0 for wide tiles.  (Tiling a wide B by columns so that K narrow rows
// stay in one XCD's L2 was measured and lost: the workgroups resident on an XCD
// span several tiles at once and evict each other's slices.)
inline int narrow_tile_bytes(int64_t K, int64_t N, int64_t nnz, size_t elem) {
  (void)K; (void)nnz;
  const int64_t row_bytes = N * (int64_t)elem;
  return row_bytes <= 256 ? (int)row_bytes : 0;
}

template <typename T, int EPI>
int spmm_entry(const char *fn, int64_t M, int64_t K, int64_t N, int64_t nnz, const int32_t *row_ptr,
               const int32_t *col_idx, const T *vals, const T *B, const T *bias, T *C,
               void *workspace, size_t workspace_bytes, void *stream,
               KernelTimer *timer = nullptr, const void *bounds_buffer = nullptr, size_t bounds_bytes = 0,
               int64_t batch = 1, bool mostly_empty_rows = false) {
  if (batch < 0 || batch > 65535)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: batch=%lld is outside [0, 65535]", fn, (long long)batch);
  if (batch == 0) return SCORCH_HIP_OK;
  if (int rc = check_csr_args(fn, M, K, nnz, row_ptr, col_idx, vals)) return rc;
  SCORCH_REQUIRE(N >= 0, "%s: negative N=%lld", fn, (long long)N);
  if (N > INT32_MAX - kWaveSize * 4)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: N=%lld is too large", fn, (long long)N);
  if (M == 0 || N == 0) return SCORCH_HIP_OK;  // nothing to write
  SCORCH_REQUIRE(C != nullptr, "%s: C is NULL", fn);
  SCORCH_REQUIRE(K == 0 || B != nullptr, "%s: B is NULL", fn);
  SCORCH_REQUIRE(EPI == kEpiNone || bias != nullptr, "%s: bias is NULL", fn);
  SCORCH_REQUIRE(aligned_to(B, sizeof(T)) && aligned_to(C, sizeof(T)) && aligned_to(vals, sizeof(T)),
                 "%s: value arrays must be aligned to their element size", fn);
  const size_t need = spmm_workspace_bytes(M, nnz, N, sizeof(T));
  if (!workspace || workspace_bytes < need)
    return fail(SCORCH_HIP_EWORKSPACE, "%s: workspace of %zu bytes needed, %zu given", fn, need,
                workspace ? workspace_bytes : (size_t)0);
  SCORCH_REQUIRE(aligned_to(workspace, 256), "%s: workspace must be 256-byte aligned", fn);

  const Boundary *bounds = static_cast<const Boundary *>(bounds_buffer);
  if (bounds) {
    const size_t have = spmm_bounds_bytes(M, nnz, N, sizeof(T));
    if (bounds_bytes < have)
      return fail(SCORCH_HIP_EWORKSPACE, "%s: chunk boundaries of %zu bytes needed, %zu given", fn, have,
                  bounds_bytes);
    SCORCH_REQUIRE(aligned_to(bounds, 8), "%s: the chunk boundaries must be 8-byte aligned", fn);
  }

  hipStream_t s = static_cast<hipStream_t>(stream);
  const int m = (int)M, n = (int)N;
  if (const int tile_bytes = timer ? 0 : narrow_tile_bytes(K, N, nnz, sizeof(T))) {
    // widest vector (at most 16 bytes) that divides N and is aligned; lanes to cover the tile
    constexpr int kMaxVec = (int)(16 / sizeof(T));
    int vec = kMaxVec;
    while (vec > 1 && !(N % vec == 0 && aligned_to(B, sizeof(T) * vec) && aligned_to(C, sizeof(T) * vec)))
      vec /= 2;
    const int64_t tile_elems = tile_bytes / (int)sizeof(T) < N ? tile_bytes / (int)sizeof(T) : N;
    const int64_t lanes = (tile_elems + vec - 1) / vec;
#define SCORCH_GROUPED(VEC, LPR) \
  return launch_spmm_grouped<T, VEC, LPR, EPI>(m, n, nnz, row_ptr, col_idx, vals, B, bias, C, workspace, s, bounds, \
                                               (int)batch, K)
#define SCORCH_GROUPED_LANES(VEC)                      \
  do {                                                 \
    if (lanes <= 8) SCORCH_GROUPED(VEC, 8);            \
    if (lanes <= 16) SCORCH_GROUPED(VEC, 16);          \
    if (lanes <= 32) SCORCH_GROUPED(VEC, 32);          \
  } while (0)
    if constexpr (sizeof(T) == 4) {
      if (vec == 4) SCORCH_GROUPED_LANES(4);
    }
    if (vec == 2) SCORCH_GROUPED_LANES(2);
    if (vec == 1) SCORCH_GROUPED_LANES(1);
#undef SCORCH_GROUPED_LANES
#undef SCORCH_GROUPED
    // more than 32 lanes needed (odd N with scalar lanes): the wide kernel handles it
  }
  const int vec = pick_vec<T>(N, B, C, workspace);
  if constexpr (sizeof(T) == 4) {
    if (vec == 4)
      return launch_spmm<T, 4, EPI>(m, n, nnz, row_ptr, col_idx, vals, B, bias, C, workspace, s, timer, bounds,
                                  (int)batch, K, mostly_empty_rows);
  }
  if (vec == 2)
    return launch_spmm<T, 2, EPI>(m, n, nnz, row_ptr, col_idx, vals, B, bias, C, workspace, s, timer, bounds,
                                  (int)batch, K, mostly_empty_rows);
  return launch_spmm<T, 1, EPI>(m, n, nnz, row_ptr, col_idx, vals, B, bias, C, workspace, s, timer, bounds,
                                  (int)batch, K, mostly_empty_rows);
}


// ---- SpMV: the same merge-path split with one output column ------------------------------
// A wavefront owns kSpmvItems consecutive items of the merged (row ends + nonzeros)
// sequence.  Its lanes first form all products val * x[col] in parallel (coalesced
// reads of col_idx / vals, gathered reads of x) and park them in LDS; then lane r
// sums the products of the r-th row the chunk touches.  A row with many entries
// in the chunk is summed by the whole wavefront instead (strided partial sums,
// butterfly reduction).  The part of the last row that continues in the next
// chunk becomes a carry, folded into y by spmv_fixup_kernel in a fixed order,
// so results are bit-reproducible.
constexpr int kSpmvItems = 512;
// large matrices take chunks twice the size: 16 loads per lane in flight instead of 8, half
// the chunks to start and to fix up (0.124 -> 0.117 ms on a 17 M-nonzero graph); smaller
// ones need the wavefronts more
constexpr int kSpmvItemsLarge = 1024;
constexpr int64_t kSpmvLargeFrom = 4 << 20;  // merged items
constexpr int kSpmvLaneRowMax = 32;  // longer in-chunk rows are summed by the whole wavefront

template <typename T, int ITEMS>
__global__ __launch_bounds__(kBlockThreads) void spmv_merge_kernel(
    int M, const int *__restrict__ row_ptr, const int *__restrict__ col_idx,
    const T *__restrict__ vals, const T *__restrict__ x, T *__restrict__ y, int64_t total_items,
    int *__restrict__ carry_row, T *__restrict__ carry_val) {
  using A = typename Acc<T>::type;
  __shared__ A s_prod[kWavesPerBlock][ITEMS];
  __shared__ int s_rp[kWavesPerBlock][ITEMS + 2];

  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  // the grid is a multiple of 8 workgroups; every XCD takes a contiguous eighth of the spans
  const int64_t span = xcd_contiguous(blockIdx.x, gridDim.x) * kWavesPerBlock + w;
  int64_t d0 = span * ITEMS;
  if (d0 >= total_items) return;  // nothing here uses workgroup barriers
  int64_t d1 = d0 + ITEMS;
  d1 = d1 < total_items ? d1 : total_items;

  auto row_end_key = [&](int i) { return (int64_t)row_ptr[i + 1] + i; };
  const int x0 = wave_count_below(M, d0, row_end_key);
  const int y0 = uniform((int)(d0 - x0));

  // Everything the chunk can touch is known from its start alone: at most
  // ITEMS nonzeros from y0 and ITEMS + 1 row pointers from x0.  All
  // of it is requested at once (one round trip for indices, values and row
  // pointers, one for the gathered x), and the chunk's end is then found in LDS.
  constexpr int kNzLoads = ITEMS / kWaveSize;
  constexpr int kRpLoads = (ITEMS + 2 + kWaveSize - 1) / kWaveSize;
  const int64_t nnz = total_items - M;
  int col[kNzLoads];
  T val[kNzLoads];
  // (a chunk that lies inside the arrays reads them at constant offsets from a scalar base:
  // no address arithmetic and no bounds checks per element)
  const bool inside = (int64_t)y0 + ITEMS <= nnz;
  if (inside) {
    const int *c0 = col_idx + y0;
    const T *v0 = vals + y0;
#pragma unroll
    for (int u = 0; u < kNzLoads; ++u) {
      col[u] = c0[lane + u * kWaveSize];
      val[u] = v0[lane + u * kWaveSize];
    }
  } else {
#pragma unroll
    for (int u = 0; u < kNzLoads; ++u) {
      const int64_t p = (int64_t)y0 + lane + u * kWaveSize;
      const bool ok = p < nnz;
      col[u] = ok ? col_idx[p] : -1;
      val[u] = ok ? vals[p] : (T)0;
    }
  }
  int rp[kRpLoads];
  if ((int64_t)x0 + kRpLoads * kWaveSize <= M) {
    const int *r0 = row_ptr + x0;
#pragma unroll
    for (int u = 0; u < kRpLoads; ++u) rp[u] = r0[lane + u * kWaveSize];
  } else {
#pragma unroll
    for (int u = 0; u < kRpLoads; ++u) {
      const int64_t r = (int64_t)x0 + lane + u * kWaveSize;
      rp[u] = row_ptr[r < M ? r : M];
    }
  }
  if (inside) {
#pragma unroll
    for (int u = 0; u < kNzLoads; ++u) s_prod[w][lane + u * kWaveSize] = (A)val[u] * (A)x[col[u]];
  } else {
#pragma unroll
    for (int u = 0; u < kNzLoads; ++u) {
      const A xv = col[u] >= 0 ? (A)x[col[u]] : (A)0;
      s_prod[w][lane + u * kWaveSize] = (A)val[u] * xv;
    }
  }
#pragma unroll
  for (int u = 0; u < kRpLoads; ++u)
    if (lane + u * kWaveSize < ITEMS + 2) s_rp[w][lane + u * kWaveSize] = rp[u];
  wave_lds_sync();

  // rows ending inside the chunk: row x0 + j ends at merged position s_rp[j + 1] + x0 + j,
  // and no row from x0 + ITEMS on can end before d1
  const int reach = M - x0 < ITEMS ? M - x0 : ITEMS;
  const int n_rows = wave_count_below(reach, d1, [&](int j) { return (int64_t)s_rp[w][j + 1] + x0 + j; });
  const int x1 = x0 + n_rows;
  const int y1 = uniform((int)(d1 - x1));

  // Row slot r is row x0 + r; slot n_rows is the row that continues past the chunk.
  for (int base = 0; base <= n_rows; base += kWaveSize) {
    const int r = base + lane;
    const bool live = r <= n_rows;
    int lo = 0, hi = 0;
    if (live) {
      const int begin = s_rp[w][r], end = s_rp[w][r + 1];
      lo = (begin > y0 ? begin : y0) - y0;
      hi = (end < y1 ? end : y1) - y0;
      if (hi < lo) hi = lo;
    }
    const int len = hi - lo;
    A sum = (A)0;
    if (len <= kSpmvLaneRowMax)
      for (int k = lo; k < hi; ++k) sum += s_prod[w][k];
    // rows with many entries in the chunk: one at a time, all lanes
    unsigned long long pending = __ballot(len > kSpmvLaneRowMax);
    while (pending) {
      const int owner = __ffsll(pending) - 1;
      pending &= pending - 1;
      const int olo = __shfl(lo, owner), ohi = __shfl(hi, owner);
      A part = (A)0;
      for (int k = olo + lane; k < ohi; k += kWaveSize) part += s_prod[w][k];
#pragma unroll
      for (int off = kWaveSize / 2; off > 0; off >>= 1) part += (A)__shfl_xor((T)part, off);
      if (lane == owner) sum = part;
    }
    if (live) {
      if (r < n_rows) {
        y[x0 + r] = (T)sum;
      } else {
        carry_row[span] = len > 0 ? x1 : -1;
        if (len > 0) carry_val[span] = (T)sum;
      }
    }
  }
}

// The carries of SpMV are single values, so a wavefront per chunk (spmm_fixup_kernel)
// would leave 63 lanes idle.  Here a thread looks at one chunk: if it heads a run
// of equal carry rows it adds the run, in chunk order, to y.  Runs of more than
// kSpmvShortRun carries (a row spread over that many wavefronts) are then taken
// one after the other by the whole wavefront: lane l sums members l, l + 64, ...
// and the lanes' sums are combined in a fixed order.  Same result on every run.
constexpr int kSpmvShortRun = 32;

template <typename T>
__global__ __launch_bounds__(kBlockThreads) void spmv_fixup_kernel(int64_t spans,
                                                                   const int *__restrict__ carry_row,
                                                                   const T *__restrict__ carry_val,
                                                                   T *__restrict__ y) {
  using A = typename Acc<T>::type;
  const int lane = wave_lane();
  const int64_t c = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  int row = -1;
  bool long_run = false;
  if (c < spans) {
    // everything the usual case needs (a run of one) is requested at once
    row = carry_row[c];
    const int before = c > 0 ? carry_row[c - 1] : -1;
    const int after = c + 1 < spans ? carry_row[c + 1] : -1;
    A sum = (A)carry_val[c];
    if (row >= 0 && before == row) row = -1;  // not the head of its run
    if (row >= 0) {
      if (after == row) {
        int64_t e = c + 1;
        for (; e < spans && e < c + kSpmvShortRun && carry_row[e] == row; ++e) sum += (A)carry_val[e];
        long_run = e == c + kSpmvShortRun && e < spans && carry_row[e] == row;
      }
      if (!long_run) y[row] = (T)(sum + (A)y[row]);
    }
  }
  unsigned long long pending = __ballot(long_run);
  while (pending) {  // uniform over the wavefront
    const int owner = __ffsll(pending) - 1;
    pending &= pending - 1;
    const int64_t start = c - lane + owner;
    const int r = __shfl(row, owner);
    const int64_t end = carry_run_end(carry_row, start, spans, r);
    A part = (A)0;
    for (int64_t e = start + lane; e < end; e += kWaveSize) part += (A)carry_val[e];
#pragma unroll
    for (int off = kWaveSize / 2; off > 0; off >>= 1) part += (A)__shfl_xor((T)part, off);
    if (lane == owner) y[r] = (T)(part + (A)y[r]);
  }
}

// (the most spans a call can use: the workspace is sized by it)
inline int64_t spmv_num_spans(int64_t M, int64_t nnz) {
  return (M + nnz + kSpmvItems - 1) / kSpmvItems;
}

inline size_t spmv_workspace_bytes(int64_t M, int64_t nnz, size_t elem) {
  const size_t spans = (size_t)spmv_num_spans(M, nnz);
  return align_up(spans * sizeof(int), 256) + align_up(spans * elem, 256);
}

template <typename T>
int spmv_entry(const char *fn, int64_t M, int64_t K, int64_t nnz, const int32_t *row_ptr,
               const int32_t *col_idx, const T *vals, const T *x, T *y, void *workspace,
               size_t workspace_bytes, void *stream) {
  if (int rc = check_csr_args(fn, M, K, nnz, row_ptr, col_idx, vals)) return rc;
  if (M == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(y != nullptr, "%s: y is NULL", fn);
  SCORCH_REQUIRE(K == 0 || x != nullptr, "%s: x is NULL", fn);
  SCORCH_REQUIRE(aligned_to(x, sizeof(T)) && aligned_to(y, sizeof(T)) && aligned_to(vals, sizeof(T)),
                 "%s: value arrays must be aligned to their element size", fn);
  const size_t need = spmv_workspace_bytes(M, nnz, sizeof(T));
  if (!workspace || workspace_bytes < need)
    return fail(SCORCH_HIP_EWORKSPACE, "%s: workspace of %zu bytes needed, %zu given", fn, need,
                workspace ? workspace_bytes : (size_t)0);
  SCORCH_REQUIRE(aligned_to(workspace, 256), "%s: workspace must be 256-byte aligned", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool large = M + nnz >= kSpmvLargeFrom;
  const int64_t items_per_span = large ? kSpmvItemsLarge : kSpmvItems;
  const int64_t spans = (M + nnz + items_per_span - 1) / items_per_span;
  int *carry_row = static_cast<int *>(workspace);
  T *carry_val = reinterpret_cast<T *>(static_cast<char *>(workspace) +
                                       align_up((size_t)spans * sizeof(int), 256));
  const int64_t blocks = round_up_8((spans + kWavesPerBlock - 1) / kWavesPerBlock);
  if (large)
    spmv_merge_kernel<T, kSpmvItemsLarge><<<dim3((unsigned)blocks), kBlockThreads, 0, s>>>(
        (int)M, row_ptr, col_idx, vals, x, y, M + nnz, carry_row, carry_val);
  else
    spmv_merge_kernel<T, kSpmvItems><<<dim3((unsigned)blocks), kBlockThreads, 0, s>>>(
        (int)M, row_ptr, col_idx, vals, x, y, M + nnz, carry_row, carry_val);
  SCORCH_HIP_CHECK(hipGetLastError());
  spmv_fixup_kernel<T><<<dim3((unsigned)((spans + kBlockThreads - 1) / kBlockThreads)), kBlockThreads, 0, s>>>(
      spans, carry_row, carry_val, y);
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

// ---- the entry point that allocates nothing --------------------------------------------------
// Scratch for scorch_hip_spmm_csr_f32_static: the carry records that the other
// entry points keep in the caller's workspace live in this array instead.  Every
// GPU the library runs on holds its own copy, at its own address, until the
// process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels are given the address that call returns.
constexpr size_t kStaticScratchBytes = SCORCH_HIP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];  // per device, filled on the first call there
static std::mutex g_scratch_mutex;

// Address of the current device's copy of `scratch`.
static int static_scratch(const char *fn, void **out) {
  int device = -1;
  SCORCH_HIP_CHECK(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: device ordinal %d is beyond the %d this library tracks", fn,
                device, kMaxDevices);
  std::lock_guard<std::mutex> guard(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    void *ptr = nullptr;
    SCORCH_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fail(SCORCH_HIP_ERUNTIME, "%s: hipGetSymbolAddress returned a null address", fn);
    g_scratch_ptr[device] = ptr;
  }
  *out = g_scratch_ptr[device];
  return SCORCH_HIP_OK;
}

}  // namespace scorch

extern "C" {

size_t scorch_hip_spmm_csr_workspace_bytes(int64_t M, int64_t nnz, int64_t N, size_t elem_size) {
  if (M < 0 || nnz < 0 || N < 0 || elem_size == 0) return 0;
  return scorch::spmm_workspace_bytes(M, nnz, N, elem_size);
}

#define SCORCH_DEFINE_SPMM(SUFFIX, T)                                                            \
  int scorch_hip_spmm_csr_##SUFFIX(int64_t M, int64_t K, int64_t N, int64_t nnz,                 \
                                   const int32_t *row_ptr, const int32_t *col_idx, const T *vals, \
                                   const T *B, T *C, void *workspace, size_t workspace_bytes,    \
                                   void *stream) {                                               \
    return scorch::spmm_entry<T, scorch::kEpiNone>("scorch_hip_spmm_csr_" #SUFFIX, M, K, N, nnz, \
                                                   row_ptr, col_idx, vals, B, nullptr, C,        \
                                                   workspace, workspace_bytes, stream);          \
  }

SCORCH_DEFINE_SPMM(f32, float)
SCORCH_DEFINE_SPMM(f64, double)
SCORCH_DEFINE_SPMM(i32, int32_t)
SCORCH_DEFINE_SPMM(i64, int64_t)

size_t scorch_hip_spmv_csr_workspace_bytes(int64_t M, int64_t nnz, size_t elem_size) {
  if (M < 0 || nnz < 0 || elem_size == 0) return 0;
  return scorch::spmv_workspace_bytes(M, nnz, elem_size);
}

#define SCORCH_DEFINE_SPMV(SUFFIX, T)                                                           \
  int scorch_hip_spmv_csr_##SUFFIX(int64_t M, int64_t K, int64_t nnz, const int32_t *row_ptr,   \
                                   const int32_t *col_idx, const T *vals, const T *x, T *y,     \
                                   void *workspace, size_t workspace_bytes, void *stream) {     \
    return scorch::spmv_entry<T>("scorch_hip_spmv_csr_" #SUFFIX, M, K, nnz, row_ptr, col_idx,   \
                                 vals, x, y, workspace, workspace_bytes, stream);               \
  }

SCORCH_DEFINE_SPMV(f32, float)
SCORCH_DEFINE_SPMV(f64, double)
SCORCH_DEFINE_SPMV(i32, int32_t)
SCORCH_DEFINE_SPMV(i64, int64_t)

int scorch_hip_spmm_csr_f32_timed(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                  const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                                  const float *B, float *C, void *workspace,
                                  size_t workspace_bytes, void *stream, float *kernel_ms) {
  const char *fn = "scorch_hip_spmm_csr_f32_timed";
  SCORCH_REQUIRE(kernel_ms != nullptr, "%s: kernel_ms is NULL", fn);
  kernel_ms[0] = kernel_ms[1] = 0.0f;
  if (M == 0 || N == 0)
    return scorch::spmm_entry<float, scorch::kEpiNone>(fn, M, K, N, nnz, row_ptr, col_idx, vals, B,
                                                       nullptr, C, workspace, workspace_bytes, stream);
  scorch::KernelTimer timer;
  if (int rc = timer.init()) return rc;
  if (int rc = scorch::spmm_entry<float, scorch::kEpiNone>(fn, M, K, N, nnz, row_ptr, col_idx, vals,
                                                           B, nullptr, C, workspace,
                                                           workspace_bytes, stream, &timer))
    return rc;
  SCORCH_HIP_CHECK(hipEventSynchronize(timer.ev[2]));
  SCORCH_HIP_CHECK(hipEventElapsedTime(&kernel_ms[0], timer.ev[0], timer.ev[1]));
  SCORCH_HIP_CHECK(hipEventElapsedTime(&kernel_ms[1], timer.ev[1], timer.ev[2]));
  return SCORCH_HIP_OK;
}

int scorch_hip_spmm_csr_bias_act_f32(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                     const int32_t *row_ptr, const int32_t *col_idx,
                                     const float *vals, const float *B, const float *bias, int act,
                                     float *C, void *workspace, size_t workspace_bytes,
                                     void *stream) {
  const char *fn = "scorch_hip_spmm_csr_bias_act_f32";
  if (act == SCORCH_HIP_ACT_NONE)
    return scorch::spmm_entry<float, scorch::kEpiBias>(fn, M, K, N, nnz, row_ptr, col_idx, vals, B,
                                                       bias, C, workspace, workspace_bytes, stream);
  if (act == SCORCH_HIP_ACT_RELU)
    return scorch::spmm_entry<float, scorch::kEpiBiasRelu>(fn, M, K, N, nnz, row_ptr, col_idx, vals,
                                                           B, bias, C, workspace, workspace_bytes,
                                                           stream);
  return scorch::fail(SCORCH_HIP_EINVAL, "%s: unknown activation %d", fn, act);
}

size_t scorch_hip_spmm_csr_bounds_bytes(int64_t M, int64_t nnz, int64_t N, size_t elem_size) {
  if (M < 0 || nnz < 0 || N < 0 || elem_size == 0) return 0;
  return scorch::spmm_bounds_bytes(M, nnz, N, elem_size);
}

int scorch_hip_spmm_csr_bounds(int64_t M, int64_t nnz, int64_t N, size_t elem_size, const int32_t *row_ptr,
                               void *bounds, size_t bounds_bytes, void *stream) {
  const char *fn = "scorch_hip_spmm_csr_bounds";
  if (M < 0 || nnz < 0 || N < 0 || elem_size == 0)
    return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size (M=%lld nnz=%lld N=%lld)", fn, (long long)M,
                        (long long)nnz, (long long)N);
  if (M >= INT32_MAX || nnz > INT32_MAX)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: M and nnz must fit the int32 index arrays", fn);
  SCORCH_REQUIRE(row_ptr != nullptr && bounds != nullptr, "%s: row_ptr or bounds is NULL", fn);
  SCORCH_REQUIRE(scorch::aligned_to(row_ptr, 4) && scorch::aligned_to(bounds, 8),
                 "%s: row_ptr must be 4-byte and bounds 8-byte aligned", fn);
  const size_t need = scorch::spmm_bounds_bytes(M, nnz, N, elem_size);
  if (bounds_bytes < need)
    return scorch::fail(SCORCH_HIP_EWORKSPACE, "%s: %zu bytes needed for the boundaries, %zu given", fn, need,
                        bounds_bytes);
  const scorch::SpmmSplit split = scorch::spmm_split(M, nnz, N, elem_size);
  const int64_t num_bounds = split.spans + 1;
  scorch::spmm_bounds_kernel<<<dim3((unsigned)((num_bounds + scorch::kBlockThreads - 1) / scorch::kBlockThreads)),
                               scorch::kBlockThreads, 0, static_cast<hipStream_t>(stream)>>>(
      (int)M, M + nnz, split.items_per_chunk, split.snap, num_bounds, row_ptr,
      static_cast<scorch::Boundary *>(bounds));
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

#define SCORCH_DEFINE_SPMM_PLANNED(SUFFIX, T)                                                              \
  int scorch_hip_spmm_csr_planned_##SUFFIX(int64_t M, int64_t K, int64_t N, int64_t nnz,                    \
                                           const int32_t *row_ptr, const int32_t *col_idx, const T *vals,   \
                                           const T *B, const T *bias, int act, T *C, const void *bounds,    \
                                           size_t bounds_bytes, void *workspace, size_t workspace_bytes,    \
                                           void *stream) {                                                  \
    const char *fn = "scorch_hip_spmm_csr_planned_" #SUFFIX;                                                \
    const bool mostly_empty = (act & SCORCH_HIP_HINT_MOSTLY_EMPTY_ROWS) != 0;                               \
    act &= ~SCORCH_HIP_HINT_MOSTLY_EMPTY_ROWS;                                                              \
    if (!bias && act == SCORCH_HIP_ACT_NONE)                                                                \
      return scorch::spmm_entry<T, scorch::kEpiNone>(fn, M, K, N, nnz, row_ptr, col_idx, vals, B, nullptr,  \
                                                     C, workspace, workspace_bytes, stream, nullptr,        \
                                                     bounds, bounds_bytes, 1, mostly_empty);                \
    if (bias && act == SCORCH_HIP_ACT_NONE)                                                                 \
      return scorch::spmm_entry<T, scorch::kEpiBias>(fn, M, K, N, nnz, row_ptr, col_idx, vals, B, bias, C,  \
                                                     workspace, workspace_bytes, stream, nullptr, bounds,   \
                                                     bounds_bytes);                                         \
    if (bias && act == SCORCH_HIP_ACT_RELU)                                                                 \
      return scorch::spmm_entry<T, scorch::kEpiBiasRelu>(fn, M, K, N, nnz, row_ptr, col_idx, vals, B, bias, \
                                                         C, workspace, workspace_bytes, stream, nullptr,    \
                                                         bounds, bounds_bytes);                             \
    return scorch::fail(SCORCH_HIP_EINVAL, "%s: activation %d (with%s bias) is not supported", fn, act,     \
                        bias ? "" : "out");                                                                 \
  }

SCORCH_DEFINE_SPMM_PLANNED(f32, float)
SCORCH_DEFINE_SPMM_PLANNED(f64, double)
SCORCH_DEFINE_SPMM_PLANNED(i32, int32_t)
SCORCH_DEFINE_SPMM_PLANNED(i64, int64_t)

size_t scorch_hip_spmm_csr_batched_workspace_bytes(int64_t batch, int64_t M, int64_t nnz, int64_t N) {
  if (batch <= 0 || M < 0 || nnz < 0 || N < 0) return 0;
  return scorch::spmm_batched_workspace_bytes(batch, M, nnz, N, sizeof(float));
}

int scorch_hip_spmm_csr_batched_f32(int64_t batch, int64_t M, int64_t K, int64_t N, int64_t nnz,
                                    const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                                    const float *B, float *C, const void *bounds, size_t bounds_bytes,
                                    void *workspace, size_t workspace_bytes, void *stream) {
  return scorch::spmm_entry<float, scorch::kEpiNone>("scorch_hip_spmm_csr_batched_f32", M, K, N, nnz, row_ptr,
                                                     col_idx, vals, B, nullptr, C, workspace, workspace_bytes,
                                                     stream, nullptr, bounds, bounds_bytes, batch);
}

int scorch_hip_spmm_csr_f32_static(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                   const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                                   const float *B, float *C, void *stream) {
  const char *fn = "scorch_hip_spmm_csr_f32_static";
  if (M < 0 || K < 0 || N < 0 || nnz < 0)
    return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size (M=%lld K=%lld N=%lld nnz=%lld)", fn,
                        (long long)M, (long long)K, (long long)N, (long long)nnz);
  const size_t need = scorch::spmm_workspace_bytes(M, nnz, N, sizeof(float));
  if (need > scorch::kStaticScratchBytes)
    return scorch::fail(SCORCH_HIP_EWORKSPACE,
                        "%s: this shape needs %zu bytes of scratch, the library's static buffer holds %zu; "
                        "use scorch_hip_spmm_csr_f32 with a workspace of the caller's",
                        fn, need, scorch::kStaticScratchBytes);
  void *ws = nullptr;
  if (M > 0 && N > 0)
    if (int rc = scorch::static_scratch(fn, &ws)) return rc;
  // nothing in the scratch has to start at zero: every chunk writes its carry row, and a carry
  // value is read only where the carry row written in the same launch says there is one
  return scorch::spmm_entry<float, scorch::kEpiNone>(fn, M, K, N, nnz, row_ptr, col_idx, vals, B, nullptr, C,
                                                     ws ? ws : (void *)nullptr,
                                                     scorch::kStaticScratchBytes, stream);
}

}  // extern "C"

SCORCH_DEFINE_PRELOAD(spmm)
