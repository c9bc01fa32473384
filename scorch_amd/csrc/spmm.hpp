// Pieces shared by the SpMM kernels of libscorch_hip.so: the merge-path work
// split (spmm.hip), the row-split kernel for short rows (spmm_rows.hip) and the
// kernel for a dense operand stored by column tiles (spmm_tiled.hip).
#pragma once

#include "common.hpp"

namespace scorch {

constexpr int kItemsPerWave = 256;  // most merge items (row ends + nonzeros) per wavefront
constexpr int kMinItemsPerWave = 32;
constexpr int kGather = 8;          // B-row loads in flight per wavefront

enum Epilogue { kEpiNone = 0, kEpiBias = 1, kEpiBiasRelu = 2 };

// Workgroup id -> (column tile, block of wavefront spans).  Workgroups are dealt
// to the 8 XCDs round robin by their linear id, and every XCD has its own L2.
// With a multiple of 8 column tiles, tile t is given to XCD t % 8 and each XCD
// works through its tiles one after the other: the B rows a tile gathers
// (K rows of 64 * VEC elements) are then fetched into one L2 only and stay
// there while the tile is processed.
struct TileMap {
  int tile;
  int64_t block;
};

__device__ __forceinline__ TileMap map_workgroup(int64_t id, int n_tiles, int64_t blocks_per_tile) {
  TileMap m;
  if (n_tiles > 1 && (n_tiles & 7) == 0) {
    const int xcd = (int)(id & 7);
    const int64_t slot = id >> 3;
    m.tile = xcd + 8 * (int)(slot / blocks_per_tile);
    m.block = slot % blocks_per_tile;
  } else {
    m.tile = (int)(id / blocks_per_tile);
    const int64_t rem = id % blocks_per_tile;
    // rem & 7 is the XCD when blocks_per_tile is a multiple of 8 (the SpMM launchers
    // see to that): every XCD gets one contiguous eighth of the chunks, so that B
    // rows shared by neighbouring rows of A are found in its L2
    m.block = (blocks_per_tile & 7) == 0 ? xcd_contiguous(rem, blocks_per_tile) : rem;
  }
  return m;
}

template <typename T, int EPI>
__device__ __forceinline__ T apply_epilogue(typename Acc<T>::type acc, T bias) {
  T r = (T)acc;
  if (EPI != kEpiNone) r = r + bias;
  if (EPI == kEpiBiasRelu) r = r > (T)0 ? r : (T)0;
  return r;
}

// Chunk boundaries.  Chunk c nominally covers the merged positions [c * items,
// (c + 1) * items).  A boundary that falls inside a row moves forward to just
// after the row's end marker when that is at most `snap` items away: the row
// is then summed by one chunk and leaves no carry.  Most rows are short, so
// most boundaries snap, and carries remain for rows that really span chunks.
// The result depends on the nominal position only, so the two chunks on either
// side of a boundary agree on it.  x: rows finished before the boundary, y:
// nonzeros before it.
constexpr int kSnapItems = 64;

struct Boundary {
  int x, y;
};

__device__ __forceinline__ Boundary chunk_boundary(int64_t d, int M, int64_t total_items,
                                                   const int *__restrict__ row_ptr, int snap) {
  Boundary b;
  if (d >= total_items) {
    b.x = M;
    b.y = (int)(total_items - M);
    return b;
  }
  auto row_end_key = [&](int i) { return (int64_t)row_ptr[i + 1] + i; };
  b.x = wave_count_below(M, d, row_end_key);
  b.y = uniform((int)(d - b.x));
  if (b.x < M) {
    const int begin = uniform(row_ptr[b.x]), end = uniform(row_ptr[b.x + 1]);
    const int64_t after_marker = (int64_t)end + b.x + 1;
    if (begin < b.y && after_marker - d <= snap) {  // the row is under way and nearly done
      b.x += 1;
      b.y = end;
    }
  }
  return b;
}

// A boundary computed beforehand (spmm_bounds_kernel): record c of `bounds`.
__device__ __forceinline__ Boundary load_boundary(const Boundary *__restrict__ bounds, int64_t c) {
  const int2 raw = *reinterpret_cast<const int2 *>(bounds + c);
  Boundary b;
  b.x = uniform(raw.x);
  b.y = uniform(raw.y);
  return b;
}

// Several products over one sparsity pattern in one launch (grid.y = problem; one per
// attention head): how far apart, in elements, the problems' value arrays, dense operands,
// results and carry rows lie.  All zero for a single product.
struct SpmmBatch {
  int64_t vals, b, c, carry;
};

// Shape of the work split.  A chunk holds nominally up to 256 merge items, one
// chunk per wavefront; small problems use smaller chunks, so that they are
// spread over more, shorter wavefronts.  (A wavefront that walked two or more
// consecutive chunks with one carry for all of them was measured: the same
// time on a graph with uniform neighbours, slower -- 0.81 against 0.69 ms on the
// 4,096-neighbour graph -- where neighbouring rows share columns, because an XCD
// then has a wider stretch of rows in flight than its L2 covers.)
struct SpmmSplit {
  int items_per_chunk;
  int snap;        // see chunk_boundary
  int64_t spans;   // chunks = wavefronts with work = carry records
};

inline SpmmSplit spmm_split(int64_t M, int64_t nnz, int64_t N, size_t elem) {
  const int64_t total = M + nnz;
  SpmmSplit sp;
  // every column tile (up to 1 KiB of a row) walks all chunks again
  const int64_t tiles = (N * (int64_t)elem + 1023) / 1024;
  const int64_t per_wave = total * (tiles > 0 ? tiles : 1) / 8192;  // 256 CUs x 32 wavefronts
  sp.items_per_chunk = kMinItemsPerWave;
  while (sp.items_per_chunk < kItemsPerWave && sp.items_per_chunk * 2 <= per_wave)
    sp.items_per_chunk *= 2;
  sp.snap = sp.items_per_chunk < kSnapItems ? sp.items_per_chunk : kSnapItems;
  sp.spans = (total + sp.items_per_chunk - 1) / sp.items_per_chunk;
  return sp;
}

// Carry records the workspace must hold: the most any kernel variant produces
// for this shape (one record per chunk of the wide-tile split).
inline int64_t spmm_num_chunks(int64_t M, int64_t nnz, int64_t N, size_t elem) {
  const SpmmSplit sp = spmm_split(M, nnz, N, elem);
  return (M + nnz + sp.items_per_chunk - 1) / sp.items_per_chunk;
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Workspace layout: carry_row int32[num_chunks] padded to 256 bytes, then
// carry_val T[num_chunks * N] padded likewise.
inline size_t spmm_workspace_bytes(int64_t M, int64_t nnz, int64_t N, size_t elem) {
  const size_t chunks = (size_t)spmm_num_chunks(M, nnz, N, elem);
  return align_up(chunks * sizeof(int), 256) + align_up(chunks * (size_t)N * elem, 256);
}

// A batch of products over one pattern: one carry_row array, then carry_val for every problem.
inline size_t spmm_batched_workspace_bytes(int64_t batch, int64_t M, int64_t nnz, int64_t N, size_t elem) {
  const size_t chunks = (size_t)spmm_num_chunks(M, nnz, N, elem);
  return align_up(chunks * sizeof(int), 256) + align_up((size_t)batch * chunks * (size_t)N * elem, 256);
}

// Elements per lane.  Preferred: the widest vector (at most 16 bytes) that
// divides N, is aligned and still keeps all 64 lanes busy (64 * VEC <= N).
// Narrow N: the narrowest vector that covers N with one column tile.
template <typename T>
int pick_vec(int64_t N, const void *B, const void *C, const void *ws) {
  constexpr int kMaxVec = (int)(16 / sizeof(T));
  auto usable = [&](int vec) {
    const size_t bytes = sizeof(T) * vec;
    return N % vec == 0 && aligned_to(B, bytes) && aligned_to(C, bytes) && aligned_to(ws, bytes);
  };
  for (int vec = kMaxVec; vec > 1; vec /= 2)
    if (usable(vec) && (int64_t)kWaveSize * vec <= N) return vec;
  for (int vec = 2; vec <= kMaxVec; vec *= 2)
    if (usable(vec) && (int64_t)kWaveSize * vec >= N && (int64_t)kWaveSize * (vec / 2) < N) return vec;
  return 1;
}

// End of the run of equal carry rows that starts at `start` (a member): a 64-way
// search by the whole wavefront.  The members of a run are consecutive, so
// "same row" holds up to the end and nowhere after.
__device__ __forceinline__ int64_t carry_run_end(const int *__restrict__ carry_row, int64_t start,
                                                 int64_t num_chunks, int row) {
  const int lane = wave_lane();
  int64_t last = start, stop = num_chunks;  // a known member; the first position known to lie beyond
  while (stop - last > 1) {
    const int64_t step = (stop - last + kWaveSize) / (kWaveSize + 1);
    const int64_t probe = last + (int64_t)(lane + 1) * step;
    const bool same = probe < stop && carry_row[probe] == row;
    const int members = __popcll(__ballot(same));  // lanes 0 .. members - 1
    const int64_t reached = last + (int64_t)members * step;
    if (members < kWaveSize && reached + step < stop) stop = reached + step;  // lane `members` saw the end
    last = reached;
  }
  return last + 1;
}

// Folds the carries into C.  A wavefront looks at kFixupChunks consecutive
// chunks' carry rows (one lane each, one load); those that head a run of equal
// rows are then taken one after the other by the whole wavefront, lanes on
// columns: the run is summed in chunk order and added to the row of C, with
// the epilogue.  Few chunks leave a carry (see chunk_boundary), so most
// wavefronts only look: fewer, wider-looking wavefronts cost less to start,
// while a matrix of long rows, where every chunk leaves a carry, still has
// its heads spread over many wavefronts.
constexpr int kFixupChunks = 8;
template <typename T, int VEC, int EPI>
__global__ __launch_bounds__(kBlockThreads) void spmm_fixup_kernel(
    int N, int64_t num_chunks, const int *__restrict__ carry_row, const T *__restrict__ carry_val,
    T *__restrict__ C, const T *__restrict__ bias, SpmmBatch batch) {
  using A = typename Acc<T>::type;
  using VecT = Vec<T, VEC>;
  carry_val += blockIdx.y * batch.carry;
  C += blockIdx.y * batch.c;
  const int lane = wave_lane();
  const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWaveSize;
  const int64_t c = wave * kFixupChunks + lane;
  int row = -1, after = -1;
  if (lane < kFixupChunks && c < num_chunks) {
    row = carry_row[c];
    after = c + 1 < num_chunks ? carry_row[c + 1] : -1;
    if (row >= 0 && c > 0 && carry_row[c - 1] == row) row = -1;  // not the head of its run
  }
  unsigned long long pending = __ballot(row >= 0);
  while (pending) {  // uniform over the wavefront
    const int owner = __ffsll(pending) - 1;
    pending &= pending - 1;
    const int r = __shfl(row, owner);
    const int64_t start = c - lane + owner;
    // a run of one, the usual case, needs no search
    const int64_t end = __shfl(after, owner) != r ? start + 1 : carry_run_end(carry_row, start, num_chunks, r);
    for (int col0 = lane * VEC; col0 < N; col0 += kWaveSize * VEC) {
      VecT *dst = reinterpret_cast<VecT *>(C + (size_t)r * (size_t)N + col0);
      VecT o = *dst;  // issued before the carries so that both are in flight together
      A sum[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) sum[v] = (A)0;
      int64_t e = start;
      constexpr int kBatch = 32;  // loads in flight: a long row spans hundreds of chunks
      for (; e + kBatch <= end; e += kBatch) {
        VecT part[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u)
          part[u] = *reinterpret_cast<const VecT *>(carry_val + (size_t)(e + u) * (size_t)N + col0);
#pragma unroll
        for (int u = 0; u < kBatch; ++u)
#pragma unroll
          for (int v = 0; v < VEC; ++v) sum[v] += (A)part[u].v[v];
      }
      for (; e < end; ++e) {
        const VecT part = *reinterpret_cast<const VecT *>(carry_val + (size_t)e * (size_t)N + col0);
#pragma unroll
        for (int v = 0; v < VEC; ++v) sum[v] += (A)part.v[v];
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const T b = EPI != kEpiNone ? bias[col0 + v] : (T)0;
        o.v[v] = apply_epilogue<T, EPI>(sum[v] + (A)o.v[v], b);
      }
      *dst = o;
    }
  }
}

}  // namespace scorch
