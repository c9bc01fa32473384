// CSR x CSR -> CSR (SpGEMM) for gfx950, in the usual two phases: a symbolic
// pass that counts the distinct columns of every output row and turns the
// counts into the row pointer, and a numeric pass that fills column indices
// (ascending within a row) and values.  Every structurally reachable column is
// stored, also when its sum happens to be zero -- the reference's rule.
//
// A row of C is the union of the rows of B selected by the row of A.  How a row
// is processed depends on an upper bound of its size, the number of products
// it sums (sum over its entries of the length of the B row they select):
//
//   up to 32 products    a quarter wavefront, hash table of 64 slots in LDS
//   up to 256 products   one wavefront, hash table of 512 slots in LDS
//                        (a wavefront takes four consecutive rows: the first kind
//                        all at once, then the second kind one after the other)
//   up to 1024 products  one workgroup, hash table of 2048 slots in LDS
//   up to 4096 products  B of at most 131,072 columns: a bitmap of the columns in LDS
//                        (256 threads, see below); wider B: one workgroup, hash
//                        table of 8192 slots in LDS
//   more                 one workgroup of 1024 threads with a bitmap of the columns
//                        in LDS, 524,288 columns at a time (B of up to 4.2 M
//                        columns is covered in up to eight such ranges, walking the
//                        row's products once more for each); wider B: a bitmap over
//                        all N columns in global memory, one per workgroup of a pool
//
// A bitmap row needs neither hashing nor sorting: one walk over the products
// sets the bits, a prefix sum over the bitmap gives every column its rank in
// the row, and (numeric pass) a second walk adds each product at its column's
// rank.
//
// Hash rows are emitted sorted: the wavefront version ranks every entry by
// counting smaller keys (at most 256 of them), the workgroup version sorts in
// LDS by buckets over the row's column range (a bitonic sort when the columns
// cluster).  Bitmap rows come out sorted by construction.
// Floating-point sums are accumulated with atomics, so their rounding can
// differ from run to run in the last bits; the structure never does, and
// integer results are exact.
#include <climits>

#include "common.hpp"

namespace scorch {

constexpr int kTinyProducts = 256;     // wavefront tier (512 slots)
constexpr int kTinySlots = 512;
constexpr int kSmallProducts = 1024;   // workgroup tier 1 (2048 slots)
constexpr int kMediumProducts = 4096;  // workgroup tier 2 (8192 slots)
constexpr int kMediumWorkgroups = 2048;
constexpr int kMinHugeWorkgroups = 64;
constexpr int kMaxHugeWorkgroups = 1024;
constexpr size_t kHugeSlabBudget = (size_t)1 << 30;
constexpr int kLdsBitmapColumns = 8 * 32 * 16384;  // widest B served by the LDS bitmap (in up to 8 ranges of columns)

// Number of bitmap workgroups: as many slabs (N bits and N / 32 ranks) as fit
// the budget, within [kMinHugeWorkgroups, kMaxHugeWorkgroups].
inline int huge_workgroups(int64_t N) {
  const size_t slab = (size_t)(N + 31) / 32 * 8 + 1;
  const size_t fit = kHugeSlabBudget / slab;
  return (int)(fit < (size_t)kMinHugeWorkgroups ? kMinHugeWorkgroups
                                                : (fit > (size_t)kMaxHugeWorkgroups ? kMaxHugeWorkgroups : fit));
}

__device__ __forceinline__ int hash_slot(int key, int mask) {
  return (int)(((unsigned)key * 2654435761u) >> 12) & mask;
}

// Slot of `key` in an open-addressing table (empty = -1); inserts it if absent.
__device__ __forceinline__ int hash_insert(int *keys, int mask, int key) {
  int s = hash_slot(key, mask);
  for (;;) {
    const int prev = atomicCAS(&keys[s], -1, key);
    if (prev == -1 || prev == key) return s;
    s = (s + 1) & mask;
  }
}

// *addr += v, atomically (LDS or global memory).  Floating-point sums use the
// hardware's add instructions (global_atomic_add_f32 / _f64, ds_add_f32 / _f64)
// rather than a compare-and-swap loop; they are exact for ordinary device
// memory, which is what the workspace must be.
template <typename A>
__device__ __forceinline__ void atomic_accumulate(A *addr, A v) { atomicAdd(addr, v); }
template <>
__device__ __forceinline__ void atomic_accumulate<float>(float *addr, float v) { unsafeAtomicAdd(addr, v); }
template <>
__device__ __forceinline__ void atomic_accumulate<double>(double *addr, double v) { unsafeAtomicAdd(addr, v); }
template <>
__device__ __forceinline__ void atomic_accumulate<uint64_t>(uint64_t *addr, uint64_t v) {
  atomicAdd(reinterpret_cast<unsigned long long *>(addr), (unsigned long long)v);
}

// A workgroup's slab in global memory is private to it: its wavefronts share one
// CU and one L2, so workgroup scope is all the ordering it needs.  (A
// device-scope fence would make the L2 write its dirty lines back, once per
// row and workgroup.)  Read after the atomics of other wavefronts of the
// workgroup, behind a __syncthreads().
template <typename A>
__device__ __forceinline__ A workgroup_load(const A *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
template <typename A>
__device__ __forceinline__ void workgroup_store(A *p, A v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// Exclusive prefix sum of one int per thread over a workgroup of WAVES
// wavefronts; `total` receives the sum.  `scratch` holds WAVES ints.
template <int WAVES>
__device__ __forceinline__ int block_exclusive_scan_n(int v, int *scratch, int &total) {
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  int incl = v;
#pragma unroll
  for (int off = 1; off < kWaveSize; off <<= 1) {
    const int up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  __syncthreads();  // scratch may still be read from a previous call
  if (lane == kWaveSize - 1) scratch[w] = incl;
  __syncthreads();
  int before = 0, all = 0;
#pragma unroll
  for (int i = 0; i < WAVES; ++i) {
    const int part = scratch[i];
    if (i < w) before += part;
    all += part;
  }
  total = all;
  return before + incl - v;
}

__device__ __forceinline__ int block_exclusive_scan(int v, int *scratch, int &total) {
  return block_exclusive_scan_n<kWavesPerBlock>(v, scratch, total);
}

// Exclusive scan of `v` over a workgroup of WAVES wavefronts and, behind the same two
// barriers, the workgroup's minimum of `lo` and maximum of `hi`.
template <int WAVES>
__device__ __forceinline__ int block_scan_min_max(int v, int &total, int &lo, int &hi, int *scan_scratch,
                                                  int *min_scratch, int *max_scratch) {
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  int incl = v;
#pragma unroll
  for (int off = 1; off < kWaveSize; off <<= 1) {
    const int up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
#pragma unroll
  for (int off = kWaveSize / 2; off > 0; off >>= 1) {
    const int l = __shfl_xor(lo, off), h = __shfl_xor(hi, off);
    lo = l < lo ? l : lo;
    hi = h > hi ? h : hi;
  }
  __syncthreads();  // the scratch arrays may still be read from a previous call
  if (lane == kWaveSize - 1) scan_scratch[w] = incl;
  if (lane == 0) {
    min_scratch[w] = lo;
    max_scratch[w] = hi;
  }
  __syncthreads();
  int before = 0, all = 0;
#pragma unroll
  for (int i = 0; i < WAVES; ++i) {
    const int part = scan_scratch[i];
    if (i < w) before += part;
    all += part;
    lo = min_scratch[i] < lo ? min_scratch[i] : lo;
    hi = max_scratch[i] > hi ? max_scratch[i] : hi;
  }
  total = all;
  return before + incl - v;
}

// ---- walking the products of one row of C ------------------------------------------------
// The products of a row are the entries of the B rows its A entries select.  B
// rows are often much shorter than a wavefront, so handing one B row to a team
// at a time wastes most lanes and chains three dependent loads per A entry.
// Instead the team (TEAM = 16: a quarter wavefront, 64: one wavefront, 256 or
// 1024: the workgroup) takes
// TEAM entries of A at once -- thread t reads entry t, its B row's start and
// length -- turns the lengths into offsets with a prefix sum, and then walks the
// batch's products flat: product x belongs to the entry e with off[e] <= x <
// off[e + 1], found by bisection in LDS.  All lanes stay busy and consecutive
// lanes read consecutive entries of a B row.
template <int TEAM, typename A>
struct ProductBatch {
  int index[2 * TEAM];  // [e]: first product of entry e within the batch; [TEAM + e]: where its B row starts
  A a_val[TEAM];
};

// Teams of up to a wavefront (64 lanes, or an aligned part of one) need no
// barrier: a wavefront's LDS operations complete in program order.
template <int TEAM>
__device__ __forceinline__ void team_sync() {
  if (TEAM <= kWaveSize) wave_lds_sync(); else __syncthreads();
}

template <int TEAM>
__device__ __forceinline__ int team_exclusive_scan(int v, int *scratch, int &total) {
  if (TEAM > kWaveSize) return block_exclusive_scan_n<TEAM / kWaveSize>(v, scratch, total);
  const int lane = wave_lane();
  const int t = lane % TEAM;
  int incl = v;
#pragma unroll
  for (int off = 1; off < TEAM; off <<= 1) {
    const int up = __shfl_up(incl, off);
    if (t >= off) incl += up;
  }
  total = __shfl(incl, lane - t + TEAM - 1);
  return incl - v;
}

constexpr int kProductsInFlight = 4;

// One step of the walk over a batch's products: products x0, x0 + TEAM, ... (U of
// them) of this thread.  Their bisections interleave and their loads from B are all
// issued before the first is used; a step of one product waits out a whole memory
// round trip for it.  PARTIAL: the batch may end within the step; slots beyond its
// last product read that product again and hand nothing to fn.
template <int TEAM, bool NUMERIC, int U, bool PARTIAL, typename T, typename A, typename Fn>
__device__ __forceinline__ void product_step(int x0, int total, const int *__restrict__ b_crd,
                                             const T *__restrict__ b_val,
                                             const ProductBatch<TEAM, A> &batch, Fn &fn) {
  int q[U], e[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int x = PARTIAL ? min(x0 + u * TEAM, total - 1) : x0 + u * TEAM;
    e[u] = 0;  // the last entry whose offset is <= x (entries without products share an offset)
#pragma unroll
    for (int step = TEAM / 2; step > 0; step >>= 1)
      if (batch.index[e[u] + step] <= x) e[u] += step;
    q[u] = batch.index[TEAM + e[u]] + (x - batch.index[e[u]]);
  }
  int col[U];
  A b[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    col[u] = b_crd[q[u]];
    b[u] = NUMERIC ? (A)b_val[q[u]] : (A)0;
  }
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (!PARTIAL || x0 + u * TEAM < total) fn(col[u], NUMERIC ? batch.a_val[e[u]] * b[u] : (A)0);
}

// fn(column, product) for every product of A entries [a_lo, a_hi); `t` is the
// thread's number in the team.  Uniform over the team.
template <int TEAM, bool NUMERIC, typename T, typename A, typename Fn>
__device__ __forceinline__ void for_each_product(int a_lo, int a_hi, int t, const int *__restrict__ a_crd,
                                                 const T *__restrict__ a_val, const int *__restrict__ b_pos,
                                                 const int *__restrict__ b_crd, const T *__restrict__ b_val,
                                                 ProductBatch<TEAM, A> &batch, int *scan_scratch, Fn fn) {
  constexpr int U = kProductsInFlight;
  for (int base = a_lo; base < a_hi; base += TEAM) {
    const int p = base + t;
    int lo = 0, len = 0;
    A av = (A)0;
    if (p < a_hi) {
      const int j = a_crd[p];
      lo = b_pos[j];
      len = b_pos[j + 1] - lo;
      if (NUMERIC) av = (A)a_val[p];
    }
    int total = 0;
    const int first = team_exclusive_scan<TEAM>(len, scan_scratch, total);
    team_sync<TEAM>();  // the previous batch has been read by everyone
    batch.index[t] = first;
    batch.index[TEAM + t] = lo;
    if (NUMERIC) batch.a_val[t] = av;
    team_sync<TEAM>();
    int x = 0;  // the team's first product of the step
    for (; x + U * TEAM <= total; x += U * TEAM)
      product_step<TEAM, NUMERIC, U, false, T, A>(x + t, total, b_crd, b_val, batch, fn);
    if (x + TEAM < total)  // more than one product a thread is left
      product_step<TEAM, NUMERIC, U, true, T, A>(x + t, total, b_crd, b_val, batch, fn);
    else if (x + t < total)
      product_step<TEAM, NUMERIC, 1, false, T, A>(x + t, total, b_crd, b_val, batch, fn);
  }
}

// ---- exclusive prefix sum of n ints, in place (counts -> row pointer) ------------------
// Three small kernels: per-tile totals, a one-workgroup scan of the totals, and
// a rescan of every tile from its offset.
constexpr int kScanPerThread = 16;
constexpr int kScanTile = kBlockThreads * kScanPerThread;

// (*grand_total also receives the sum of all counts in 64 bits: the row pointer is int32,
// and a result of 2^31 entries or more must be reported, not wrapped)
__global__ __launch_bounds__(kBlockThreads) void scan_tile_totals_kernel(const int *__restrict__ data,
                                                                         int64_t n,
                                                                         int *__restrict__ totals,
                                                                         unsigned long long *__restrict__ grand_total) {
  __shared__ int s_scan[kWavesPerBlock + 1];
  const int64_t first = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
  int mine = 0;
  long long wide = 0;
  for (int e = 0; e < kScanPerThread; ++e) {
    const int v = first + e < n ? data[first + e] : 0;
    mine += v;
    wide += v;
  }
  int total = 0;
  (void)block_exclusive_scan(mine, s_scan, total);
  if (threadIdx.x == 0) totals[blockIdx.x] = total;
#pragma unroll
  for (int off = kWaveSize / 2; off > 0; off >>= 1) wide += __shfl_xor(wide, off);
  if (wave_lane() == 0 && wide > 0) atomicAdd(grand_total, (unsigned long long)wide);
}

__global__ __launch_bounds__(kBlockThreads) void scan_spine_kernel(int *__restrict__ totals,
                                                                   int64_t n_tiles) {
  __shared__ int s_scan[kWavesPerBlock + 1];
  int carried = 0;
  for (int64_t base = 0; base < n_tiles; base += kBlockThreads) {
    const int64_t i = base + threadIdx.x;
    const int v = i < n_tiles ? totals[i] : 0;
    int total = 0;
    const int before = block_exclusive_scan(v, s_scan, total);
    if (i < n_tiles) totals[i] = carried + before;
    carried += total;
  }
}

// (the last element, the total, becomes -1 when the 64-bit total does not fit an int32)
__global__ __launch_bounds__(kBlockThreads) void scan_apply_kernel(int *__restrict__ data, int64_t n,
                                                                   const int *__restrict__ totals,
                                                                   const unsigned long long *__restrict__ grand_total) {
  __shared__ int s_scan[kWavesPerBlock + 1];
  const int64_t first = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
  int v[kScanPerThread];
  int mine = 0;
  for (int e = 0; e < kScanPerThread; ++e) {
    v[e] = first + e < n ? data[first + e] : 0;
    mine += v[e];
  }
  int total = 0;
  int running = totals[blockIdx.x] + block_exclusive_scan(mine, s_scan, total);
  for (int e = 0; e < kScanPerThread; ++e) {
    if (first + e < n) data[first + e] = first + e == n - 1 && *grand_total > (unsigned long long)INT32_MAX ? -1 : running;
    running += v[e];
  }
}

// ---- pass 0: products per row, and the lists of rows too big for a wavefront ----
// A workgroup takes up to kBoundsRows consecutive rows, eight lanes per row; rows
// of A with more than kBoundsLongRow entries are queued in LDS and summed
// afterwards, by a wavefront each or, beyond kBoundsWaveRow entries, by the whole
// workgroup one after the other, so that a hub row does not leave its neighbours'
// lanes waiting on a long dependent chain.  The three row lists are gathered in LDS
// first and appended to the global lists with one atomic per list and
// workgroup: thousands of atomics on one counter would serialise in the L2.
// Rows beyond kMediumProducts products come in two classes: the workgroups that
// take them get them one at a time from a counter, and the longest rows decide
// when that kernel ends, so those of at least kGiantProducts are listed apart
// (from the back of the same array) and handed out first.
constexpr int kGiantProducts = 16384;
constexpr int kBoundsLongRow = 64;
constexpr int kBoundsWaveRow = 2048;
constexpr int kBoundsRows = 256;

// Rows to a workgroup: fewer for matrices that would not fill the chip otherwise
// (their rows tend to be the long ones, which a workgroup takes a few at a time).
inline int bounds_rows_per_group(int64_t M) {
  const int64_t rows = (M / 1024 + 31) / 32 * 32;
  return (int)(rows < 32 ? 32 : rows > kBoundsRows ? kBoundsRows : rows);
}

__global__ __launch_bounds__(kBlockThreads) void spgemm_bounds_kernel(
    int M, int rows_per_group, const int *__restrict__ a_pos, const int *__restrict__ a_crd,
    const int *__restrict__ b_pos, int *__restrict__ products, int *__restrict__ small_rows,
    int *__restrict__ medium_rows, int *__restrict__ huge_rows, int *__restrict__ counters,
    const int *__restrict__ c_pos_if_narrow) {
  constexpr int G = 8;  // lanes per row
  constexpr int kStep = kBlockThreads / G;
  __shared__ int s_long[kBoundsRows];
  __shared__ int s_very_long[kBoundsRows];
  __shared__ int s_list[4][kBoundsRows];  // medium, huge, small, giant
  __shared__ int s_n[6];                  // [4], [5]: long and very long rows queued
  __shared__ int s_base[4];
  __shared__ long long s_part[kWavesPerBlock];
  if (threadIdx.x < 6) s_n[threadIdx.x] = 0;
  __syncthreads();
  auto file_row = [&](int row, long long sum) {
    const int bound = sum > INT_MAX ? INT_MAX : (int)sum;
    products[row] = bound;
    int list = bound >= kGiantProducts ? 3 : bound > kMediumProducts ? 1 : bound > kSmallProducts ? 0
                     : bound > kTinyProducts ? 2 : -1;
    // The numeric pass knows the row's length: a row of many products but at most
    // kMediumProducts distinct columns fits the sums of the tier below, whose
    // smaller workgroups share a compute unit (B no wider than its bitmap).
    if (list == 1 && c_pos_if_narrow && c_pos_if_narrow[row + 1] - c_pos_if_narrow[row] <= kMediumProducts) list = 0;
    if (list >= 0) s_list[list][atomicAdd(&s_n[list], 1)] = row;
  };

  const int t = threadIdx.x % G;
  const int64_t first = (int64_t)blockIdx.x * rows_per_group;
  for (int it = 0; it < rows_per_group / kStep; ++it) {
    const int64_t row = first + it * kStep + threadIdx.x / G;
    int lo = 0, hi = 0;
    if (row < M) {
      lo = a_pos[row];
      hi = a_pos[row + 1];
    }
    const bool is_long = hi - lo > kBoundsLongRow;
    if (is_long) {
      if (t == 0) {
        if (hi - lo > kBoundsWaveRow) s_very_long[atomicAdd(&s_n[5], 1)] = (int)row;
        else s_long[atomicAdd(&s_n[4], 1)] = (int)row;
      }
      hi = lo;
    }
    long long sum = 0;
    for (int p = lo + t; p < hi; p += G) {
      const int j = a_crd[p];
      sum += b_pos[j + 1] - b_pos[j];
    }
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
    if (row < M && t == 0 && !is_long) file_row((int)row, sum);
  }
  __syncthreads();

  const int n_long = s_n[4];
  for (int i = threadIdx.x / kWaveSize; i < n_long; i += kWavesPerBlock) {  // uniform over the wavefront
    const int r = s_long[i];
    long long part = 0;
#pragma unroll 4
    for (int p = a_pos[r] + wave_lane(); p < a_pos[r + 1]; p += kWaveSize) {
      const int j = a_crd[p];
      part += b_pos[j + 1] - b_pos[j];
    }
#pragma unroll
    for (int off = kWaveSize / 2; off > 0; off >>= 1) part += __shfl_xor(part, off);
    if (wave_lane() == 0) file_row(r, part);
  }
  const int n_very_long = s_n[5];
  for (int i = 0; i < n_very_long; ++i) {  // uniform over the workgroup
    const int r = s_very_long[i];
    long long part = 0;
#pragma unroll 4
    for (int p = a_pos[r] + (int)threadIdx.x; p < a_pos[r + 1]; p += kBlockThreads) {
      const int j = a_crd[p];
      part += b_pos[j + 1] - b_pos[j];
    }
#pragma unroll
    for (int off = kWaveSize / 2; off > 0; off >>= 1) part += __shfl_xor(part, off);
    __syncthreads();
    if (wave_lane() == 0) s_part[threadIdx.x / kWaveSize] = part;
    __syncthreads();
    if (threadIdx.x == 0) {
      long long total = 0;
      for (int w = 0; w < kWavesPerBlock; ++w) total += s_part[w];
      file_row(r, total);
    }
  }
  __syncthreads();
  if (threadIdx.x < 4 && s_n[threadIdx.x] > 0)
    s_base[threadIdx.x] = atomicAdd(&counters[threadIdx.x < 3 ? threadIdx.x : 5], s_n[threadIdx.x]);
  __syncthreads();
  int *const lists[3] = {medium_rows, huge_rows, small_rows};
#pragma unroll
  for (int l = 0; l < 3; ++l)
    for (int i = threadIdx.x; i < s_n[l]; i += kBlockThreads) lists[l][s_base[l] + i] = s_list[l][i];
  for (int i = threadIdx.x; i < s_n[3]; i += kBlockThreads) huge_rows[M - 1 - (s_base[3] + i)] = s_list[3][i];
}

// Entry `idx` of the rows beyond kMediumProducts products, the giant ones first.
__device__ __forceinline__ int huge_row(const int *__restrict__ rows, int M, int n_giant, int idx) {
  return idx < n_giant ? rows[M - 1 - idx] : rows[idx - n_giant];
}

// counters: [0] medium rows, [1] huge rows, [2] small rows, [5] giant rows listed; [3], [4] next row to hand out;
// [6..7] one 64-bit sum: the number of entries of the result
__global__ void spgemm_reset_kernel(int *counters, int *c_pos_last) {
  if (threadIdx.x < 8) counters[threadIdx.x] = 0;
  if (threadIdx.x == 0 && c_pos_last) *c_pos_last = 0;
}

// ---- rows of at most kMicroProducts products: a quarter wavefront each -----------------
// Most rows of a very sparse product have a few dozen products: a wavefront each
// would mean a wavefront's start-up and its chain of dependent loads (A's row,
// B's row pointers, B's entries) for every such row.  Sixteen lanes do the same
// steps on tables a quarter the size, four rows to a wavefront.  The teams of a
// wavefront take different numbers of steps; all synchronisation is the
// wavefront's own program order, and shuffles and ballots only look at a
// team's own lanes.
constexpr int kMicroTeam = 16;
constexpr int kMicroProducts = 32;
constexpr int kMicroSlots = 64;

// What TEAMS teams keep in LDS for their rows: the hash table (its occupied slots
// are later compacted to the front of the same arrays: less LDS, more wavefronts
// per CU, and these rows are bound by how many are in flight) and the batch of A
// entries being walked.
template <typename A, bool NUMERIC, int TEAM, int TEAMS, int SLOTS, int PRODUCTS>
struct TeamTables {
  int keys[TEAMS][SLOTS];
  A vals[TEAMS][NUMERIC ? SLOTS : 1];
  ProductBatch<TEAM, A> batch[TEAMS];
};

// One row of C by team number `team` of TEAM lanes (a wavefront or an aligned
// part of one; this lane is its number t): hash the row's products, count or
// compact the occupied slots, sort by rank.
template <typename T, bool NUMERIC, int TEAM, int TEAMS, int SLOTS, int PRODUCTS>
__device__ __forceinline__ void spgemm_team_row(
    TeamTables<typename Acc<T>::type, NUMERIC, TEAM, TEAMS, SLOTS, PRODUCTS> &lds, int team, int t, int row,
    const int *__restrict__ a_pos, const int *__restrict__ a_crd, const T *__restrict__ a_val,
    const int *__restrict__ b_pos, const int *__restrict__ b_crd, const T *__restrict__ b_val,
    int *__restrict__ c_pos, int *__restrict__ c_crd, T *__restrict__ c_val) {
  using A = typename Acc<T>::type;
  const int lane = wave_lane();

  for (int s = t; s < SLOTS; s += TEAM) {
    lds.keys[team][s] = -1;
    if (NUMERIC) lds.vals[team][s] = (A)0;
  }
  wave_lds_sync();

  for_each_product<TEAM, NUMERIC, T, A>(
      a_pos[row], a_pos[row + 1], t, a_crd, a_val, b_pos, b_crd, b_val, lds.batch[team], nullptr,
      [&](int col, A product) {
        const int slot = hash_insert(lds.keys[team], SLOTS - 1, col);
        if (NUMERIC) atomic_accumulate<A>(&lds.vals[team][slot], product);
      });
  wave_lds_sync();

  // Count the occupied slots; in the numeric pass, also compact them, in place: a
  // step's TEAM slots are read by all lanes before any is written, and entry
  // number `at` never lies beyond the slot it came from.
  int n = 0;
  for (int base = 0; base < SLOTS; base += TEAM) {
    const int key = lds.keys[team][base + t];
    A val = (A)0;
    if (NUMERIC) val = lds.vals[team][base + t];
    unsigned long long occupied = __ballot(key != -1) >> (lane - t);  // the team's lanes from bit 0
    if (TEAM < kWaveSize) occupied &= (1ull << (TEAM % kWaveSize)) - 1ull;
    if (NUMERIC) {
      wave_lds_sync();  // everyone has read this step's slots
      if (key != -1) {
        const int at = n + __popcll(occupied & ((1ull << t) - 1ull));
        lds.keys[team][at] = key;
        lds.vals[team][at] = val;
      }
    }
    n += __popcll(occupied);
  }
  if (!NUMERIC) {
    if (t == 0) c_pos[row] = n;
    return;
  }
  wave_lds_sync();

  const int out = c_pos[row];
  // Whole wavefronts with more than a key per lane sort by buckets: counting
  // ranks below costs n compares per key, half of this tier's time at 256 keys a
  // row.  The keys' range is cut into 2 * TEAM equal power-of-two intervals; a
  // prefix sum of the bucket counts (kept where the batch's indices were) places
  // the buckets, the entries are scattered bucket by bucket into the tables'
  // upper halves (free: n <= PRODUCTS <= SLOTS / 2), and an entry's rank is
  // its bucket's start plus the smaller keys in its bucket.  Crowded buckets
  // (clustered columns) leave the row to the rank count.
  if (TEAM == kWaveSize && 2 * PRODUCTS <= SLOTS && n > TEAM) {
    constexpr int kBuckets = 2 * TEAM;
    constexpr int kPerLane = PRODUCTS / TEAM;
    constexpr int kCrowd = 16;
    int *const cnt = lds.batch[team].index;
    int key[kPerLane], pos[kPerLane];
    int key_min = INT_MAX, key_max = -1;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      const int e = t + i * TEAM;
      key[i] = e < n ? lds.keys[team][e] : -1;
      if (e < n) {
        key_min = key[i] < key_min ? key[i] : key_min;
        key_max = key[i] > key_max ? key[i] : key_max;
      }
    }
#pragma unroll
    for (int off = TEAM / 2; off > 0; off >>= 1) {
      const int lo = __shfl_xor(key_min, off), hi = __shfl_xor(key_max, off);
      key_min = lo < key_min ? lo : key_min;
      key_max = hi > key_max ? hi : key_max;
    }
    int shift = 0;
    while (((key_max - key_min) >> shift) >= kBuckets) ++shift;
    cnt[t] = 0;
    cnt[TEAM + t] = 0;
    wave_lds_sync();
#pragma unroll
    for (int i = 0; i < kPerLane; ++i)
      if (t + i * TEAM < n) pos[i] = atomicAdd(&cnt[(key[i] - key_min) >> shift], 1);
    wave_lds_sync();
    const int c0 = cnt[2 * t], c1 = cnt[2 * t + 1];  // lane t places buckets 2t and 2t + 1
    int unused = 0;
    const int before = team_exclusive_scan<TEAM>(c0 + c1, nullptr, unused);
    int crowd = c0 > c1 ? c0 : c1;
#pragma unroll
    for (int off = TEAM / 2; off > 0; off >>= 1) {
      const int other = __shfl_xor(crowd, off);
      crowd = other > crowd ? other : crowd;
    }
    if (crowd <= kCrowd) {  // uniform
      wave_lds_sync();  // everyone has read the counts
      cnt[2 * t] = before;
      cnt[2 * t + 1] = before + c0;
      wave_lds_sync();
#pragma unroll
      for (int i = 0; i < kPerLane; ++i) {
        const int e = t + i * TEAM;
        if (e < n) {
          const int p = PRODUCTS + cnt[(key[i] - key_min) >> shift] + pos[i];
          lds.keys[team][p] = key[i];
          lds.vals[team][p] = lds.vals[team][e];
        }
      }
      wave_lds_sync();
#pragma unroll
      for (int i = 0; i < kPerLane; ++i) {
        const int e = t + i * TEAM;
        if (e < n) {
          const int k = lds.keys[team][PRODUCTS + e];
          const int b = (k - key_min) >> shift;
          const int lo = cnt[b], hi = b + 1 < kBuckets ? cnt[b + 1] : n;
          int rank = lo;
          for (int x = lo; x < hi; ++x) rank += lds.keys[team][PRODUCTS + x] < k ? 1 : 0;
          c_crd[out + rank] = k;
          c_val[out + rank] = (T)lds.vals[team][PRODUCTS + e];
        }
      }
      return;
    }
  }

  // Rank = number of smaller keys (keys are distinct): the sorted position.
  for (int e = t; e < n; e += TEAM) {
    const int key = lds.keys[team][e];
    int rank = 0;
    for (int x = 0; x < n; ++x) rank += lds.keys[team][x] < key ? 1 : 0;
    c_crd[out + rank] = key;
    c_val[out + rank] = (T)lds.vals[team][e];
  }
}

// A wavefront takes four consecutive rows: those of at most kMicroProducts
// products by its four quarters at once, then those of up to kTinyProducts one
// after the other with all its lanes (rows beyond that belong to the workgroup
// kernels).  The two kinds of table share the wavefront's LDS.
// QUARTERS = false: one row per wavefront, all lanes on it whatever its size; for
// matrices of too few rows to fill the chip four to a wavefront.
template <typename T, bool NUMERIC, bool QUARTERS>
__global__ __launch_bounds__(kBlockThreads) void spgemm_tiny_kernel(
    int M, const int *__restrict__ a_pos, const int *__restrict__ a_crd, const T *__restrict__ a_val,
    const int *__restrict__ b_pos, const int *__restrict__ b_crd, const T *__restrict__ b_val,
    const int *__restrict__ products, int *__restrict__ c_pos, int *__restrict__ c_crd,
    T *__restrict__ c_val) {
  using A = typename Acc<T>::type;
  constexpr int kQuarters = kWaveSize / kMicroTeam;
  if (!QUARTERS) {
    __shared__ TeamTables<A, NUMERIC, kWaveSize, kWavesPerBlock, kTinySlots, kTinyProducts> one;
    const int w = threadIdx.x / kWaveSize;
    const int64_t row = xcd_contiguous(blockIdx.x, gridDim.x) * kWavesPerBlock + w;
    if (row >= M || products[row] > kTinyProducts) return;
    spgemm_team_row<T, NUMERIC, kWaveSize, kWavesPerBlock, kTinySlots, kTinyProducts>(
        one, w, wave_lane(), (int)row, a_pos, a_crd, a_val, b_pos, b_crd, b_val, c_pos, c_crd, c_val);
    return;
  }
  union Tables {
    TeamTables<A, NUMERIC, kWaveSize, 1, kTinySlots, kTinyProducts> wave;
    TeamTables<A, NUMERIC, kMicroTeam, kQuarters, kMicroSlots, kMicroProducts> quarter;
  };
  __shared__ Tables lds[kWavesPerBlock];
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  // (the grid is a multiple of 8 workgroups: neighbouring rows, which may well select the same
  // rows of B, go to one XCD)
  const int64_t first = (xcd_contiguous(blockIdx.x, gridDim.x) * kWavesPerBlock + w) * kQuarters;
  if (first >= M) return;
  const int q = lane / kMicroTeam;
  const int64_t mine = first + q;
  const int bound = mine < M ? products[mine] : INT_MAX;
  if (bound <= kMicroProducts)
    spgemm_team_row<T, NUMERIC, kMicroTeam, kQuarters, kMicroSlots, kMicroProducts>(
        lds[w].quarter, q, lane % kMicroTeam, (int)mine, a_pos, a_crd, a_val, b_pos, b_crd, b_val, c_pos, c_crd,
        c_val);
#pragma unroll
  for (int i = 0; i < kQuarters; ++i) {
    const int b = __shfl(bound, i * kMicroTeam);  // uniform
    if (b > kMicroProducts && b <= kTinyProducts) {
      wave_lds_sync();  // the tables' previous users are done
      spgemm_team_row<T, NUMERIC, kWaveSize, 1, kTinySlots, kTinyProducts>(
          lds[w].wave, 0, lane, (int)(first + i), a_pos, a_crd, a_val, b_pos, b_crd, b_val, c_pos, c_crd, c_val);
    }
  }
}

// ---- rows of at most PRODUCTS products: one workgroup each, 2 * PRODUCTS hash slots ----
// THREADS: workgroup size (the tables of the larger form leave room for one workgroup per
// CU: it is given 1024 threads rather than 256).
template <typename T, bool NUMERIC, int PRODUCTS, int COUNTER, int THREADS>
__global__ __launch_bounds__(THREADS) void spgemm_medium_kernel(
    const int *__restrict__ a_pos, const int *__restrict__ a_crd, const T *__restrict__ a_val,
    const int *__restrict__ b_pos, const int *__restrict__ b_crd, const T *__restrict__ b_val,
    const int *__restrict__ rows, const int *__restrict__ counters, int *__restrict__ c_pos,
    int *__restrict__ c_crd, T *__restrict__ c_val) {
  using A = typename Acc<T>::type;
  constexpr int kSlots = 2 * PRODUCTS;
  constexpr int kBuckets = PRODUCTS / 2;
  constexpr int kBucketCrowd = 32;  // a fuller bucket sends the row to the bitonic sort
  __shared__ int s_keys[kSlots];
  __shared__ A s_vals[NUMERIC ? kSlots : 1];
  __shared__ int s_ck[NUMERIC ? PRODUCTS : 1];
  __shared__ A s_cv[NUMERIC ? PRODUCTS : 1];
  __shared__ int s_scan[(THREADS / kWaveSize) + 1];
  __shared__ int s_red[2][(THREADS / kWaveSize)];
  __shared__ int s_cnt[NUMERIC ? kBuckets : 1];
  __shared__ ProductBatch<THREADS, A> s_batch;

  const int tid = threadIdx.x;
  const int n_rows = counters[COUNTER];

  // (rows handed out one at a time through a counter, as in the bitmap tiers, measured
  // slower: these rows are short enough for the counter's round trip to show)
  for (int idx = blockIdx.x; idx < n_rows; idx += gridDim.x) {
    const int row = rows[idx];
    for (int s = tid; s < kSlots; s += THREADS) {
      s_keys[s] = -1;
      if (NUMERIC) s_vals[s] = (A)0;
    }
    if (NUMERIC)
      for (int bkt = tid; bkt < kBuckets; bkt += THREADS) s_cnt[bkt] = 0;
    __syncthreads();

    for_each_product<THREADS, NUMERIC, T, A>(
        a_pos[row], a_pos[row + 1], tid, a_crd, a_val, b_pos, b_crd, b_val, s_batch, s_scan,
        [&](int col, A product) {
          const int slot = hash_insert(s_keys, kSlots - 1, col);
          if (NUMERIC) atomic_accumulate<A>(&s_vals[slot], product);
        });
    __syncthreads();

    // Each thread owns kRun slots, a workgroup's width apart (neighbouring threads
    // on neighbouring LDS banks); an exclusive scan of the per-thread counts
    // places the occupied ones.
    constexpr int kRun = kSlots / THREADS;
    int mine = 0, key_min = INT_MAX, key_max = -1;
    for (int s = 0; s < kRun; ++s) {
      const int key = s_keys[s * THREADS + tid];
      if (key != -1) {
        ++mine;
        key_min = key < key_min ? key : key_min;
        key_max = key > key_max ? key : key_max;
      }
    }
    int n = 0;
    int at = NUMERIC ? block_scan_min_max<THREADS / kWaveSize>(mine, n, key_min, key_max, s_scan, s_red[0], s_red[1])
                     : block_exclusive_scan_n<THREADS / kWaveSize>(mine, s_scan, n);
    if (!NUMERIC) {
      if (tid == 0) c_pos[row] = n;
      __syncthreads();
      continue;
    }

    // Sorting the row's (column, value) pairs.  First choice: buckets.  The
    // columns' range [min, max] is cut into kBuckets equal power-of-two intervals
    // (about two entries each when the columns are spread evenly), a prefix sum of
    // the bucket counts places the buckets, the entries are scattered bucket by
    // bucket, and an entry's rank is its bucket's start plus the smaller keys in
    // its bucket.  If some bucket is crowded (clustered columns), a bitonic sort
    // of the whole row takes over.
    int shift = 0;
    while (((key_max - key_min) >> shift) >= kBuckets) ++shift;  // n > 0 here: the row has products
    for (int s = 0; s < kRun; ++s) {  // (the counts were cleared with the tables)
      const int key = s_keys[s * THREADS + tid];
      if (key != -1) atomicAdd(&s_cnt[(key - key_min) >> shift], 1);
    }
    __syncthreads();
    constexpr int kBucketRun = kBuckets / THREADS;
    int run_total = 0, crowd = 0;
    for (int i = 0; i < kBucketRun; ++i) {
      const int c = s_cnt[tid * kBucketRun + i];
      run_total += c;
      crowd = c > crowd ? c : crowd;
    }
    int unused = 0, unused_min = 0;
    int start = block_scan_min_max<THREADS / kWaveSize>(run_total, unused, unused_min, crowd, s_scan, s_red[0], s_red[1]);
    if (crowd <= kBucketCrowd) {
      for (int i = 0; i < kBucketRun; ++i) {  // counts -> first positions
        const int c = s_cnt[tid * kBucketRun + i];
        s_cnt[tid * kBucketRun + i] = start;
        start += c;
      }
      __syncthreads();
      for (int s = 0; s < kRun; ++s) {
        const int key = s_keys[s * THREADS + tid];
        if (key != -1) {
          const int pos = atomicAdd(&s_cnt[(key - key_min) >> shift], 1);  // ends as the bucket's end
          s_ck[pos] = key;
          s_cv[pos] = s_vals[s * THREADS + tid];
        }
      }
      __syncthreads();
      const int out = c_pos[row];
      for (int e = tid; e < n; e += THREADS) {
        const int key = s_ck[e];
        const int bkt = (key - key_min) >> shift;
        const int lo = bkt ? s_cnt[bkt - 1] : 0, hi = s_cnt[bkt];
        int rank = lo;
        for (int x = lo; x < hi; ++x) rank += s_ck[x] < key ? 1 : 0;
        c_crd[out + rank] = key;
        c_val[out + rank] = (T)s_cv[e];
      }
      __syncthreads();
      continue;
    } else {
      for (int s = 0; s < kRun; ++s) {
        const int key = s_keys[s * THREADS + tid];
        if (key != -1) {
          s_ck[at] = key;
          s_cv[at] = s_vals[s * THREADS + tid];
          ++at;
        }
      }
      int padded = 1;
      while (padded < n) padded <<= 1;
      __syncthreads();
      for (int e = n + tid; e < padded; e += THREADS) s_ck[e] = INT_MAX;
      __syncthreads();
      for (int size = 2; size <= padded; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
          for (int e = tid; e < padded / 2; e += THREADS) {
            const int lo = 2 * e - (e & (stride - 1));
            const int hi = lo + stride;
            const bool ascending = (lo & size) == 0;
            const int klo = s_ck[lo], khi = s_ck[hi];
            if ((klo > khi) == ascending) {
              s_ck[lo] = khi;
              s_ck[hi] = klo;
              const A v = s_cv[lo];
              s_cv[lo] = s_cv[hi];
              s_cv[hi] = v;
            }
          }
          __syncthreads();
        }
      }
    }
    const int out = c_pos[row];
    for (int e = tid; e < n; e += THREADS) {
      c_crd[out + e] = s_ck[e];
      c_val[out + e] = (T)s_cv[e];
    }
    __syncthreads();
  }
}

// ---- rows beyond that: a bitmap over all columns -------------------------------------------
// Workgroups of 1024 threads: such a row has tens of thousands of products and
// is one workgroup's alone, so its width is the row's parallelism.  The
// symbolic pass sets a bit per product and counts the bits.  The numeric pass
// walks the products twice: first for the bits again, from which it writes the
// row's column indices (ascending by construction), zeroes the row's values and
// notes the rank of every bitmap word's first column; then for the values, each
// product adding itself to the row's output at rank(word) + (bits below its own)
// -- no accumulator over all N columns, whose lines would go through the L2 once
// per product.
constexpr int kHugeThreads = 1024;
constexpr int kHugeWaves = kHugeThreads / kWaveSize;
constexpr int kHugeEmitWords = 256;  // bitmap words emitted per step (at most 8192 columns)

template <typename T, bool NUMERIC>
__global__ __launch_bounds__(kHugeThreads) void spgemm_huge_kernel(
    int M, int N, const int *__restrict__ a_pos, const int *__restrict__ a_crd, const T *__restrict__ a_val,
    const int *__restrict__ b_pos, const int *__restrict__ b_crd, const T *__restrict__ b_val,
    const int *__restrict__ rows, const int *__restrict__ counters, unsigned *__restrict__ bitmaps,
    int *__restrict__ ranks, int *__restrict__ c_pos, int *__restrict__ c_crd, T *__restrict__ c_val) {
  using A = typename Acc<T>::type;
  __shared__ int s_scan[kHugeWaves];
  __shared__ ProductBatch<kHugeThreads, A> s_batch;
  __shared__ int s_cols[NUMERIC ? kHugeEmitWords * 32 : 1];
  const int tid = threadIdx.x;
  const int n_giant = counters[5];
  const int n_rows = counters[1] + n_giant;
  if ((int)blockIdx.x >= n_rows) return;

  const int words = (N + 31) / 32;
  unsigned *bitmap = bitmaps + (size_t)blockIdx.x * (size_t)words;
  int *rank = NUMERIC ? ranks + (size_t)blockIdx.x * (size_t)words : nullptr;
  A *acc = reinterpret_cast<A *>(c_val);  // sums wrap (integers) or round (floating point) as T's do
  // This workgroup's bitmap starts clean and is left clean after every row.
  for (int i = tid; i < words; i += kHugeThreads) workgroup_store(&bitmap[i], 0u);
  __syncthreads();

  for (int idx = blockIdx.x; idx < n_rows; idx += gridDim.x) {
    const int row = huge_row(rows, M, n_giant, idx);
    const int a_lo = a_pos[row], a_hi = a_pos[row + 1];
    for_each_product<kHugeThreads, false, T, A>(
        a_lo, a_hi, tid, a_crd, a_val, b_pos, b_crd, b_val, s_batch, s_scan, [&](int k, A) {
          __hip_atomic_fetch_or(&bitmap[k >> 5], 1u << (k & 31), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        });
    __syncthreads();

    if (!NUMERIC) {
      // count the set bits and clear them
      int mine = 0;
      for (int word = tid; word < words; word += kHugeThreads) {
        const unsigned bits = workgroup_load(&bitmap[word]);
        if (bits) {
          mine += __popc(bits);
          workgroup_store(&bitmap[word], 0u);
        }
      }
      int total = 0;
      block_exclusive_scan_n<kHugeWaves>(mine, s_scan, total);
      if (tid == 0) c_pos[row] = total;
    } else {
      // The bitmap in order, kHugeEmitWords words at a time: the set bits of a step
      // are listed in LDS, then written as column indices, coalesced.
      const int out = c_pos[row];
      int emitted = 0;
      for (int base = 0; base < words; base += kHugeEmitWords) {
        const int word = base + tid;
        const bool mine = tid < kHugeEmitWords && word < words;
        unsigned bits = mine ? workgroup_load(&bitmap[word]) : 0u;
        int total = 0;
        int at = block_exclusive_scan_n<kHugeWaves>(__popc(bits), s_scan, total);
        if (mine) workgroup_store(&rank[word], emitted + at);
        while (bits) {
          const int bit = __ffs(bits) - 1;
          bits &= bits - 1;
          s_cols[at++] = word * 32 + bit;
        }
        __syncthreads();
        for (int e = tid; e < total; e += kHugeThreads) {
          c_crd[out + emitted + e] = s_cols[e];
          workgroup_store(&acc[out + emitted + e], (A)0);
        }
        emitted += total;
        // the next step's scan starts with a barrier, which also protects s_cols
      }
      __syncthreads();
      for_each_product<kHugeThreads, true, T, A>(
          a_lo, a_hi, tid, a_crd, a_val, b_pos, b_crd, b_val, s_batch, s_scan, [&](int k, A product) {
            const unsigned bits = workgroup_load(&bitmap[k >> 5]);
            const int at = out + workgroup_load(&rank[k >> 5]) + __popc(bits & ((1u << (k & 31)) - 1u));
            __hip_atomic_fetch_add(&acc[at], product, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          });
      __syncthreads();
      for (int word = tid; word < words; word += kHugeThreads)
        if (workgroup_load(&bitmap[word])) workgroup_store(&bitmap[word], 0u);
    }
    __syncthreads();
  }
}

// ---- the same tier when the bitmap fits LDS ---------------------------------------------------
// Atomics on a bitmap in global memory all land on a few hundred cache lines and
// queue up in the L2's atomic units (the 13.7 M products of a power-law square
// spend 0.4 ms there per walk).  For N up to 32 * WORDS columns the bitmap lives
// in LDS instead, with one rank per four bitmap words, and so do the sums of the
// row's first kAccEntries output entries (the others are added into the output
// with global atomics as above).
constexpr int kLdsBudget = 160 * 1024 - 1024;

// THREADS: workgroup size.  ACC: LDS sums to provide (0: all the LDS that is left).
// LIST, WORK: which of `counters` holds the length of `rows` and the next row to hand out.
template <typename T, bool NUMERIC, int WORDS, int THREADS, int ACC, int LIST, int WORK>
__global__ __launch_bounds__(THREADS) void spgemm_lds_bitmap_kernel(
    int M, int N, const int *__restrict__ a_pos, const int *__restrict__ a_crd, const T *__restrict__ a_val,
    const int *__restrict__ b_pos, const int *__restrict__ b_crd, const T *__restrict__ b_val,
    const int *__restrict__ rows, int *__restrict__ counters, int *__restrict__ c_pos,
    int *__restrict__ c_crd, T *__restrict__ c_val) {
  using A = typename Acc<T>::type;
  constexpr int kGroups = WORDS / 4;
  constexpr int kFixed = WORDS * 4 + (NUMERIC ? kGroups * 4 : 0) + (int)sizeof(ProductBatch<THREADS, A>) + 512;
  constexpr int kAccEntries = !NUMERIC ? 1 : ACC > 0 ? ACC : (kLdsBudget - kFixed) / (int)sizeof(A);
  constexpr int kWaves = THREADS / kWaveSize;
  __shared__ __align__(16) unsigned s_bits[WORDS];
  __shared__ int s_rank[NUMERIC ? kGroups : 1];  // rank of the first column of every group of four words
  __shared__ A s_acc[kAccEntries];
  __shared__ ProductBatch<THREADS, A> s_batch;
  __shared__ int s_scan[kWaves];
  __shared__ int s_next;
  const int tid = threadIdx.x;
  const int n_giant = LIST == 1 ? counters[5] : 0;  // only the list of the longest rows has the class
  const int n_rows = counters[LIST] + n_giant;
  if ((int)blockIdx.x >= n_rows) return;  // more workgroups than rows: no need to queue at the counter
  constexpr int kRangeColumns = 32 * WORDS;
  A *acc = reinterpret_cast<A *>(c_val);
  // B with no more columns than the LDS holds sums: the numeric pass keeps a sum
  // per column and walks the row's products once (bits and sums together)
  // instead of twice (bits, then sums at their ranks).
  const bool sums_by_column = NUMERIC && N <= kAccEntries && N <= kRangeColumns;

  // The longest rows are handed out through a counter, one at a time, so that the
  // workgroups stay evenly loaded; the rows of the tier below are short enough
  // for the counter's round trip to show, and are taken in fixed strides.
  for (int turn = 0;; ++turn) {
    __syncthreads();  // everyone is done with the previous row (and with s_next)
    int idx;
    if (LIST == 1) {
      if (tid == 0) s_next = atomicAdd(&counters[WORK], 1);
      __syncthreads();
      idx = s_next;
    } else {
      idx = (int)blockIdx.x + turn * (int)gridDim.x;
    }
    if (idx >= n_rows) return;  // the same for every thread
    const int row = LIST == 1 ? huge_row(rows, M, n_giant, idx) : rows[idx];
    const int a_lo = a_pos[row], a_hi = a_pos[row + 1];
    const int out = NUMERIC ? c_pos[row] : 0;
    int done = 0;  // distinct columns found in the ranges before this one

    // B wider than the bitmap: one range of kRangeColumns columns after the other,
    // walking the row's products again for each (ranges ascend, so the row comes
    // out sorted all the same)
    for (int c0 = 0; c0 < N; c0 += kRangeColumns) {
      const int columns = N - c0 < kRangeColumns ? N - c0 : kRangeColumns;
      const int groups = ((columns + 31) / 32 + 3) / 4;
      if (c0 > 0) __syncthreads();  // the previous range's bits, ranks and sums have been used
      for (int i = tid; i < 4 * groups; i += THREADS) s_bits[i] = 0u;
      if (sums_by_column)
        for (int i = tid; i < columns; i += THREADS) s_acc[i] = (A)0;
      __syncthreads();
      if (sums_by_column) {
        for_each_product<THREADS, true, T, A>(
            a_lo, a_hi, tid, a_crd, a_val, b_pos, b_crd, b_val, s_batch, s_scan, [&](int k, A product) {
              atomicOr(&s_bits[k >> 5], 1u << (k & 31));
              atomic_accumulate<A>(&s_acc[k], product);
            });
      } else {
        for_each_product<THREADS, false, T, A>(
            a_lo, a_hi, tid, a_crd, a_val, b_pos, b_crd, b_val, s_batch, s_scan, [&](int k, A) {
              const unsigned rel = (unsigned)(k - c0);
              if (rel < (unsigned)columns) atomicOr(&s_bits[rel >> 5], 1u << (rel & 31));
            });
      }
      __syncthreads();

      // distinct columns of the range, and the rank of each group's first one
      int n = 0;
      for (int base = 0; base < groups; base += THREADS) {
        const int g = base + tid;
        int cnt = 0;
        if (g < groups)
          cnt = __popc(s_bits[4 * g]) + __popc(s_bits[4 * g + 1]) + __popc(s_bits[4 * g + 2]) +
                __popc(s_bits[4 * g + 3]);
        int total = 0;
        const int at = block_exclusive_scan_n<kWaves>(cnt, s_scan, total);
        if (NUMERIC && g < groups) s_rank[g] = n + at;
        n += total;
      }
      if (NUMERIC && n > 0) {  // uniform
        const int first = out + done;  // the range's place in the row's output
        // The first kAccEntries output entries have their sums, and before that their
        // column indices, in LDS; entries beyond go straight to the output: a
        // thread's columns lie far apart there (single 4-byte stores), and sums added
        // with global atomics queue up in the L2's atomic units.
        const int in_lds = n < kAccEntries ? n : kAccEntries;
        __syncthreads();  // s_rank is complete
        for (int g = tid; g < groups; g += THREADS) {
          int at = s_rank[g];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            unsigned bits = s_bits[4 * g + i];
            while (bits) {
              const int bit = __ffs(bits) - 1;
              bits &= bits - 1;
              const int col = c0 + (4 * g + i) * 32 + bit;
              c_crd[first + at] = col;
              if (sums_by_column) c_val[first + at] = (T)s_acc[col];
              ++at;
            }
          }
        }
        if (sums_by_column) break;  // uniform; the only range: the row is complete
        for (int e = in_lds + tid; e < n; e += THREADS) workgroup_store(&acc[first + e], (A)0);
        for (int e = tid; e < in_lds; e += THREADS) s_acc[e] = (A)0;
        __syncthreads();
        for_each_product<THREADS, true, T, A>(
            a_lo, a_hi, tid, a_crd, a_val, b_pos, b_crd, b_val, s_batch, s_scan, [&](int k, A product) {
              const unsigned rel = (unsigned)(k - c0);
              if (rel >= (unsigned)columns) return;
              // rank = the group's + the bits below the column's in the group's four words,
              // which come in one read (a loop over the words before the column's
              // would chain up to three more LDS round trips)
              const int w = (int)(rel >> 5), sub = w & 3;
              const uint4 grp = *reinterpret_cast<const uint4 *>(&s_bits[w & ~3]);
              const unsigned below = (1u << (rel & 31)) - 1u;
              const int at = s_rank[w >> 2] + __popc(grp.x & (sub == 0 ? below : ~0u)) +
                             __popc(grp.y & (sub == 1 ? below : sub > 1 ? ~0u : 0u)) +
                             __popc(grp.z & (sub == 2 ? below : sub > 2 ? ~0u : 0u)) +
                             __popc(grp.w & (sub == 3 ? below : 0u));
              if (at < kAccEntries) atomic_accumulate<A>(&s_acc[at], product);
              else __hip_atomic_fetch_add(&acc[first + at], product, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            });
        __syncthreads();
        for (int e = tid; e < in_lds; e += THREADS) c_val[first + e] = (T)s_acc[e];
      }
      done += n;
    }
    if (!NUMERIC && tid == 0) c_pos[row] = done;
  }
}

// ---- host side ------------------------------------------------------------------------------
struct SpgemmWorkspace {
  int *products, *small_rows, *medium_rows, *huge_rows, *counters;
  int huge_pool;
  int *scan_totals;
  unsigned *bitmaps;
  int *ranks;
  size_t total;
};

inline size_t round256(size_t v) { return (v + 255) / 256 * 256; }

inline SpgemmWorkspace spgemm_layout(char *base, int64_t M, int64_t N, size_t elem) {
  SpgemmWorkspace ws;
  size_t off = 0;
  auto take = [&](size_t bytes) { char *p = base ? base + off : nullptr; off += round256(bytes); return p; };
  ws.products = reinterpret_cast<int *>(take((size_t)M * 4));
  ws.small_rows = reinterpret_cast<int *>(take((size_t)M * 4));
  ws.medium_rows = reinterpret_cast<int *>(take((size_t)M * 4));
  ws.huge_rows = reinterpret_cast<int *>(take((size_t)M * 4));
  ws.counters = reinterpret_cast<int *>(take(32));
  ws.scan_totals = reinterpret_cast<int *>(take(((size_t)(M + 1) / kScanTile + 1) * 4));
  ws.huge_pool = huge_workgroups(N);
  // up to kLdsBitmapColumns columns the bitmap tier lives in LDS and needs no slabs
  const size_t slab_words = N <= kLdsBitmapColumns ? 0 : (size_t)(N + 31) / 32;
  ws.bitmaps = reinterpret_cast<unsigned *>(take((size_t)ws.huge_pool * slab_words * 4));
  ws.ranks = reinterpret_cast<int *>(take((size_t)ws.huge_pool * slab_words * 4));
  (void)elem;  // no part of the workspace depends on the value type
  ws.total = off;
  return ws;
}

inline int spgemm_check(const char *fn, int64_t M, int64_t K, int64_t N, const void *a_pos,
                        const void *a_crd, const void *b_pos, const void *b_crd, const void *c_pos,
                        const void *workspace, size_t workspace_bytes, size_t elem) {
  if (M < 0 || K < 0 || N < 0)
    return fail(SCORCH_HIP_EINVAL, "%s: negative size (M=%lld K=%lld N=%lld)", fn, (long long)M,
                (long long)K, (long long)N);
  if (M >= INT32_MAX || K >= INT32_MAX || N >= INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  SCORCH_REQUIRE(a_pos && b_pos && c_pos, "%s: NULL row pointer", fn);
  SCORCH_REQUIRE(aligned_to(a_pos, 4) && aligned_to(a_crd, 4) && aligned_to(b_pos, 4) &&
                     aligned_to(b_crd, 4) && aligned_to(c_pos, 4),
                 "%s: index arrays must be 4-byte aligned", fn);
  const size_t need = spgemm_layout(nullptr, M, N, elem).total;
  if (!workspace || workspace_bytes < need)
    return fail(SCORCH_HIP_EWORKSPACE, "%s: workspace of %zu bytes needed, %zu given", fn, need,
                workspace ? workspace_bytes : (size_t)0);
  SCORCH_REQUIRE(aligned_to(workspace, 256), "%s: workspace must be 256-byte aligned", fn);
  return SCORCH_HIP_OK;
}

template <typename T, bool NUMERIC>
int spgemm_run(int M, int N, const int *a_pos, const int *a_crd, const T *a_val, const int *b_pos,
               const int *b_crd, const T *b_val, int *c_pos, int *c_crd, T *c_val,
               const SpgemmWorkspace &ws, hipStream_t stream) {
  spgemm_reset_kernel<<<1, 64, 0, stream>>>(ws.counters, NUMERIC ? nullptr : c_pos + M);
  SCORCH_HIP_CHECK(hipGetLastError());
  const int rows_per_group = bounds_rows_per_group(M);
  const unsigned row_groups = (unsigned)(((int64_t)M + rows_per_group - 1) / rows_per_group);
  spgemm_bounds_kernel<<<row_groups, kBlockThreads, 0, stream>>>(M, rows_per_group, a_pos, a_crd, b_pos, ws.products,
                                                                ws.small_rows, ws.medium_rows,
                                                                ws.huge_rows, ws.counters,
                                                                NUMERIC && N <= 32 * 4096 ? c_pos : nullptr);
  SCORCH_HIP_CHECK(hipGetLastError());
  // four rows to a wavefront once that still leaves every wavefront slot of the chip a wavefront
  if ((int64_t)M >= 4 * 8192) {
    const int64_t rows_per_block = kWavesPerBlock * (kWaveSize / kMicroTeam);
    const unsigned tiny_blocks = (unsigned)round_up_8(((int64_t)M + rows_per_block - 1) / rows_per_block);
    spgemm_tiny_kernel<T, NUMERIC, true><<<tiny_blocks, kBlockThreads, 0, stream>>>(
        M, a_pos, a_crd, a_val, b_pos, b_crd, b_val, ws.products, c_pos, c_crd, c_val);
  } else {
    const unsigned tiny_blocks = (unsigned)round_up_8(((int64_t)M + kWavesPerBlock - 1) / kWavesPerBlock);
    spgemm_tiny_kernel<T, NUMERIC, false><<<tiny_blocks, kBlockThreads, 0, stream>>>(
        M, a_pos, a_crd, a_val, b_pos, b_crd, b_val, ws.products, c_pos, c_crd, c_val);
  }
  SCORCH_HIP_CHECK(hipGetLastError());
  const unsigned medium_blocks = (unsigned)(M < kMediumWorkgroups ? M : kMediumWorkgroups);
  spgemm_medium_kernel<T, NUMERIC, kSmallProducts, 2, kBlockThreads><<<medium_blocks, kBlockThreads, 0, stream>>>(
      a_pos, a_crd, a_val, b_pos, b_crd, b_val, ws.small_rows, ws.counters, c_pos, c_crd, c_val);
  SCORCH_HIP_CHECK(hipGetLastError());
  if (N <= 32 * 4096) {
    // narrow enough for a bitmap in LDS beside other workgroups: no hashing, nothing to sort
    spgemm_lds_bitmap_kernel<T, NUMERIC, 4096, kBlockThreads, kMediumProducts, 0, 4>
        <<<medium_blocks, kBlockThreads, 0, stream>>>(M, N, a_pos, a_crd, a_val, b_pos, b_crd, b_val,
                                                      ws.medium_rows, ws.counters, c_pos, c_crd, c_val);
  } else {
    // tables for 4096 products leave room for one workgroup per CU: as many threads as still fit
    // beside them (with 8-byte sums, no more than 256)
    constexpr int kThreads = sizeof(typename Acc<T>::type) > 4 ? kBlockThreads : kHugeThreads;
    spgemm_medium_kernel<T, NUMERIC, kMediumProducts, 0, kThreads><<<medium_blocks, kThreads, 0, stream>>>(
        a_pos, a_crd, a_val, b_pos, b_crd, b_val, ws.medium_rows, ws.counters, c_pos, c_crd, c_val);
  }
  SCORCH_HIP_CHECK(hipGetLastError());
  // one workgroup per CU's worth of LDS; more only queue up behind them
  const unsigned lds_pool = (unsigned)(M < 512 ? M : 512);
  if (N <= 32 * 4096)
    spgemm_lds_bitmap_kernel<T, NUMERIC, 4096, kHugeThreads, 0, 1, 3><<<lds_pool, kHugeThreads, 0, stream>>>(
        M, N, a_pos, a_crd, a_val, b_pos, b_crd, b_val, ws.huge_rows, ws.counters, c_pos, c_crd, c_val);
  else if (!NUMERIC && N > 32 * 16384 && N <= 32 * 32768)
    // the symbolic pass keeps no ranks or sums: its bitmap can be twice as wide, one range instead of two
    spgemm_lds_bitmap_kernel<T, NUMERIC, NUMERIC ? 16384 : 32768, kHugeThreads, 0, 1, 3>
        <<<lds_pool, kHugeThreads, 0, stream>>>(M, N, a_pos, a_crd, a_val, b_pos, b_crd, b_val, ws.huge_rows,
                                                ws.counters, c_pos, c_crd, c_val);
  else if (N <= kLdsBitmapColumns)
    spgemm_lds_bitmap_kernel<T, NUMERIC, 16384, kHugeThreads, 0, 1, 3><<<lds_pool, kHugeThreads, 0, stream>>>(
        M, N, a_pos, a_crd, a_val, b_pos, b_crd, b_val, ws.huge_rows, ws.counters, c_pos, c_crd, c_val);
  else
    spgemm_huge_kernel<T, NUMERIC><<<ws.huge_pool, kHugeThreads, 0, stream>>>(
        M, N, a_pos, a_crd, a_val, b_pos, b_crd, b_val, ws.huge_rows, ws.counters, ws.bitmaps,
        ws.ranks, c_pos, c_crd, c_val);
  SCORCH_HIP_CHECK(hipGetLastError());
  if (!NUMERIC) {
    const int64_t n = (int64_t)M + 1;
    const unsigned tiles = (unsigned)((n + kScanTile - 1) / kScanTile);
    unsigned long long *grand_total = reinterpret_cast<unsigned long long *>(ws.counters + 6);
    scan_tile_totals_kernel<<<tiles, kBlockThreads, 0, stream>>>(c_pos, n, ws.scan_totals, grand_total);
    SCORCH_HIP_CHECK(hipGetLastError());
    scan_spine_kernel<<<1, kBlockThreads, 0, stream>>>(ws.scan_totals, tiles);
    SCORCH_HIP_CHECK(hipGetLastError());
    scan_apply_kernel<<<tiles, kBlockThreads, 0, stream>>>(c_pos, n, ws.scan_totals, grand_total);
    SCORCH_HIP_CHECK(hipGetLastError());
  }
  return SCORCH_HIP_OK;
}

template <typename T>
int spgemm_numeric_entry(const char *fn, int64_t M, int64_t K, int64_t N, const int32_t *a_pos,
                         const int32_t *a_crd, const T *a_val, const int32_t *b_pos,
                         const int32_t *b_crd, const T *b_val, const int32_t *c_pos, int32_t *c_crd,
                         T *c_val, void *workspace, size_t workspace_bytes, void *stream) {
  if (int rc = spgemm_check(fn, M, K, N, a_pos, a_crd, b_pos, b_crd, c_pos, workspace, workspace_bytes,
                            sizeof(T)))
    return rc;
  if (M == 0 || N == 0 || K == 0) return SCORCH_HIP_OK;
  const SpgemmWorkspace ws = spgemm_layout(static_cast<char *>(workspace), M, N, sizeof(T));
  return spgemm_run<T, true>((int)M, (int)N, a_pos, a_crd, a_val, b_pos, b_crd, b_val,
                             const_cast<int32_t *>(c_pos), c_crd, c_val, ws,
                             static_cast<hipStream_t>(stream));
}

}  // namespace scorch

extern "C" {

size_t scorch_hip_spgemm_csr_workspace_bytes(int64_t M, int64_t N, size_t elem_size) {
  if (M < 0 || N < 0 || M >= INT32_MAX || elem_size == 0) return 0;
  return scorch::spgemm_layout(nullptr, M, N, elem_size).total;
}

int scorch_hip_spgemm_csr_symbolic(int64_t M, int64_t K, int64_t N, const int32_t *a_row_ptr,
                                   const int32_t *a_col_idx, const int32_t *b_row_ptr,
                                   const int32_t *b_col_idx, int32_t *c_row_ptr, void *workspace,
                                   size_t workspace_bytes, void *stream) {
  using namespace scorch;
  const char *fn = "scorch_hip_spgemm_csr_symbolic";
  if (int rc = spgemm_check(fn, M, K, N, a_row_ptr, a_col_idx, b_row_ptr, b_col_idx, c_row_ptr,
                            workspace, workspace_bytes, 1))
    return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (M == 0) {
    spgemm_reset_kernel<<<1, 64, 0, s>>>(static_cast<int *>(workspace), c_row_ptr);
    SCORCH_HIP_CHECK(hipGetLastError());
    return SCORCH_HIP_OK;
  }
  const SpgemmWorkspace ws = spgemm_layout(static_cast<char *>(workspace), M, N, 1);
  return spgemm_run<float, false>((int)M, (int)N, a_row_ptr, a_col_idx, nullptr, b_row_ptr, b_col_idx,
                                  nullptr, c_row_ptr, nullptr, nullptr, ws, s);
}

#define SCORCH_DEFINE_SPGEMM(SUFFIX, T)                                                             \
  int scorch_hip_spgemm_csr_numeric_##SUFFIX(                                                        \
      int64_t M, int64_t K, int64_t N, const int32_t *a_row_ptr, const int32_t *a_col_idx,           \
      const T *a_vals, const int32_t *b_row_ptr, const int32_t *b_col_idx, const T *b_vals,          \
      const int32_t *c_row_ptr, int32_t *c_col_idx, T *c_vals, void *workspace,                      \
      size_t workspace_bytes, void *stream) {                                                        \
    return scorch::spgemm_numeric_entry<T>("scorch_hip_spgemm_csr_numeric_" #SUFFIX, M, K, N,       \
                                           a_row_ptr, a_col_idx, a_vals, b_row_ptr, b_col_idx,      \
                                           b_vals, c_row_ptr, c_col_idx, c_vals, workspace,         \
                                           workspace_bytes, stream);                                \
  }

SCORCH_DEFINE_SPGEMM(f32, float)
SCORCH_DEFINE_SPGEMM(f64, double)
SCORCH_DEFINE_SPGEMM(i32, int32_t)
SCORCH_DEFINE_SPGEMM(i64, int64_t)

}  // extern "C"

SCORCH_DEFINE_PRELOAD(spgemm)
