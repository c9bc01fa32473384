// SDDMM and SpMM in fp32 for CSR operands whose entries cluster in 64 x 64 blocks (attention
// masks: block-sparse, sliding windows, causal), on the fp32 matrix instruction.
//
// The general kernels (sddmm.hip, spmm*.hip) gather one dense row per stored entry; that is what
// a graph or an activation matrix needs, and it ends at the rate at which the L2s answer gathers.
// Where at least a few hundred of a block's 4,096 positions are stored, computing the whole
// block as a dense 64 x 64 x D product costs less: the dense rows of a block are then fetched
// once per block, not once per entry.  These kernels are the two halves of the fused fp32
// attention kernel (attn_f32.hip) with the CSR value array in the middle, so that the
// reference's own composition -- SDDMM, row softmax, SpMM per head
// (bench/bench_sparse_transformer.py:354-372; csrc/kernels.h:508-570 and csrc/spmm.h:2007-2089
// for the two products) -- runs on the matrix cores without its caller changing a line.
//
// The caller describes the CSR pattern by blocks (once per pattern): the active blocks in block
// row major order (block_col_idx), per active block and row of it a 64-bit word whose bit c says
// that column 64 bj + c of the row is stored (block_words), and the position in the CSR arrays of
// the row's first stored entry inside the block (block_off).  Rows must hold strictly increasing
// column indices: the entry of bit c is then block_off + (number of set bits below c).
//
// Lane (g, n) = (lane / 16, lane % 16); a wavefront serves 16 rows of the block row, and around
// the MFMAs lane (g, n) holds row n's values for columns 16 t + 4 g + r (t, r = 0 .. 3) of a
// block: the layout in which v_mfma_f32_16x16x4_f32 returns (B A^T) and the one in which it takes
// P^T for B^T P^T.  To and from memory the values travel a row at a time (below).
#include "common.hpp"

namespace scorch {
namespace blocked {

constexpr int kBlock = 64;
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int D>
struct Tile {
  static constexpr int kStride = D + 4;  // floats per LDS row: no bank conflicts for either reader
  static constexpr int kFloats = kBlock * kStride;
  static constexpr int kChunksPerRow = D / 4;
  static constexpr int kChunksPerThread = kBlock * kChunksPerRow / kBlockThreads;
};

// A workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global
// access of the wavefront, stores included -- here that would be a block's results on their way to
// memory, and the tile requested for the next block, at every block.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Which head and which work item a workgroup serves: all workgroups of a head on one XCD when the
// head count allows it (workgroup ids go round the 8 XCDs), so that a head's dense operand is
// fetched into one L2 only.
__device__ __forceinline__ void head_and_rank(int n_heads, int n_items, int &head, int &rank) {
  const int id = blockIdx.x;
  if (n_heads % 8 == 0) {
    const int xcd = id & 7, slot = id >> 3;
    head = xcd + 8 * (slot / n_items);
    rank = slot % n_items;
  } else {
    head = id / n_items;
    rank = id % n_items;
  }
}

// The CSR value arrays are read and written a row at a time: for row r of the wavefront's 16,
// lane c stands for column c of the block, the word of row r says which lanes have an entry, and
// a lane's entry is the row's first in the block plus the number of stored columns below c --
// the lanes' addresses are contiguous whatever the mask, so a row of a block is one or two
// memory transactions.  Between that layout and the matrix instruction's (lane (g, n): row n,
// columns 16 t + 4 g + r) the values pass through a wavefront-private LDS tile of 16 rows.
constexpr int kRowStride = kBlock + 4;          // floats; both layouts then read and write without bank conflicts
constexpr int kRowsFloats = 16 * kRowStride;    // per wavefront

// Word and first position of row r (a compile-time constant under unrolling) of the wavefront's
// rows, from the lanes that hold them (lane (0, r)), as scalars.
__device__ __forceinline__ unsigned long long row_word(unsigned long long word, int r) {
  const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)word, r);
  const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(word >> 32), r);
  return ((unsigned long long)hi << 32) | lo;
}
// Number of set bits of `word` below this lane's position.
__device__ __forceinline__ int bits_below_lane(unsigned long long word) {
  return (int)__builtin_amdgcn_mbcnt_hi((unsigned)(word >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)word, 0u));
}

// out[h][p] = mask_vals[p] * <A[h][row of p], B[h][column of p]> for the entries p of a stretch of
// a block row (SCALED = false: mask_vals is not read, every value is taken to be 1 -- an
// attention mask).  items: x = block row, y and z = the stretch within block_col_idx.
template <int D, bool SCALED>
__global__ __launch_bounds__(kBlockThreads) __attribute__((amdgpu_waves_per_eu(D == 128 ? 2 : 4))) void sddmm_blocked_kernel(
    int M, int n_cols, long long nnz, int n_heads, const int *__restrict__ block_col_idx,
    const unsigned long long *__restrict__ block_words, const int *__restrict__ block_off,
    const float *__restrict__ mask_vals, const float *__restrict__ A, const float *__restrict__ B,
    float *__restrict__ out, int *__restrict__ rows_out, int n_items, const int4 *__restrict__ items) {
  using T = Tile<D>;
  constexpr int kStride = T::kStride;
  constexpr int kSlabs = D / 16;
  constexpr int kCpt = T::kChunksPerThread;
  __shared__ __attribute__((aligned(16))) float s_b[T::kFloats];
  __shared__ __attribute__((aligned(16))) float s_rows[kWavesPerBlock * kRowsFloats];

  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int w = uniform(tid / kWaveSize);
  const int g = lane >> 4;
  const int n = lane & 15;
  int head, rank;
  head_and_rank(n_heads, n_items, head, rank);
  const int4 item = items[rank];
  const int qb = uniform(item.x), kb_begin = uniform(item.y), kb_end = uniform(item.z);
  const int in_block = w * 16 + n;
  const int row = qb * kBlock + in_block;
  const int first_row = qb * kBlock + w * 16;  // of this wavefront
  const float *Bh = B + (size_t)head * (size_t)n_cols * D;
  float *out_h = out + (size_t)head * (size_t)nnz;
  if (head != 0) rows_out = nullptr;
  float *mine = s_rows + w * kRowsFloats;

  floatx4 a_op[kSlabs];
#pragma unroll
  for (int j = 0; j < kSlabs; ++j)
    a_op[j] = *reinterpret_cast<const floatx4 *>(A + ((size_t)head * M + row) * D + 16 * j + 4 * g);

  floatx4 b_next[kCpt];
  auto fetch = [&](int it) {
    const size_t tile = (size_t)uniform(block_col_idx[it]) * kBlock * D;
#pragma unroll
    for (int u = 0; u < kCpt; ++u)
      b_next[u] = *reinterpret_cast<const floatx4 *>(Bh + tile + (size_t)(tid + u * kBlockThreads) * 4);
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int u = 0; u < kCpt; ++u) {
      const int chunk = tid + u * kBlockThreads;
      *reinterpret_cast<floatx4 *>(&s_b[(chunk / T::kChunksPerRow) * kStride + (chunk % T::kChunksPerRow) * 4]) =
          b_next[u];
    }
  };

  unsigned long long word_next = 0;
  int off_next = 0;
  if (kb_begin < kb_end) {
    fetch(kb_begin);
    word_next = block_words[(size_t)kb_begin * kBlock + in_block];
    off_next = block_off[(size_t)kb_begin * kBlock + in_block];
    store_tile();
  }
  __syncthreads();

  for (int it = kb_begin; it < kb_end; ++it) {
    const bool more = it + 1 < kb_end;
    const unsigned long long word = word_next;
    const int off = off_next;
    if (more) {
      fetch(it + 1);
      word_next = block_words[(size_t)(it + 1) * kBlock + in_block];
      off_next = block_off[(size_t)(it + 1) * kBlock + in_block];
    }
    // a block of which every row of the 16 is fully stored (lane c's entry of row r is then the
    // row's first plus c): its mask values are asked for before the products
    const bool whole = __all(word == ~0ull);
    float scale_of[16];
    if (SCALED && whole) {
#pragma unroll
      for (int r = 0; r < 16; ++r) scale_of[r] = mask_vals[__builtin_amdgcn_readlane(off, r) + lane];
    }

    // (A B^T)^T: tile t holds columns 16 t + 4 g + r (r = 0 .. 3) of the block against row n
    floatx4 st[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) st[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < kSlabs; ++j) {
      floatx4 b_op[4];
#pragma unroll
      for (int t = 0; t < 4; ++t)
        b_op[t] = *reinterpret_cast<const floatx4 *>(&s_b[(16 * t + n) * kStride + 16 * j + 4 * g]);
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(b_op[t][c], a_op[j][c], st[t], 0, 0, 0);
    }

    // through the wavefront's LDS rows into the row-at-a-time layout, scaled by the mask's values,
    // out (the other wavefronts of the SIMD are in their products meanwhile)
#pragma unroll
    for (int t = 0; t < 4; ++t) *reinterpret_cast<floatx4 *>(&mine[n * kRowStride + 16 * t + 4 * g]) = st[t];
    wave_lds_sync();
    if (whole) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int at = __builtin_amdgcn_readlane(off, r) + lane;
        const float x = mine[r * kRowStride + lane];
        store_streaming(out_h + at, SCALED ? scale_of[r] * x : x);
        if (rows_out) rows_out[at] = first_row + r;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const unsigned long long stored = row_word(word, r);
        if ((stored >> lane) & 1ull) {
          const int at = __builtin_amdgcn_readlane(off, r) + bits_below_lane(stored);
          const float x = mine[r * kRowStride + lane];
          store_streaming(out_h + at, SCALED ? mask_vals[at] * x : x);
          if (rows_out) rows_out[at] = first_row + r;
        }
      }
    }

    lds_barrier();  // every wavefront is done with this tile (and with its own LDS rows)
    if (more) store_tile();
    lds_barrier();
  }
}

// C[h][row] = sum over the row's entries p of vals[h][p] * B[h][column of p] for a block row or a
// stretch of one.  items: x = block row, y and z = the range within block_col_idx (possibly empty:
// zero rows), w = -1 if the item is the whole block row and writes C, else the slot of `partials`
// (H x n_slots tiles of 64 x D) its sums go to, for spmm_blocked_merge_kernel to add up.
template <int D>
__global__ __launch_bounds__(kBlockThreads) __attribute__((amdgpu_waves_per_eu(D == 128 ? 2 : 4))) void spmm_blocked_kernel(
    int M, int K, long long nnz, int n_heads, const int *__restrict__ block_col_idx,
    const unsigned long long *__restrict__ block_words, const int *__restrict__ block_off,
    const unsigned long long *__restrict__ block_cols, const float *__restrict__ vals, const float *__restrict__ B, float *__restrict__ C, int n_items,
    const int4 *__restrict__ items, int n_slots, float *__restrict__ partials) {
  using T = Tile<D>;
  constexpr int kStride = T::kStride;
  constexpr int kFeat = D / 16;
  constexpr int kCpt = T::kChunksPerThread;
  __shared__ __attribute__((aligned(16))) float s_b[T::kFloats];
  __shared__ __attribute__((aligned(16))) float s_rows[kWavesPerBlock * kRowsFloats];

  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int w = uniform(tid / kWaveSize);
  const int g = lane >> 4;
  const int n = lane & 15;
  int head, rank;
  head_and_rank(n_heads, n_items, head, rank);
  const int4 item = items[rank];
  const int qb = uniform(item.x), kb_begin = uniform(item.y), kb_end = uniform(item.z);
  const int in_block = w * 16 + n;
  const int row = qb * kBlock + in_block;
  const float *Bh = B + (size_t)head * (size_t)K * D;
  const float *vals_h = vals + (size_t)head * (size_t)nnz;
  float *mine = s_rows + w * kRowsFloats;

  floatx4 acc[kFeat];
#pragma unroll
  for (int dt = 0; dt < kFeat; ++dt) acc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // A row of B that no entry of the block refers to is not used: it goes into LDS as zeros, so
  // that whatever it holds (the padding of a batch, never written) meets the zeros standing for
  // "not stored" as 0 x 0.  (A row that some of the block's rows refer to meets the other rows'
  // zeros as it is: a NaN or infinity in it reaches all 64 rows of the block.)
  floatx4 b_next[kCpt];
  unsigned long long cols_next = ~0ull;  // bit c: some row of the tile's block stores column c
  auto fetch = [&](int it) {
    const size_t tile = (size_t)uniform(block_col_idx[it]) * kBlock * D;
    if (block_cols) cols_next = block_cols[it];
#pragma unroll
    for (int u = 0; u < kCpt; ++u)
      b_next[u] = *reinterpret_cast<const floatx4 *>(Bh + tile + (size_t)(tid + u * kBlockThreads) * 4);
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int u = 0; u < kCpt; ++u) {
      const int chunk = tid + u * kBlockThreads;
      const int tile_row = chunk / T::kChunksPerRow;
      const bool used = (cols_next >> tile_row) & 1ull;
      *reinterpret_cast<floatx4 *>(&s_b[tile_row * kStride + (chunk % T::kChunksPerRow) * 4]) =
          used ? b_next[u] : floatx4{0.f, 0.f, 0.f, 0.f};
    }
  };
  // The values of a block, a row at a time (lane c: column c; zero where nothing is stored), and
  // the description of the block after it, one step further ahead so that no load waits for another.
  unsigned long long word_next = 0;
  int off_next = 0;
  auto fetch_description = [&](int it) {
    word_next = block_words[(size_t)it * kBlock + in_block];
    off_next = block_off[(size_t)it * kBlock + in_block];
  };
  float row_next[16];
  auto fetch_values = [&]() {
    if (__all(word_next == ~0ull)) {  // every row of the 16 fully stored: lane c's entry is the row's first plus c
#pragma unroll
      for (int r = 0; r < 16; ++r) row_next[r] = vals_h[__builtin_amdgcn_readlane(off_next, r) + lane];
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const unsigned long long stored = row_word(word_next, r);
        const int at = __builtin_amdgcn_readlane(off_next, r) + bits_below_lane(stored);
        row_next[r] = (stored >> lane) & 1ull ? vals_h[at] : 0.0f;
      }
    }
  };

  if (kb_begin < kb_end) {
    fetch(kb_begin);
    fetch_description(kb_begin);
    fetch_values();
    if (kb_begin + 1 < kb_end) fetch_description(kb_begin + 1);
    store_tile();
  }
  __syncthreads();

  for (int it = kb_begin; it < kb_end; ++it) {
    const bool more = it + 1 < kb_end;
    // this block's values into the operand layout: lane (g, n) takes row n, columns 16 t + 4 g + r
#pragma unroll
    for (int r = 0; r < 16; ++r) mine[r * kRowStride + lane] = row_next[r];
    wave_lds_sync();
    floatx4 p[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) p[t] = *reinterpret_cast<const floatx4 *>(&mine[n * kRowStride + 16 * t + 4 * g]);
    if (more) {
      fetch_values();
      if (it + 2 < kb_end) fetch_description(it + 2);
    }
    // C^T += B^T P^T: step (t, r) contracts columns 16 t + 4 g + r of the block, whose values lane
    // (g, n) holds for row n; the B^T operand is B[that row of B][16 dt + n]
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      if (t == 2 && more) fetch(it + 1);  // (after half of the products: fewer registers live at once)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float *b_row = &s_b[(16 * t + 4 * g + r) * kStride + n];
#pragma unroll
        for (int dt = 0; dt < kFeat; ++dt)
          acc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(b_row[16 * dt], p[t][r], acc[dt], 0, 0, 0);
      }
    }
    lds_barrier();  // every wavefront is done with this tile (and has read its own LDS rows)
    if (more) store_tile();
    lds_barrier();
  }

  const int slot = uniform(item.w);
  float *c_row = slot < 0 ? C + ((size_t)head * M + row) * D
                          : partials + (((size_t)head * n_slots + slot) * kBlock + in_block) * D;
#pragma unroll
  for (int dt = 0; dt < kFeat; ++dt) *reinterpret_cast<floatx4 *>(c_row + 16 * dt + 4 * g) = acc[dt];
}

// The block rows that went out in stretches: C = the stretches' sums added in their order.
// One workgroup per (split row, head); split_rows: x = block row, y = first slot, z = stretches.
template <int D>
__global__ __launch_bounds__(kBlockThreads) void spmm_blocked_merge_kernel(int M, int n_slots,
                                                                           const int4 *__restrict__ split_rows,
                                                                           const float *__restrict__ partials,
                                                                           float *__restrict__ C) {
  const int4 row = split_rows[blockIdx.x];
  const int head = blockIdx.y;
  constexpr int kTile = kBlock * D;  // floats; 256 threads x 4 floats per pass
  const float *base = partials + ((size_t)head * n_slots + row.y) * kTile;
  float *out = C + ((size_t)head * M + (size_t)row.x * kBlock) * D;
  for (int at = threadIdx.x * 4; at < kTile; at += kBlockThreads * 4) {
    floatx4 sum = *reinterpret_cast<const floatx4 *>(base + at);
    for (int p = 1; p < row.z; ++p) {
      const floatx4 x = *reinterpret_cast<const floatx4 *>(base + (size_t)p * kTile + at);
#pragma unroll
      for (int r = 0; r < 4; ++r) sum[r] += x[r];
    }
    *reinterpret_cast<floatx4 *>(out + at) = sum;
  }
}

static int check_blocked(const char *fn, int64_t H, int64_t M, int64_t K, int64_t D, int64_t nnz, int64_t n_active,
                         const void *block_col_idx, const void *block_words, const void *block_off,
                         int64_t n_items, const void *items) {
  if (H < 0 || M < 0 || K < 0 || D < 0 || nnz < 0 || n_active < 0 || n_items < 0)
    return fail(SCORCH_HIP_EINVAL, "%s: negative size", fn);
  if (D != 32 && D != 64 && D != 128)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: the dense operands must be 32, 64 or 128 wide (got %lld)", fn,
                (long long)D);
  if (M % kBlock != 0 || K % kBlock != 0)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: both dimensions of the sparse operand must be multiples of %d "
                "(got %lld x %lld)", fn, kBlock, (long long)M, (long long)K);
  if (nnz > INT32_MAX || M * D > INT32_MAX || K * D > INT32_MAX || n_items * H > INT32_MAX ||
      n_active > INT32_MAX / kBlock)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: operand too large for the int32 index arrays", fn);
  if (n_items > 0) {
    SCORCH_REQUIRE(items != nullptr && aligned_to(items, 16), "%s: items must be 16-byte aligned", fn);
    SCORCH_REQUIRE(n_active == 0 || (block_col_idx && block_words && block_off), "%s: NULL block arrays", fn);
    SCORCH_REQUIRE(aligned_to(block_words, 8) && aligned_to(block_col_idx, 4) && aligned_to(block_off, 4),
                   "%s: misaligned block arrays", fn);
  }
  return SCORCH_HIP_OK;
}

}  // namespace blocked
}  // namespace scorch

extern "C" int scorch_hip_sddmm_csr_blocked_f32(int64_t H, int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                                                int64_t n_active_blocks, const int32_t *block_col_idx,
                                                const uint64_t *block_words, const int32_t *block_off,
                                                int64_t n_items, const int32_t *items, const float *mask_vals,
                                                const float *A, const float *B, float *out_vals,
                                                int32_t *out_row_idx, void *stream) {
  using namespace scorch;
  const char *fn = "scorch_hip_sddmm_csr_blocked_f32";
  const int rc = blocked::check_blocked(fn, H, M, n_cols, K, nnz, n_active_blocks, block_col_idx, block_words,
                                        block_off, n_items, items);
  if (rc != SCORCH_HIP_OK) return rc;
  if (H == 0 || nnz == 0 || n_items == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(A && B && out_vals, "%s: NULL operand", fn);
  SCORCH_REQUIRE(aligned_to(A, 16) && aligned_to(B, 16) && aligned_to(out_vals, 4) && aligned_to(mask_vals, 4),
                 "%s: A and B must be 16-byte aligned", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(n_items * H));
  const unsigned long long *words = reinterpret_cast<const unsigned long long *>(block_words);
  const int4 *item_list = reinterpret_cast<const int4 *>(items);
  mark_launch(s);
#define SCORCH_BLOCKED_SDDMM(DIM, SCALED)                                                                           \
  blocked::sddmm_blocked_kernel<DIM, SCALED><<<grid, kBlockThreads, 0, s>>>(                                        \
      (int)M, (int)n_cols, (long long)nnz, (int)H, block_col_idx, words, block_off, mask_vals, A, B, out_vals,      \
      out_row_idx, (int)n_items, item_list)
  if (mask_vals) {
    if (K == 32) SCORCH_BLOCKED_SDDMM(32, true);
    else if (K == 64) SCORCH_BLOCKED_SDDMM(64, true);
    else SCORCH_BLOCKED_SDDMM(128, true);
  } else {
    if (K == 32) SCORCH_BLOCKED_SDDMM(32, false);
    else if (K == 64) SCORCH_BLOCKED_SDDMM(64, false);
    else SCORCH_BLOCKED_SDDMM(128, false);
  }
#undef SCORCH_BLOCKED_SDDMM
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(s);
  return SCORCH_HIP_OK;
}

extern "C" size_t scorch_hip_spmm_csr_blocked_workspace_bytes(int64_t H, int64_t n_slots, int64_t N) {
  if (H <= 0 || n_slots <= 0 || N <= 0) return 0;
  return (size_t)H * (size_t)n_slots * scorch::blocked::kBlock * (size_t)N * sizeof(float);
}

extern "C" int scorch_hip_spmm_csr_blocked_f32(int64_t H, int64_t M, int64_t K, int64_t N, int64_t nnz,
                                               int64_t n_active_blocks, const int32_t *block_col_idx,
                                               const uint64_t *block_words, const int32_t *block_off,
                                               const uint64_t *block_cols, int64_t n_items, const int32_t *items,
                                               int64_t n_split_rows,
                                               const int32_t *split_rows, int64_t n_slots, const float *vals,
                                               const float *B, float *C, void *workspace, size_t workspace_bytes,
                                               void *stream) {
  using namespace scorch;
  const char *fn = "scorch_hip_spmm_csr_blocked_f32";
  const int rc = blocked::check_blocked(fn, H, M, K, N, nnz, n_active_blocks, block_col_idx, block_words, block_off,
                                        n_items, items);
  if (rc != SCORCH_HIP_OK) return rc;
  if (H == 0 || M == 0) return SCORCH_HIP_OK;
  if (n_split_rows < 0 || n_slots < 0 || n_slots > INT32_MAX || (n_split_rows == 0) != (n_slots == 0))
    return fail(SCORCH_HIP_EINVAL, "%s: %lld split rows with %lld slots", fn, (long long)n_split_rows,
                (long long)n_slots);
  if (n_items < M / blocked::kBlock)
    return fail(SCORCH_HIP_EINVAL, "%s: %lld items for %lld block rows (every block row must be covered)", fn,
                (long long)n_items, (long long)(M / blocked::kBlock));
  SCORCH_REQUIRE((nnz == 0 || vals) && B && C, "%s: NULL operand", fn);
  SCORCH_REQUIRE(aligned_to(B, 16) && aligned_to(C, 16) && aligned_to(vals, 4), "%s: B and C must be 16-byte aligned",
                 fn);
  float *partials = nullptr;
  if (n_split_rows > 0) {
    SCORCH_REQUIRE(split_rows != nullptr && aligned_to(split_rows, 16), "%s: split_rows must be 16-byte aligned", fn);
    const size_t need = scorch_hip_spmm_csr_blocked_workspace_bytes(H, n_slots, N);
    if (!workspace || workspace_bytes < need || !aligned_to(workspace, 256))
      return fail(SCORCH_HIP_EWORKSPACE, "%s: a 256-byte aligned workspace of %zu bytes is needed, %zu given", fn,
                  need, workspace ? workspace_bytes : (size_t)0);
    partials = static_cast<float *>(workspace);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((unsigned)(n_items * H));
  const dim3 merge_grid((unsigned)n_split_rows, (unsigned)H);
  SCORCH_REQUIRE(aligned_to(block_cols, 8), "%s: block_cols must be 8-byte aligned", fn);
  const unsigned long long *words = reinterpret_cast<const unsigned long long *>(block_words);
  const unsigned long long *cols = reinterpret_cast<const unsigned long long *>(block_cols);
  const int4 *item_list = reinterpret_cast<const int4 *>(items);
  const int4 *rows = reinterpret_cast<const int4 *>(split_rows);
  mark_launch(s);
#define SCORCH_BLOCKED_SPMM(DIM)                                                                                  \
  do {                                                                                                            \
    blocked::spmm_blocked_kernel<DIM><<<grid, kBlockThreads, 0, s>>>((int)M, (int)K, (long long)nnz, (int)H,      \
                                                                     block_col_idx, words, block_off, cols, vals, \
                                                                     B, C,                                        \
                                                                     (int)n_items, item_list, (int)n_slots,       \
                                                                     partials);                                   \
    SCORCH_HIP_CHECK(hipGetLastError());                                                                          \
    mark_launch(s);                                                                                               \
    if (n_split_rows > 0) {                                                                                       \
      blocked::spmm_blocked_merge_kernel<DIM><<<merge_grid, kBlockThreads, 0, s>>>((int)M, (int)n_slots, rows,    \
                                                                                   partials, C);                  \
      SCORCH_HIP_CHECK(hipGetLastError());                                                                        \
      mark_launch(s);                                                                                             \
    }                                                                                                             \
  } while (0)
  if (N == 32) SCORCH_BLOCKED_SPMM(32);
  else if (N == 64) SCORCH_BLOCKED_SPMM(64);
  else SCORCH_BLOCKED_SPMM(128);
#undef SCORCH_BLOCKED_SPMM
  return SCORCH_HIP_OK;
}

SCORCH_DEFINE_PRELOAD(blocked)
