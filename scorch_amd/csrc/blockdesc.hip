// A CSR pattern described by 64 x 64 blocks, built on the device.
//
// The block kernels (blocked.hip) and the fused attention kernels (attn.hip, attn_f32.hip) read a
// pattern as: the active blocks in block row major order (block_row_ptr, block_col_idx), per
// active block and row of it a 64-bit word of stored columns (block_words) and the position in the
// CSR arrays of the row's first entry inside the block (block_off), per block the columns any of
// its rows stores (block_cols) and the number of stored positions (block_nnz).  An attention layer
// hands over a fresh mask per call in the reference's loop
// (bench/bench_sparse_transformer.py:354-372), so building this has to cost about what one product
// costs: two passes over the entries, one workgroup per block row, with one host read between them
// (the number of active blocks sizes the arrays of the second).
//
// Pass 1 (count): a workgroup marks the block columns its 64 rows touch in an LDS bitmap and
// counts them; a one-workgroup scan turns the counts into block_row_ptr.
// Pass 2 (fill): the same bitmap, ranked by a prefix sum, gives every entry its block; a
// wavefront takes 64 consecutive entries, the lanes of one (row, block) run OR their column bits
// together (segmented scan by shuffles) and the run's last lane adds the word to memory -- one
// atomic per run and wavefront, to distinct addresses except where a run straddles two
// wavefronts.  Entries may repeat and rows need not be sorted for the words to be right (a
// repeated or out-of-order column just starts another run for the same word); block_off is the
// position of a row's first entry in the block only when the row's columns increase strictly,
// which scorch_hip_csr_inspect reports.
#include "common.hpp"

namespace scorch {
namespace blockdesc {

constexpr int kBlock = 64;
constexpr int kMaxBlockCols = 1 << 17;  // bitmap and ranks: 2 x 16 KB of LDS at most

__device__ __forceinline__ unsigned long long shfl_up_u64(unsigned long long v, int delta) {
  const unsigned lo = (unsigned)__shfl_up((int)(unsigned)v, delta);
  const unsigned hi = (unsigned)__shfl_up((int)(unsigned)(v >> 32), delta);
  return ((unsigned long long)hi << 32) | lo;
}

// The block columns touched by rows [64 br, 64 br + 64) as a bitmap in LDS (s_bits, cleared
// here); s_rp receives the 65 row pointers.  Ends with a workgroup barrier.
__device__ __forceinline__ void mark_block_columns(int br, int nbc, const int *__restrict__ row_ptr,
                                                   const int *__restrict__ col_idx, unsigned *s_bits, int *s_rp) {
  const int tid = threadIdx.x;
  const int nw = (nbc + 31) >> 5;
  for (int i = tid; i < nw; i += kBlockThreads) s_bits[i] = 0;
  if (tid <= kBlock) s_rp[tid] = row_ptr[(size_t)br * kBlock + tid];
  __syncthreads();
  const int lo = s_rp[0], hi = s_rp[kBlock];
  for (int base = lo; base < hi; base += kBlockThreads) {
    const int p = base + tid;
    const int bj = p < hi ? (int)((unsigned)col_idx[p] >> 6) : -1;
    const int before = __shfl_up(bj, 1);
    // consecutive entries mostly share a block: one LDS atomic per run inside a wavefront
    if (p < hi && (wave_lane() == 0 || before != bj) && (unsigned)bj < (unsigned)nbc)
      atomicOr(&s_bits[bj >> 5], 1u << (bj & 31));
  }
  __syncthreads();
}

__global__ __launch_bounds__(kBlockThreads) void count_kernel(int nbc, const int *__restrict__ row_ptr,
                                                              const int *__restrict__ col_idx,
                                                              int *__restrict__ block_row_ptr) {
  extern __shared__ unsigned s_dyn[];
  __shared__ int s_rp[kBlock + 1];
  __shared__ int s_part[kWavesPerBlock];
  const int br = blockIdx.x;
  mark_block_columns(br, nbc, row_ptr, col_idx, s_dyn, s_rp);
  const int nw = (nbc + 31) >> 5;
  int count = 0;
  for (int i = threadIdx.x; i < nw; i += kBlockThreads) count += __popc(s_dyn[i]);
#pragma unroll
  for (int off = kWaveSize / 2; off > 0; off >>= 1) count += __shfl_xor(count, off);
  if (wave_lane() == 0) s_part[threadIdx.x / kWaveSize] = count;
  __syncthreads();
  if (threadIdx.x == 0) {
    int total = 0;
    for (int w = 0; w < kWavesPerBlock; ++w) total += s_part[w];
    block_row_ptr[br + 1] = total;
  }
}

// block_row_ptr[1 .. n] holds counts; afterwards their running sums.  One workgroup.
__global__ __launch_bounds__(kBlockThreads) void scan_kernel(int n, int *__restrict__ block_row_ptr) {
  constexpr int kPerThread = 8;
  __shared__ int s_wave[kWavesPerBlock];
  __shared__ int s_carry;
  if (threadIdx.x == 0) {
    s_carry = 0;
    block_row_ptr[0] = 0;
  }
  __syncthreads();
  const int lane = wave_lane(), w = threadIdx.x / kWaveSize;
  for (int base = 0; base < n; base += kBlockThreads * kPerThread) {
    const int first = base + threadIdx.x * kPerThread;
    int v[kPerThread], sum = 0;
#pragma unroll
    for (int u = 0; u < kPerThread; ++u) {
      v[u] = first + u < n ? block_row_ptr[1 + first + u] : 0;
      sum += v[u];
    }
    int incl = sum;
#pragma unroll
    for (int off = 1; off < kWaveSize; off <<= 1) {
      const int t = __shfl_up(incl, off);
      if (lane >= off) incl += t;
    }
    if (lane == kWaveSize - 1) s_wave[w] = incl;
    __syncthreads();
    int before = s_carry;
    for (int k = 0; k < w; ++k) before += s_wave[k];
    int run = before + incl - sum;
#pragma unroll
    for (int u = 0; u < kPerThread; ++u) {
      run += v[u];
      if (first + u < n) block_row_ptr[1 + first + u] = run;
    }
    __syncthreads();
    if (threadIdx.x == kBlockThreads - 1) s_carry = run;
    __syncthreads();
  }
}

__global__ void clear_kernel(size_t n_words, unsigned long long *__restrict__ words, int *__restrict__ off) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_words; i += stride) {
    words[i] = 0ull;
    off[i] = 0;
  }
}

__global__ __launch_bounds__(kBlockThreads) void fill_kernel(int nbc, const int *__restrict__ row_ptr,
                                                             const int *__restrict__ col_idx,
                                                             const int *__restrict__ block_row_ptr,
                                                             int *__restrict__ block_col_idx,
                                                             unsigned long long *__restrict__ words,
                                                             int *__restrict__ off) {
  extern __shared__ unsigned s_dyn[];
  __shared__ int s_rp[kBlock + 1];
  __shared__ int s_wave[kWavesPerBlock];
  const int br = blockIdx.x;
  const int tid = threadIdx.x, lane = wave_lane(), w = tid / kWaveSize;
  const int nw = (nbc + 31) >> 5;
  unsigned *s_bits = s_dyn;
  int *s_rank = reinterpret_cast<int *>(s_dyn + nw);  // set bits in the words before this one
  mark_block_columns(br, nbc, row_ptr, col_idx, s_bits, s_rp);

  // ranks: every thread a contiguous stretch of the bitmap's words
  const int per = (nw + kBlockThreads - 1) / kBlockThreads;
  const int begin = tid * per < nw ? tid * per : nw;
  const int end = begin + per < nw ? begin + per : nw;
  int sum = 0;
  for (int i = begin; i < end; ++i) sum += __popc(s_bits[i]);
  int incl = sum;
#pragma unroll
  for (int o = 1; o < kWaveSize; o <<= 1) {
    const int t = __shfl_up(incl, o);
    if (lane >= o) incl += t;
  }
  if (lane == kWaveSize - 1) s_wave[w] = incl;
  __syncthreads();
  int rank = incl - sum;
  for (int k = 0; k < w; ++k) rank += s_wave[k];
  for (int i = begin; i < end; ++i) {
    s_rank[i] = rank;
    rank += __popc(s_bits[i]);
  }
  __syncthreads();

  const int first_block = block_row_ptr[br];
  for (int i = tid; i < nw; i += kBlockThreads) {
    unsigned bits = s_bits[i];
    int at = first_block + s_rank[i];
    while (bits) {
      block_col_idx[at++] = i * 32 + __ffs(bits) - 1;
      bits &= bits - 1;
    }
  }

  const int lo = s_rp[0], hi = s_rp[kBlock];
  for (int base = lo; base < hi; base += kBlockThreads) {
    const int p = base + tid;
    const bool in_range = p < hi;
    const int c = in_range ? col_idx[p] : 0;
    const int bj = (int)((unsigned)c >> 6);
    const bool ok = in_range && (unsigned)bj < (unsigned)nbc;
    int r = 0;  // the row of entry p: the last of the 64 whose pointer is at most p
    if (in_range) {
#pragma unroll
      for (int step = kBlock / 2; step > 0; step >>= 1)
        if (s_rp[r + step] <= p) r += step;
    }
    const int key = ok ? (r << 20) ^ bj : -1 - lane;  // (a lane without an entry is a run of its own)
    const int key_before = __shfl_up(key, 1);
    const bool starts_run = lane == 0 || key_before != key;
    const unsigned long long heads = __ballot(starts_run);
    const int run_start = 63 - __clzll(heads & ((2ull << lane) - 1ull));
    unsigned long long word = ok ? 1ull << (c & 63) : 0ull;
#pragma unroll
    for (int o = 1; o < kWaveSize; o <<= 1) {
      const unsigned long long t = shfl_up_u64(word, o);
      if (lane - o >= run_start) word |= t;
    }
    // the entry before this one (for the wavefront's first lane: from memory)
    int c_before = __shfl_up(c, 1);
    if (lane == 0 && in_range && p > lo) c_before = col_idx[p - 1];
    if (ok) {
      const int blk = first_block + s_rank[bj >> 5] + __popc(s_bits[bj >> 5] & ((1u << (bj & 31)) - 1u));
      const size_t at = (size_t)blk * kBlock + r;
      const bool ends_run = lane == kWaveSize - 1 || ((heads >> (lane + 1)) & 1ull);
      if (ends_run) atomicOr(&words[at], word);
      // the row's first entry in the block: the row begins here, or the entry before lies in another block
      if (p == s_rp[r] || (int)((unsigned)c_before >> 6) != bj) off[at] = p;
    }
  }
}

// One wavefront per block: the columns any row stores, and the number of stored positions.
__global__ __launch_bounds__(kBlockThreads) void summary_kernel(int64_t n_active,
                                                                const unsigned long long *__restrict__ words,
                                                                unsigned long long *__restrict__ block_cols,
                                                                int *__restrict__ block_nnz) {
  const int64_t blk = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWaveSize;
  if (blk >= n_active) return;
  unsigned long long word = words[blk * kBlock + wave_lane()];
  int stored = __popcll(word);
#pragma unroll
  for (int o = kWaveSize / 2; o > 0; o >>= 1) {
    const unsigned lo = (unsigned)__shfl_xor((int)(unsigned)word, o);
    const unsigned hi = (unsigned)__shfl_xor((int)(unsigned)(word >> 32), o);
    word |= ((unsigned long long)hi << 32) | lo;
    stored += __shfl_xor(stored, o);
  }
  if (wave_lane() == 0) {
    block_cols[blk] = word;
    block_nnz[blk] = stored;
  }
}

static int check_pattern(const char *fn, int64_t M, int64_t n_cols, int64_t nnz, const void *row_ptr,
                         const void *col_idx) {
  if (M < 0 || n_cols < 0 || nnz < 0) return fail(SCORCH_HIP_EINVAL, "%s: negative size", fn);
  if (M % kBlock || n_cols % kBlock)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: both dimensions must be multiples of %d (got %lld x %lld)", fn, kBlock,
                (long long)M, (long long)n_cols);
  if (M >= INT32_MAX || nnz > INT32_MAX || n_cols / kBlock > kMaxBlockCols)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: pattern too large (at most %d block columns)", fn, kMaxBlockCols);
  SCORCH_REQUIRE(row_ptr != nullptr && (nnz == 0 || col_idx != nullptr), "%s: NULL index array", fn);
  SCORCH_REQUIRE(aligned_to(row_ptr, 4) && aligned_to(col_idx, 4), "%s: index arrays must be 4-byte aligned", fn);
  return SCORCH_HIP_OK;
}

inline size_t lds_bytes(int64_t nbc, int arrays) { return (size_t)((nbc + 31) / 32) * sizeof(unsigned) * arrays; }

}  // namespace blockdesc
}  // namespace scorch

extern "C" int scorch_hip_csr_block_count(int64_t M, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                                          const int32_t *col_idx, int32_t *block_row_ptr, void *stream) {
  using namespace scorch;
  const char *fn = "scorch_hip_csr_block_count";
  if (int rc = blockdesc::check_pattern(fn, M, n_cols, nnz, row_ptr, col_idx)) return rc;
  SCORCH_REQUIRE(block_row_ptr != nullptr && aligned_to(block_row_ptr, 4), "%s: block_row_ptr is NULL or misaligned", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t nbr = M / blockdesc::kBlock, nbc = n_cols / blockdesc::kBlock;
  if (nbr > 0) {
    blockdesc::count_kernel<<<dim3((unsigned)nbr), kBlockThreads, blockdesc::lds_bytes(nbc, 1), s>>>(
        (int)nbc, row_ptr, col_idx, block_row_ptr);
    SCORCH_HIP_CHECK(hipGetLastError());
  }
  blockdesc::scan_kernel<<<1, kBlockThreads, 0, s>>>((int)nbr, block_row_ptr);  // (also writes block_row_ptr[0])
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

extern "C" int scorch_hip_csr_block_fill(int64_t M, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                                         const int32_t *col_idx, const int32_t *block_row_ptr,
                                         int64_t n_active_blocks, int32_t *block_col_idx, uint64_t *block_words,
                                         int32_t *block_off, uint64_t *block_cols, int32_t *block_nnz,
                                         void *stream) {
  using namespace scorch;
  const char *fn = "scorch_hip_csr_block_fill";
  if (int rc = blockdesc::check_pattern(fn, M, n_cols, nnz, row_ptr, col_idx)) return rc;
  if (n_active_blocks < 0 || n_active_blocks > INT32_MAX / blockdesc::kBlock)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: %lld active blocks", fn, (long long)n_active_blocks);
  if (n_active_blocks == 0 || M == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(block_row_ptr && block_col_idx && block_words && block_off && block_cols && block_nnz,
                 "%s: NULL output array", fn);
  SCORCH_REQUIRE(aligned_to(block_words, 8) && aligned_to(block_cols, 8) && aligned_to(block_off, 4) &&
                     aligned_to(block_col_idx, 4) && aligned_to(block_nnz, 4) && aligned_to(block_row_ptr, 4),
                 "%s: misaligned array", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t nbr = M / blockdesc::kBlock, nbc = n_cols / blockdesc::kBlock;
  const size_t n_words = (size_t)n_active_blocks * blockdesc::kBlock;
  unsigned long long *words = reinterpret_cast<unsigned long long *>(block_words);
  size_t clear_blocks = (n_words + kBlockThreads - 1) / kBlockThreads;
  if (clear_blocks > 4096) clear_blocks = 4096;
  blockdesc::clear_kernel<<<dim3((unsigned)clear_blocks), kBlockThreads, 0, s>>>(n_words, words, block_off);
  SCORCH_HIP_CHECK(hipGetLastError());
  blockdesc::fill_kernel<<<dim3((unsigned)nbr), kBlockThreads, blockdesc::lds_bytes(nbc, 2), s>>>(
      (int)nbc, row_ptr, col_idx, block_row_ptr, block_col_idx, words, block_off);
  SCORCH_HIP_CHECK(hipGetLastError());
  const int64_t groups = (n_active_blocks + kWavesPerBlock - 1) / kWavesPerBlock;
  blockdesc::summary_kernel<<<dim3((unsigned)groups), kBlockThreads, 0, s>>>(
      n_active_blocks, words, reinterpret_cast<unsigned long long *>(block_cols), block_nnz);
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

SCORCH_DEFINE_PRELOAD(blockdesc)
