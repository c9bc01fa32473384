// Smaller kernels around the SpMM/SDDMM path: CSR row softmax, the
// CSR -> coordinate row expansion, and the library's error/version calls.
#include "common.hpp"

namespace scorch {

char *error_buffer() {
  static thread_local char buf[kErrorBufferBytes] = {0};
  return buf;
}

LaunchMarks *launch_marks() {
  static thread_local LaunchMarks marks;
  return &marks;
}

// ---- CSR row softmax ----------------------------------------------------------
// p = exp(s - max_row) / sum_row over the stored entries of each row, in three
// phases (maximum, sum of exponentials, normalised write) like the five torch
// passes it replaces.  One kernel; a workgroup owns 256 / G consecutive rows and
// serves them in tiers by length, so that a long row never stalls the lanes
// beside it:
//   up to kSoftmaxRegs * G entries   one group of G lanes per row, all at once;
//   up to kSoftmaxRegs * 16 entries  quarter wavefronts, sixteen rows at a time
//                                    (only when G < 16);
//   up to kSoftmaxRegs * 64 entries  one wavefront per row, the workgroup's four
//                                    wavefronts sharing those rows out;
//   up to 1024 entries               the same with sixteen entries per lane;
//   up to 4096 entries               the whole workgroup, one row after the other.
// In all of these a row sits in registers between the phases and is read from
// memory once.  Rows beyond 4096 entries are only noted, in a list in the
// caller's workspace (one atomic per workgroup that has any), and
// softmax_csr_giant_kernel then deals them out, one row at a time, to
// workgroups of 1024 threads (the first 8192 entries in registers, the rest
// read twice: a running maximum and sum first, the write second; the next
// row's entries are requested before the current row's phases start): however such rows are placed in the matrix, few among
// many short ones or all of them long, they are spread over the whole chip.
// Some rows are not one workgroup's either (the reference's softmax is torch scatter operations
// over entries, bench/bench_sparse_transformer.py:277-297: a single row of millions costs it what
// any other four million entries cost): the giant-row kernel only enters such a row in a second
// list, cut into up to 1024 stretches, and two more kernels serve the stretches --
// softmax_split_partial_kernel a stretch's maximum and its sum of exponentials relative to that,
// softmax_split_finish_kernel the row's maximum and sum from its stretches' (in stretch order: the
// same bits on every run) and the stretch's results.  Which rows: one that holds more than one
// part in kSoftmaxLoneRowShare of all the giant rows' entries (the short-row kernel sums them)
// from kSoftmaxLoneSplitRow entries on -- alone, its workgroup's dozens of dependent round trips
// would set the giant-row kernel's time while the other workgroups have finished -- and any row
// of kSoftmaxFarRow entries or more.  A row between those that has many like itself beside it stays
// one workgroup's: its second sweep finds the row in an L2 or the memory-side cache, where the
// stretches' second read comes from memory (2,048 rows of 131,072 entries: 0.52 against 0.67 ms).
// Values are loaded raw and scaled at their first use, so that a row's loads
// are all issued before any of them is waited for.
constexpr int kSoftmaxRegs = 4;
// rows a lane group of G lanes has in flight (whole wavefronts take fewer: their
// workgroup's rows are long, and what the later tiers take they take one after the other)
constexpr int softmax_team_rows(int G) { return G == kWaveSize ? 2 : 4; }
constexpr int kSoftmaxBlockRegs = 16;
constexpr int kSoftmaxGiantRegs = 8;
constexpr int kSoftmaxQuarter = kWaveSize / 4;
constexpr int kSoftmaxQuarterRowMax = kSoftmaxRegs * kSoftmaxQuarter;
constexpr int kSoftmaxWaveRowMax = kSoftmaxRegs * kWaveSize;
constexpr int kSoftmaxLongWaveRowMax = kSoftmaxBlockRegs * kWaveSize;
constexpr int kSoftmaxBlockRowMax = kSoftmaxBlockRegs * kBlockThreads;
constexpr int kSoftmaxGiantThreads = 1024;
constexpr int kSoftmaxSplitRow = 65536;     // rows longer than this are shared out in stretches of kSoftmaxStretch
constexpr int kSoftmaxStretch = 16384;      // entries of a stretch, at least
// A row with more than 1 / kSoftmaxLoneRowShare of the entries of all giant rows is shared out from
// kSoftmaxLoneSplitRow entries on, in shorter stretches.
constexpr int kSoftmaxLoneRowShare = 100;
// From this many entries on a row is shared out whatever the others are like: a workgroup's second
// sweep over it would come from memory, not from an L2, as the stretches' second read does.
constexpr int kSoftmaxFarRow = 1 << 19;
constexpr int kSoftmaxLoneSplitRow = 16384;
constexpr int kSoftmaxLoneStretch = 8192;
constexpr int kSoftmaxMaxStretches = 1024;  // stretches of a row, at most (one per thread of the combining workgroup)
constexpr int kSoftmaxSplitBlocks = 512;   // most workgroups the two stretch kernels start
constexpr int kSoftmaxGiantBlocks = 512;  // most workgroups the giant-row kernel starts
constexpr float kSoftmaxLowest = -3.402823466e38f;

// Lanes per row: the smallest power of two, between 2 and 64, whose groups hold
// a row of mean length in registers.
inline int softmax_group_width(int64_t M, int64_t nnz) {
  const int64_t mean = M > 0 ? (nnz + M - 1) / M : 0;
  int g = 2;
  while (g < kWaveSize && (int64_t)g * kSoftmaxRegs < mean) g *= 2;
  return g;
}

// exp(d) for d <= 0 (every exponential here is taken relative to a maximum) as one multiplication
// and the hardware's 2^x: the library routine costs about ten instructions, and with four of
// them and four divisions per lane and row the short-row kernel was bound by its vector
// instructions, not by memory (31.6 M of them for the 17.8 M entries of a 1 M-row graph: 57 us of
// issue time on 1024 SIMDs).  The product's rounding moves the result by at most |d| * 1.2e-7
// relative: 1e-5 at the edge of the fp32 range, 1e-6 for d = -10.  -inf and the lowest float give 0.
__device__ __forceinline__ float softmax_exp(float d) { return __builtin_amdgcn_exp2f(d * 1.44269504088896341f); }
// 1 / sum for a row's sum of exponentials (>= 1: the maximum's own term), to within one unit in
// the last place; every entry of the row is multiplied by it where it was divided by the sum.
__device__ __forceinline__ float softmax_reciprocal(float sum) { return __builtin_amdgcn_rcpf(sum); }

// A row's entries [lo, hi) for a team of TEAM threads (this one is number t):
// the first REGS * TEAM of them are read into registers, raw ...
// (Every load is issued, the ones past the row's end at the array's last entry, `last`: a load under
// a condition is a branch around it, and the loads of a row would not be in flight together.  What
// those lanes read is replaced when the entries are scaled.)
template <int TEAM, int REGS>
__device__ __forceinline__ void softmax_load(int lo, int hi, int t, const float *vals, int last,
                                             float (&v)[REGS]) {
#pragma unroll
  for (int u = 0; u < REGS; ++u) {
    const int p = lo + t + u * TEAM;
    v[u] = vals[(unsigned)(p < hi ? p : last)];
  }
}

// ... and the three phases on them; `reduce(value, take_max)` combines a value
// over the team.  TAIL: the row may be longer than the registers hold; the
// rest is read once for maximum and sum together and once more for the write.
template <int TEAM, int REGS, bool TAIL, typename Reduce>
__device__ __forceinline__ void softmax_finish(int lo, int hi, int t, const float *vals, float scale,
                                               float *out, float (&v)[REGS], Reduce reduce) {
  float mx = kSoftmaxLowest;
#pragma unroll
  for (int u = 0; u < REGS; ++u) {
    v[u] = lo + t + u * TEAM < hi ? v[u] * scale : kSoftmaxLowest;
    mx = fmaxf(mx, v[u]);
  }
  const int rest = lo + REGS * TEAM + t;  // this thread's first entry beyond the registers
  // The entries beyond the registers are read twice, not three times: the first
  // sweep keeps a running maximum and the sum of exponentials relative to it
  // (rescaled whenever the maximum moves: one exponential per entry either way).
  constexpr int kTailBatch = 8;
  float tail_max = mx, tail_sum = 0.0f;
  if (TAIL) {
    // (kTailBatch loads are issued together in both sweeps: out may alias vals, so
    // the compiler would not move a load above the store of the entry before)
    for (int p0 = rest; p0 < hi; p0 += kTailBatch * TEAM) {
      float raw[kTailBatch];
#pragma unroll
      for (int u = 0; u < kTailBatch; ++u) {
        const int p = p0 + u * TEAM;
        raw[u] = p < hi ? vals[p] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < kTailBatch; ++u) {
        if (p0 + u * TEAM >= hi) break;
        const float x = raw[u] * scale;
        const float e = softmax_exp(-fabsf(x - tail_max));
        const bool higher = x > tail_max;
        tail_sum = higher ? tail_sum * e + 1.0f : tail_sum + e;
        tail_max = higher ? x : tail_max;
      }
    }
    mx = tail_max;
  }
  mx = reduce(mx, true);
  float sum = TAIL ? tail_sum * softmax_exp(tail_max - mx) : 0.0f;
#pragma unroll
  for (int u = 0; u < REGS; ++u) {
    v[u] = softmax_exp(v[u] - mx);  // (past the row's end: the lowest float less the maximum, which gives 0)
    sum += v[u];
  }
  const float inv_sum = softmax_reciprocal(reduce(sum, false));
#pragma unroll
  for (int u = 0; u < REGS; ++u) {
    const int p = lo + t + u * TEAM;
    if (p < hi) out[(unsigned)p] = v[u] * inv_sum;
  }
  if (TAIL) {
    for (int p0 = rest; p0 < hi; p0 += kTailBatch * TEAM) {
      float raw[kTailBatch];
#pragma unroll
      for (int u = 0; u < kTailBatch; ++u) {
        const int p = p0 + u * TEAM;
        raw[u] = p < hi ? vals[p] : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < kTailBatch; ++u) {
        const int p = p0 + u * TEAM;
        if (p < hi) out[p] = softmax_exp(raw[u] * scale - mx) * inv_sum;
      }
    }
  }
}

template <int TEAM, int REGS, bool TAIL, typename Reduce>
__device__ __forceinline__ void softmax_row(int lo, int hi, int t, const float *vals, int last, float scale,
                                            float *out, Reduce reduce) {
  float v[REGS];
  softmax_load<TEAM, REGS>(lo, hi, t, vals, last, v);
  softmax_finish<TEAM, REGS, TAIL>(lo, hi, t, vals, scale, out, v, reduce);
}

template <int WIDTH>
__device__ __forceinline__ float softmax_shuffle_reduce(float v, bool take_max) {
#pragma unroll
  for (int off = WIDTH / 2; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off);
    v = take_max ? fmaxf(v, o) : v + o;
  }
  return v;
}

template <int G>
__global__ __launch_bounds__(kBlockThreads) void softmax_csr_kernel(int M,
                                                                    const int *__restrict__ row_ptr,
                                                                    const float *vals, float scale,
                                                                    float *out, int *giant_count,
                                                                    int *__restrict__ giant_rows, int64_t nnz) {
  // grid.y > 1: several value arrays over one pattern; problem h reads and writes nnz entries
  // further on, and only problem 0 lists the pattern's giant rows (they are the same for all)
  vals += blockIdx.y * nnz;
  out += blockIdx.y * nnz;
  // (no list: the caller has vouched that no row is that long; one that is anyway is left unwritten)
  const bool list_giants = blockIdx.y == 0 && giant_count != nullptr;
  // A lane group takes kTeamRows rows, one from each block of 256 / G consecutive rows
  // the workgroup owns, and requests the entries of all of them before it works on the
  // first: these rows are short, and with one row in flight per group the kernel waits on
  // memory latency rather than bandwidth.
  constexpr int kGroups = kBlockThreads / G;
  constexpr int kTeamRows = softmax_team_rows(G);
  constexpr int kRows = kGroups * kTeamRows;  // rows per workgroup
  __shared__ float s_red[kWavesPerBlock];
  __shared__ int s_lo[kRows], s_hi[kRows];
  // row slots left to the quarter wavefronts [0], the wavefronts with few [1] and with many
  // [2] entries per lane, and the workgroup [3]; [4]: rows left to the giant-row kernel
  __shared__ int s_list[5][kRows];
  __shared__ int s_count[5];
  __shared__ int s_giant_base, s_giant_entries;
  if (threadIdx.x < 5) s_count[threadIdx.x] = 0;
  if (threadIdx.x == 5) s_giant_entries = 0;
  __syncthreads();
  const int t = threadIdx.x % G;
  const int last = (int)nnz - 1;
  // The row pointers of all of the group's rows are requested before any is looked at (a row past
  // the matrix's end reads the last row's and is given no entries).
  int lo[kTeamRows], hi[kTeamRows];
#pragma unroll
  for (int j = 0; j < kTeamRows; ++j) {
    const int64_t row = (int64_t)blockIdx.x * kRows + j * kGroups + threadIdx.x / G;
    const int64_t r = row < M ? row : (int64_t)M - 1;
    lo[j] = row_ptr[r];
    hi[j] = row_ptr[r + 1];
  }
#pragma unroll
  for (int j = 0; j < kTeamRows; ++j) {
    const int slot = j * kGroups + threadIdx.x / G;
    const int64_t row = (int64_t)blockIdx.x * kRows + slot;
    if (row >= M) hi[j] = lo[j];
    const int len = hi[j] - lo[j];
    if (len > G * kSoftmaxRegs) {
      if (t == 0 && len <= kSoftmaxBlockRowMax) {
        const int tier = len > kSoftmaxLongWaveRowMax ? 3
                         : len > kSoftmaxWaveRowMax   ? 2
                                                      : (len > kSoftmaxQuarterRowMax || G >= kSoftmaxQuarter);
        s_lo[slot] = lo[j];
        s_hi[slot] = hi[j];
        s_list[tier][atomicAdd(&s_count[tier], 1)] = slot;  // order only decides which wavefront serves a row
      } else if (t == 0) {
        s_list[4][atomicAdd(&s_count[4], 1)] = (int)row;
        atomicAdd(&s_giant_entries, len);
      }
      hi[j] = lo[j];
    }
  }
  float v[kTeamRows][kSoftmaxRegs];
#pragma unroll
  for (int j = 0; j < kTeamRows; ++j) softmax_load<G, kSoftmaxRegs>(lo[j], hi[j], t, vals, last, v[j]);
#pragma unroll
  for (int j = 0; j < kTeamRows; ++j)
    softmax_finish<G, kSoftmaxRegs, false>(lo[j], hi[j], t, vals, scale, out, v[j], softmax_shuffle_reduce<G>);
  __syncthreads();
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  const int n_quarter = s_count[0], n_wave = s_count[1], n_long_wave = s_count[2], n_block = s_count[3],
            n_giant = s_count[4];
  if (n_giant > 0 && list_giants) {  // uniform over the workgroup; rows are independent, so the list's order is free
    if (threadIdx.x == 0) {
      s_giant_base = atomicAdd(giant_count, n_giant);
      atomicAdd(giant_count + 3, s_giant_entries);  // (all entries of a matrix fit an int)
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n_giant; i += kBlockThreads) giant_rows[s_giant_base + i] = s_list[4][i];
  }
  if (G < kSoftmaxQuarter) {
    constexpr int kTeams = kBlockThreads / kSoftmaxQuarter;
    // (a wavefront none of whose four teams has a row left is done: nothing here waits for the others)
    for (int base = 0; base + w * (kWaveSize / kSoftmaxQuarter) < n_quarter; base += kTeams) {
      const int i = base + (int)threadIdx.x / kSoftmaxQuarter;
      int l = 0, h = 0;
      if (i < n_quarter) {
        const int k = s_list[0][i];
        l = s_lo[k];
        h = s_hi[k];
      }
      softmax_row<kSoftmaxQuarter, kSoftmaxRegs, false>(l, h, lane % kSoftmaxQuarter, vals, last, scale, out,
                                                        softmax_shuffle_reduce<kSoftmaxQuarter>);
    }
  }
  if (G < kWaveSize) {
    for (int i = w; i < n_wave; i += kWavesPerBlock) {
      const int k = s_list[1][i];
      softmax_row<kWaveSize, kSoftmaxRegs, false>(s_lo[k], s_hi[k], lane, vals, last, scale, out,
                                                  softmax_shuffle_reduce<kWaveSize>);
    }
  }
  // up to 1024 entries: still one wavefront per row, sixteen entries per lane, so that the four
  // wavefronts work on four such rows at once and need no barriers
  for (int i = w; i < n_long_wave; i += kWavesPerBlock) {
    const int k = s_list[2][i];
    softmax_row<kWaveSize, kSoftmaxBlockRegs, false>(s_lo[k], s_hi[k], lane, vals, last, scale, out,
                                                     softmax_shuffle_reduce<kWaveSize>);
  }
  for (int i = 0; i < n_block; ++i) {  // uniform over the workgroup
    const int k = s_list[3][i];
    softmax_row<kBlockThreads, kSoftmaxBlockRegs, false>(
        s_lo[k], s_hi[k], (int)threadIdx.x, vals, last, scale, out, [&](float v, bool take_max) {
          v = softmax_shuffle_reduce<kWaveSize>(v, take_max);  // fixed order: lanes, then wavefronts
          __syncthreads();
          if (lane == 0) s_red[w] = v;
          __syncthreads();
          float r = s_red[0];
#pragma unroll
          for (int j = 1; j < kWavesPerBlock; ++j) r = take_max ? fmaxf(r, s_red[j]) : r + s_red[j];
          return r;
        });
  }
}

// counters[0]: giant rows listed; [1]: rows served in stretches; [2]: their stretches in all;
// [3]: entries of the giant rows
__global__ void softmax_reset_kernel(int *counters) {
  if (threadIdx.x < 4) counters[threadIdx.x] = 0;
}

// The rows that are served in stretches, in the caller's workspace: rows[j] = (row, its first
// stretch's number, its stretches, entries per stretch), units[u] = (j, number of the stretch within
// its row), partials[u] = (the stretch's maximum, its sum of exponentials relative to that).
struct SoftmaxSplit {
  int *counters;
  int4 *rows;
  int2 *units;
  float2 *partials;
};

// (maximum, sum of exponentials relative to it) of the entries of a stretch, for every stretch.
__global__ __launch_bounds__(kSoftmaxGiantThreads) void softmax_split_partial_kernel(
    const int *__restrict__ row_ptr, const float *__restrict__ vals, float scale, SoftmaxSplit split) {
  constexpr int kWaves = kSoftmaxGiantThreads / kWaveSize;
  __shared__ float s_red[kWaves];
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  auto reduce = [&](float v, bool take_max) {
    v = softmax_shuffle_reduce<kWaveSize>(v, take_max);  // fixed order: lanes, then wavefronts
    __syncthreads();
    if (lane == 0) s_red[w] = v;
    __syncthreads();
    float r = s_red[0];
#pragma unroll
    for (int j = 1; j < kWaves; ++j) r = take_max ? fmaxf(r, s_red[j]) : r + s_red[j];
    return r;
  };
  const int n_units = split.counters[2];
  for (int u = blockIdx.x; u < n_units; u += gridDim.x) {  // uniform over the workgroup
    const int2 unit = split.units[u];
    const int4 row = split.rows[unit.x];
    const int begin = row_ptr[row.x] + unit.y * row.w;
    const int row_end = row_ptr[row.x + 1];
    const int end = row_end - begin > row.w ? begin + row.w : row_end;  // (no overflow near 2^31 entries)
    constexpr int kBatch = 8;
    float mx = kSoftmaxLowest, sum = 0.0f;
    for (int p0 = begin + (int)threadIdx.x; p0 < end; p0 += kBatch * kSoftmaxGiantThreads) {
      float raw[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const int p = p0 + k * kSoftmaxGiantThreads;
        raw[k] = p < end ? vals[p] : 0.0f;
      }
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        if (p0 + k * kSoftmaxGiantThreads >= end) break;
        const float x = raw[k] * scale;
        const float e = softmax_exp(-fabsf(x - mx));
        const bool higher = x > mx;
        sum = higher ? sum * e + 1.0f : sum + e;
        mx = higher ? x : mx;
      }
    }
    const float unit_max = reduce(mx, true);
    const float unit_sum = reduce(sum * softmax_exp(mx - unit_max), false);  // (a thread without entries: 0 * exp(lowest - max) = 0)
    if (threadIdx.x == 0) split.partials[u] = make_float2(unit_max, unit_sum);
  }
}

// The row's maximum and sum from its stretches', then the stretch's results.
__global__ __launch_bounds__(kSoftmaxGiantThreads) void softmax_split_finish_kernel(
    const int *__restrict__ row_ptr, const float *vals, float scale, float *out, SoftmaxSplit split) {
  constexpr int kWaves = kSoftmaxGiantThreads / kWaveSize;
  __shared__ float s_red[kWaves];
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  auto reduce = [&](float v, bool take_max) {
    v = softmax_shuffle_reduce<kWaveSize>(v, take_max);
    __syncthreads();
    if (lane == 0) s_red[w] = v;
    __syncthreads();
    float r = s_red[0];
#pragma unroll
    for (int j = 1; j < kWaves; ++j) r = take_max ? fmaxf(r, s_red[j]) : r + s_red[j];
    return r;
  };
  const int n_units = split.counters[2];
  for (int u = blockIdx.x; u < n_units; u += gridDim.x) {  // uniform over the workgroup
    const int2 unit = split.units[u];
    const int4 row = split.rows[unit.x];
    float2 part = make_float2(kSoftmaxLowest, 0.0f);  // thread t: stretch t of the row
    if ((int)threadIdx.x < row.z) part = split.partials[row.y + threadIdx.x];
    const float row_max = reduce(part.x, true);
    const float inv_sum = softmax_reciprocal(reduce(part.y * softmax_exp(part.x - row_max), false));
    const int begin = row_ptr[row.x] + unit.y * row.w;
    const int row_end = row_ptr[row.x + 1];
    const int end = row_end - begin > row.w ? begin + row.w : row_end;  // (no overflow near 2^31 entries)
    constexpr int kBatch = 8;  // (loads issued together: out may alias vals, see softmax_finish)
    for (int p0 = begin + (int)threadIdx.x; p0 < end; p0 += kBatch * kSoftmaxGiantThreads) {
      float raw[kBatch];
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const int p = p0 + k * kSoftmaxGiantThreads;
        raw[k] = p < end ? vals[p] : 0.0f;
      }
#pragma unroll
      for (int k = 0; k < kBatch; ++k) {
        const int p = p0 + k * kSoftmaxGiantThreads;
        if (p < end) out[p] = softmax_exp(raw[k] * scale - row_max) * inv_sum;
      }
    }
  }
}

__global__ __launch_bounds__(kSoftmaxGiantThreads) void softmax_csr_giant_kernel(
    const int *__restrict__ row_ptr, const float *vals, float scale, float *out,
    const int *__restrict__ giant_count, const int *__restrict__ giant_rows, int64_t nnz, SoftmaxSplit split) {
  constexpr int kWaves = kSoftmaxGiantThreads / kWaveSize;
  __shared__ float s_red[kWaves];
  __shared__ int s_claim[2];
  vals += blockIdx.y * nnz;  // problem blockIdx.y of a batch over one pattern
  out += blockIdx.y * nnz;
  const int n = *giant_count;
  const int giant_entries = giant_count[3];
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  const int t = (int)threadIdx.x;
  const int last = (int)nnz - 1;
  auto reduce = [&](float v, bool take_max) {
    v = softmax_shuffle_reduce<kWaveSize>(v, take_max);  // fixed order: lanes, then wavefronts
    __syncthreads();
    if (lane == 0) s_red[w] = v;
    __syncthreads();
    float r = s_red[0];
#pragma unroll
    for (int j = 1; j < kWaves; ++j) r = take_max ? fmaxf(r, s_red[j]) : r + s_red[j];
    return r;
  };
  // A row that is served in stretches (see the head of this section) is entered in their list (by
  // problem 0 of a batch: the pattern is the same for all) and skipped here.  Uniform over the workgroup.
  auto leave_to_the_stretch_kernels = [&](int row, int lo, int &hi) {
    const int len = hi - lo;
    const bool lone = (int64_t)len * kSoftmaxLoneRowShare > giant_entries;
    const int limit = lone ? kSoftmaxLoneSplitRow : len >= kSoftmaxFarRow ? kSoftmaxSplitRow : len;
    if (split.rows == nullptr || len <= limit) return;
    hi = lo;
    if (blockIdx.y != 0) return;
    const int least = len > kSoftmaxSplitRow ? kSoftmaxStretch : kSoftmaxLoneStretch;
    int stretch = (len + kSoftmaxMaxStretches - 1) / kSoftmaxMaxStretches;
    stretch = stretch < least ? least : (stretch + 1023) / 1024 * 1024;
    const int n_units = (len + stretch - 1) / stretch;
    __syncthreads();  // (s_claim may still be read from the row before)
    if (threadIdx.x == 0) {
      s_claim[0] = atomicAdd(split.counters + 1, 1);
      s_claim[1] = atomicAdd(split.counters + 2, n_units);
    }
    __syncthreads();
    const int j = s_claim[0], first = s_claim[1];
    if (threadIdx.x == 0) split.rows[j] = make_int4(row, first, n_units, stretch);
    if ((int)threadIdx.x < n_units) split.units[first + threadIdx.x] = make_int2(j, (int)threadIdx.x);
  };
  // The next row's first entries are requested before this row's phases begin,
  // so that its memory latency passes behind their barriers.  (out may alias
  // vals: rows do not overlap, so the early read sees the row unchanged.)
  int i = blockIdx.x;
  if (i >= n) return;
  int row = giant_rows[i];
  int lo = row_ptr[row], hi = row_ptr[row + 1];
  leave_to_the_stretch_kernels(row, lo, hi);
  float v[kSoftmaxGiantRegs];
  softmax_load<kSoftmaxGiantThreads, kSoftmaxGiantRegs>(lo, hi, t, vals, last, v);
  for (;;) {  // uniform over the workgroup
    const int i_next = i + gridDim.x;
    int lo_next = 0, hi_next = 0;
    float v_next[kSoftmaxGiantRegs];
    if (i_next < n) {
      const int row_next = giant_rows[i_next];
      lo_next = row_ptr[row_next];
      hi_next = row_ptr[row_next + 1];
      leave_to_the_stretch_kernels(row_next, lo_next, hi_next);
    }
    softmax_load<kSoftmaxGiantThreads, kSoftmaxGiantRegs>(lo_next, hi_next, t, vals, last, v_next);
    softmax_finish<kSoftmaxGiantThreads, kSoftmaxGiantRegs, true>(lo, hi, t, vals, scale, out, v, reduce);
    if (i_next >= n) break;
    i = i_next;
    lo = lo_next;
    hi = hi_next;
#pragma unroll
    for (int u = 0; u < kSoftmaxGiantRegs; ++u) v[u] = v_next[u];
  }
}

// Rows the giant-row list must have room for: a row is listed only if it has
// more than kSoftmaxBlockRowMax entries.
inline int64_t softmax_giant_capacity(int64_t M, int64_t nnz) {
  const int64_t by_entries = nnz / (kSoftmaxBlockRowMax + 1);
  return by_entries < M ? by_entries : M;
}

// Rows that may have to be served in stretches (those beyond kSoftmaxSplitRow entries; of those
// beyond kSoftmaxLoneSplitRow, the fewer than kSoftmaxLoneRowShare that can each hold more than that
// part of the giant rows' entries), and stretches in all.
inline int64_t softmax_split_rows(int64_t M, int64_t nnz) {
  int64_t lone = nnz / (kSoftmaxLoneSplitRow + 1);
  if (lone > kSoftmaxLoneRowShare) lone = kSoftmaxLoneRowShare;
  const int64_t by_entries = nnz / (kSoftmaxSplitRow + 1) + lone;
  return by_entries < M ? by_entries : M;
}
inline int64_t softmax_split_units(int64_t M, int64_t nnz) {
  const int64_t rows = softmax_split_rows(M, nnz);
  return rows > 0 ? nnz / kSoftmaxLoneStretch + rows : 0;
}
inline size_t softmax_round_256(size_t v) { return (v + 255) / 256 * 256; }

// Workspace: three counters (256 bytes), the giant rows' numbers, then -- only when a row can be
// long enough -- the rows served in stretches, the stretches and their partial results.
inline size_t softmax_workspace_bytes(int64_t M, int64_t nnz) {
  const int64_t rows = softmax_giant_capacity(M, nnz);
  if (rows <= 0) return 0;
  const size_t split_rows = (size_t)softmax_split_rows(M, nnz), units = (size_t)softmax_split_units(M, nnz);
  return 256 + softmax_round_256((size_t)rows * sizeof(int)) + softmax_round_256(split_rows * sizeof(int4)) +
         softmax_round_256(units * sizeof(int2)) + softmax_round_256(units * sizeof(float2));
}

inline SoftmaxSplit softmax_split_layout(void *workspace, int64_t M, int64_t nnz) {
  SoftmaxSplit split{nullptr, nullptr, nullptr, nullptr};
  const size_t split_rows = (size_t)softmax_split_rows(M, nnz), units = (size_t)softmax_split_units(M, nnz);
  if (split_rows == 0) return split;
  char *base = static_cast<char *>(workspace);
  size_t at = 256 + softmax_round_256((size_t)softmax_giant_capacity(M, nnz) * sizeof(int));
  split.counters = reinterpret_cast<int *>(base);
  split.rows = reinterpret_cast<int4 *>(base + at);
  at += softmax_round_256(split_rows * sizeof(int4));
  split.units = reinterpret_cast<int2 *>(base + at);
  at += softmax_round_256(units * sizeof(int2));
  split.partials = reinterpret_cast<float2 *>(base + at);
  return split;
}

// ---- CSR -> coordinate rows ---------------------------------------------------
__global__ __launch_bounds__(kBlockThreads) void csr_row_indices_kernel(
    int M, int64_t nnz, const int *__restrict__ row_ptr, int *__restrict__ row_idx) {
  const int lane = wave_lane();
  const int64_t wave = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWaveSize;
  const int64_t first = wave * kWaveSize;
  if (first >= nnz) return;
  const int64_t last = first + kWaveSize < nnz ? first + kWaveSize : nnz;
  auto end_key = [&](int i) { return (int64_t)row_ptr[i + 1]; };
  int lo = wave_count_below(M, first + 1, end_key);  // row of the first entry
  int hi = wave_count_below(M, last, end_key);       // row of the last entry
  const int64_t p = first + lane;
  if (p >= last) return;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)row_ptr[mid + 1] <= p) lo = mid + 1; else hi = mid;
  }
  row_idx[p] = lo;
}

// ---- coordinate rows -> CSR row pointer -------------------------------------------
// row_ptr[r] = number of entries whose row is below r, found by bisection in the
// sorted row coordinates (every thread one r: the work is the same whatever the
// gaps between rows).  The same threads look at the coordinates themselves, one
// pair of neighbours each, and raise *unsorted if a row lies outside [0, M) or
// below its predecessor; row_ptr is meaningless then.
__global__ __launch_bounds__(kBlockThreads) void coo_row_ptr_kernel(
    int M, int64_t nnz, const int *__restrict__ row_idx, int *__restrict__ row_ptr,
    int *__restrict__ unsorted) {
  const int64_t stride = (int64_t)gridDim.x * kBlockThreads;
  const int64_t first = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x;
  for (int64_t r = first; r <= M; r += stride) {
    int64_t lo = 0, hi = nnz;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (row_idx[mid] < r) lo = mid + 1; else hi = mid;
    }
    row_ptr[r] = (int)lo;
  }
  bool bad = false;
  for (int64_t p = first; p < nnz; p += stride) {
    const int row = row_idx[p];
    bad |= row < 0 || row >= M || (p > 0 && row_idx[p - 1] > row);
  }
  if (bad) *unsorted = 1;  // every writer stores the same value
}

// Whether some element of vals differs from `value` (a NaN differs from everything).
__global__ void values_differ_clear_kernel(int *differ) { *differ = 0; }
__global__ __launch_bounds__(kBlockThreads) void values_differ_kernel(int64_t n, const float *__restrict__ vals,
                                                                       float value, int *__restrict__ differ) {
  bool any = false;
  const int64_t stride = (int64_t)gridDim.x * kBlockThreads;
  for (int64_t i = (int64_t)blockIdx.x * kBlockThreads + threadIdx.x; i < n; i += stride) any |= !(vals[i] == value);
  if (__ballot(any) != 0 && wave_lane() == 0) atomicOr(differ, 1);
}

}  // namespace scorch

extern "C" {

int scorch_hip_abi_version(void) { return SCORCH_HIP_ABI_VERSION; }

const char *scorch_hip_last_error(void) { return scorch::error_buffer(); }

int scorch_hip_timing_begin(void) {
  scorch::LaunchMarks *m = scorch::launch_marks();
  if (!m->created) {
    for (int i = 0; i < scorch::kMaxLaunchMarks; ++i) SCORCH_HIP_CHECK(hipEventCreate(&m->ev[i]));
    m->created = true;
  }
  m->count = 0;
  m->active = true;
  return SCORCH_HIP_OK;
}

int scorch_hip_timing_end(float *interval_ms, int capacity, int *count) {
  const char *fn = "scorch_hip_timing_end";
  scorch::LaunchMarks *m = scorch::launch_marks();
  SCORCH_REQUIRE(m->active, "%s: no scorch_hip_timing_begin on this thread", fn);
  m->active = false;
  SCORCH_REQUIRE(count != nullptr && (capacity == 0 || interval_ms != nullptr), "%s: NULL output", fn);
  const int intervals = m->count > 0 ? m->count - 1 : 0;
  *count = intervals;
  if (m->count > 0) SCORCH_HIP_CHECK(hipEventSynchronize(m->ev[m->count - 1]));
  for (int i = 0; i < intervals && i < capacity; ++i)
    SCORCH_HIP_CHECK(hipEventElapsedTime(&interval_ms[i], m->ev[i], m->ev[i + 1]));
  return SCORCH_HIP_OK;
}

size_t scorch_hip_softmax_csr_workspace_bytes(int64_t M, int64_t nnz) {
  if (M <= 0 || nnz <= 0) return 0;
  return scorch::softmax_workspace_bytes(M, nnz);
}

static int softmax_csr_entry(const char *fn, int64_t batch, int64_t M, int64_t nnz, const int32_t *row_ptr,
                             const float *vals, float scale, float *out, void *workspace,
                             size_t workspace_bytes, void *stream, int64_t longest_row = -1) {
  if (batch < 0 || batch > 65535)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: batch=%lld is outside [0, 65535]", fn, (long long)batch);
  if (M < 0 || nnz < 0) return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size", fn);
  if (M >= INT32_MAX || nnz > INT32_MAX)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  SCORCH_REQUIRE(row_ptr != nullptr, "%s: row_ptr is NULL", fn);
  if (batch == 0 || M == 0 || nnz == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(vals && out, "%s: NULL value array", fn);
  // longest_row >= 0: the caller vouches that no row has more entries than that.  Up to 4096 there is
  // no list of giant rows to reset, fill or serve; up to kSoftmaxLoneSplitRow no row is served in stretches.
  const bool short_rows = longest_row >= 0 && longest_row <= 4096;
  const bool no_stretches = longest_row >= 0 && longest_row <= scorch::kSoftmaxLoneSplitRow;
  const size_t need = short_rows ? 0 : scorch::softmax_workspace_bytes(M, nnz);
  if (need > 0 && (!workspace || workspace_bytes < need))
    return scorch::fail(SCORCH_HIP_EWORKSPACE, "%s: workspace of %zu bytes needed, %zu given", fn, need,
                        workspace ? workspace_bytes : (size_t)0);
  SCORCH_REQUIRE(need == 0 || scorch::aligned_to(workspace, 256), "%s: workspace must be 256-byte aligned", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // workspace: the number of giant rows, then (256 bytes on) their row numbers
  int *giant_count = static_cast<int *>(workspace);
  int *giant_rows = need > 0 ? giant_count + 64 : nullptr;
  if (need > 0) {
    scorch::softmax_reset_kernel<<<1, scorch::kWaveSize, 0, s>>>(giant_count);
    SCORCH_HIP_CHECK(hipGetLastError());
  }
  const int g = scorch::softmax_group_width(M, nnz);
  const int64_t rows_per_block = scorch::kBlockThreads / g * scorch::softmax_team_rows(g);
  const dim3 grid((unsigned)((M + rows_per_block - 1) / rows_per_block), (unsigned)batch);
  const int m = (int)M;
#define SCORCH_SOFTMAX(G)                                                                               \
  scorch::softmax_csr_kernel<G><<<grid, scorch::kBlockThreads, 0, s>>>(m, row_ptr, vals, scale, out, \
                                                                       giant_count, giant_rows, nnz)
  switch (g) {
    case 2: SCORCH_SOFTMAX(2); break;
    case 4: SCORCH_SOFTMAX(4); break;
    case 8: SCORCH_SOFTMAX(8); break;
    case 16: SCORCH_SOFTMAX(16); break;
    case 32: SCORCH_SOFTMAX(32); break;
    default: SCORCH_SOFTMAX(64); break;
  }
#undef SCORCH_SOFTMAX
  SCORCH_HIP_CHECK(hipGetLastError());
  if (need > 0) {  // else no row can be that long
    int64_t most = scorch::softmax_giant_capacity(M, nnz);
    if (most > scorch::kSoftmaxGiantBlocks) most = scorch::kSoftmaxGiantBlocks;
    if (batch > 1 && most > 128) most = 128;  // every problem brings its own workgroups
    const dim3 giant_grid((unsigned)most, (unsigned)batch);
    const scorch::SoftmaxSplit split =
        no_stretches ? scorch::SoftmaxSplit{} : scorch::softmax_split_layout(workspace, M, nnz);
    scorch::softmax_csr_giant_kernel<<<giant_grid, scorch::kSoftmaxGiantThreads, 0, s>>>(
        row_ptr, vals, scale, out, giant_count, giant_rows, nnz, split);
    SCORCH_HIP_CHECK(hipGetLastError());
    if (split.rows != nullptr) {  // a row can be long enough to be served in stretches
      int64_t blocks = scorch::softmax_split_units(M, nnz);
      if (blocks > scorch::kSoftmaxSplitBlocks) blocks = scorch::kSoftmaxSplitBlocks;
      // the stretches' partial results are one problem's: the problems of a batch take their turns
      for (int64_t h = 0; h < batch; ++h) {
        scorch::softmax_split_partial_kernel<<<dim3((unsigned)blocks), scorch::kSoftmaxGiantThreads, 0, s>>>(
            row_ptr, vals + h * nnz, scale, split);
        SCORCH_HIP_CHECK(hipGetLastError());
        scorch::softmax_split_finish_kernel<<<dim3((unsigned)blocks), scorch::kSoftmaxGiantThreads, 0, s>>>(
            row_ptr, vals + h * nnz, scale, out + h * nnz, split);
        SCORCH_HIP_CHECK(hipGetLastError());
      }
    }
  }
  return SCORCH_HIP_OK;
}

int scorch_hip_softmax_csr_f32(int64_t M, int64_t nnz, const int32_t *row_ptr, const float *vals,
                               float scale, float *out, void *workspace, size_t workspace_bytes,
                               void *stream) {
  return softmax_csr_entry("scorch_hip_softmax_csr_f32", 1, M, nnz, row_ptr, vals, scale, out, workspace,
                           workspace_bytes, stream);
}

int scorch_hip_softmax_csr_batched_f32(int64_t batch, int64_t M, int64_t nnz, const int32_t *row_ptr,
                                       const float *vals, float scale, float *out, void *workspace,
                                       size_t workspace_bytes, void *stream) {
  return softmax_csr_entry("scorch_hip_softmax_csr_batched_f32", batch, M, nnz, row_ptr, vals, scale, out,
                           workspace, workspace_bytes, stream);
}

int scorch_hip_softmax_csr_known_rows_f32(int64_t batch, int64_t M, int64_t nnz, int64_t longest_row,
                                          const int32_t *row_ptr, const float *vals, float scale, float *out,
                                          void *workspace, size_t workspace_bytes, void *stream) {
  if (longest_row < 0)
    return scorch::fail(SCORCH_HIP_EINVAL, "scorch_hip_softmax_csr_known_rows_f32: longest_row=%lld",
                        (long long)longest_row);
  return softmax_csr_entry("scorch_hip_softmax_csr_known_rows_f32", batch, M, nnz, row_ptr, vals, scale, out,
                           workspace, workspace_bytes, stream, longest_row);
}

int scorch_hip_csr_row_indices(int64_t M, int64_t nnz, const int32_t *row_ptr, int32_t *row_idx,
                               void *stream) {
  const char *fn = "scorch_hip_csr_row_indices";
  if (M < 0 || nnz < 0) return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size", fn);
  if (M >= INT32_MAX || nnz > INT32_MAX)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  SCORCH_REQUIRE(row_ptr != nullptr, "%s: row_ptr is NULL", fn);
  if (nnz == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(M > 0, "%s: nnz=%lld with no rows", fn, (long long)nnz);
  SCORCH_REQUIRE(row_idx != nullptr, "%s: row_idx is NULL", fn);
  const int64_t waves = (nnz + scorch::kWaveSize - 1) / scorch::kWaveSize;
  const dim3 grid((unsigned)((waves + scorch::kWavesPerBlock - 1) / scorch::kWavesPerBlock));
  scorch::csr_row_indices_kernel<<<grid, scorch::kBlockThreads, 0, static_cast<hipStream_t>(stream)>>>(
      (int)M, nnz, row_ptr, row_idx);
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

int scorch_hip_coo_row_ptr(int64_t M, int64_t nnz, const int32_t *row_idx, int32_t *row_ptr,
                           int32_t *unsorted, void *stream) {
  const char *fn = "scorch_hip_coo_row_ptr";
  if (M < 0 || nnz < 0) return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size", fn);
  if (M >= INT32_MAX || nnz > INT32_MAX)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  SCORCH_REQUIRE(row_ptr != nullptr && unsorted != nullptr, "%s: NULL output", fn);
  SCORCH_REQUIRE(nnz == 0 || row_idx != nullptr, "%s: row_idx is NULL", fn);
  const int64_t items = M + 1 > nnz ? M + 1 : nnz;
  int64_t blocks = (items + scorch::kBlockThreads - 1) / scorch::kBlockThreads;
  if (blocks > 65536) blocks = 65536;  // the kernel strides
  scorch::coo_row_ptr_kernel<<<dim3((unsigned)blocks), scorch::kBlockThreads, 0,
                               static_cast<hipStream_t>(stream)>>>((int)M, nnz, row_idx, row_ptr, unsorted);
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

int scorch_hip_values_differ_f32(int64_t n, const float *vals, float value, int32_t *differ, void *stream) {
  const char *fn = "scorch_hip_values_differ_f32";
  if (n < 0) return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size", fn);
  SCORCH_REQUIRE(differ != nullptr, "%s: NULL output", fn);
  SCORCH_REQUIRE(n == 0 || vals != nullptr, "%s: vals is NULL", fn);
  SCORCH_REQUIRE(scorch::aligned_to(vals, 4) && scorch::aligned_to(differ, 4), "%s: arrays must be 4-byte aligned", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  scorch::values_differ_clear_kernel<<<1, 1, 0, s>>>(differ);
  SCORCH_HIP_CHECK(hipGetLastError());
  if (n == 0) return SCORCH_HIP_OK;
  int64_t blocks = (n + scorch::kBlockThreads * 8 - 1) / (scorch::kBlockThreads * 8);
  if (blocks > 4096) blocks = 4096;  // the kernel strides
  scorch::values_differ_kernel<<<dim3((unsigned)blocks), scorch::kBlockThreads, 0, s>>>(n, vals, value, differ);
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}

}  // extern "C"

SCORCH_DEFINE_PRELOAD(misc)
