// Smaller kernels around the SpMM/SDDMM path: CSR row softmax, the
// CSR -> coordinate row expansion, and the library's error/version calls.
#include "common.hpp"

namespace scorch {

char *error_buffer() {
  static thread_local char buf[kErrorBufferBytes] = {0};
  return buf;
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
//   up to 2048 entries               the whole workgroup, one row after the other.
// In all of these a row sits in registers between the phases and is read from
// memory once.  Rows beyond 2048 entries are left to softmax_csr_giant_kernel:
// workgroups of 1024 threads that look through 1024 row lengths each and sweep
// the giant rows among them, the first 8192 entries in registers and the rest
// re-read from cache.
constexpr int kSoftmaxRegs = 4;
constexpr int kSoftmaxBlockRegs = 8;
constexpr int kSoftmaxQuarter = kWaveSize / 4;
constexpr int kSoftmaxQuarterRowMax = kSoftmaxRegs * kSoftmaxQuarter;
constexpr int kSoftmaxWaveRowMax = kSoftmaxRegs * kWaveSize;
constexpr int kSoftmaxBlockRowMax = kSoftmaxBlockRegs * kBlockThreads;
constexpr int kSoftmaxGiantThreads = 1024;
constexpr float kSoftmaxLowest = -3.402823466e38f;

// Lanes per row: the smallest power of two, between 2 and 64, whose groups hold
// a row of mean length in registers.
inline int softmax_group_width(int64_t M, int64_t nnz) {
  const int64_t mean = M > 0 ? (nnz + M - 1) / M : 0;
  int g = 2;
  while (g < kWaveSize && (int64_t)g * kSoftmaxRegs < mean) g *= 2;
  return g;
}

// The three phases for entries [lo, hi) by a team of TEAM threads (this one is
// number t); `reduce(value, take_max)` combines a value over the team.
template <int TEAM, int REGS, bool TAIL, typename Reduce>
__device__ __forceinline__ void softmax_row(int lo, int hi, int t, const float *vals, float scale,
                                            float *out, Reduce reduce) {
  float v[REGS];
  float mx = kSoftmaxLowest;
#pragma unroll
  for (int u = 0; u < REGS; ++u) {
    const int p = lo + t + u * TEAM;
    v[u] = p < hi ? vals[p] * scale : kSoftmaxLowest;
    mx = fmaxf(mx, v[u]);
  }
  const int rest = lo + REGS * TEAM + t;  // this thread's first entry beyond the registers
  if (TAIL) {
#pragma unroll 8
    for (int p = rest; p < hi; p += TEAM) mx = fmaxf(mx, vals[p] * scale);
  }
  mx = reduce(mx, true);
  float sum = 0.0f;
#pragma unroll
  for (int u = 0; u < REGS; ++u) {
    v[u] = lo + t + u * TEAM < hi ? expf(v[u] - mx) : 0.0f;
    sum += v[u];
  }
  if (TAIL) {
#pragma unroll 8
    for (int p = rest; p < hi; p += TEAM) sum += expf(vals[p] * scale - mx);
  }
  sum = reduce(sum, false);
#pragma unroll
  for (int u = 0; u < REGS; ++u) {
    const int p = lo + t + u * TEAM;
    if (p < hi) out[p] = v[u] / sum;
  }
  if (TAIL) {
#pragma unroll 8
    for (int p = rest; p < hi; p += TEAM) out[p] = expf(vals[p] * scale - mx) / sum;
  }
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
                                                                    float *out) {
  constexpr int kRows = kBlockThreads / G;  // rows per workgroup
  __shared__ float s_red[kWavesPerBlock];
  __shared__ int s_lo[kRows], s_hi[kRows];
  // row slots left to the quarter wavefronts [0], the wavefronts [1] and the workgroup [2]
  __shared__ int s_list[3][kRows];
  __shared__ int s_count[3];
  if (threadIdx.x < 3) s_count[threadIdx.x] = 0;
  __syncthreads();
  const int slot = threadIdx.x / G;
  const int t = threadIdx.x % G;
  const int64_t row = (int64_t)blockIdx.x * kRows + slot;
  int lo = 0, hi = 0;
  if (row < M) {
    lo = row_ptr[row];
    hi = row_ptr[row + 1];
  }
  const int len = hi - lo;
  if (len > G * kSoftmaxRegs) {
    if (t == 0 && len <= kSoftmaxBlockRowMax) {
      const int tier = len > kSoftmaxWaveRowMax ? 2 : (len > kSoftmaxQuarterRowMax || G >= kSoftmaxQuarter);
      s_lo[slot] = lo;
      s_hi[slot] = hi;
      s_list[tier][atomicAdd(&s_count[tier], 1)] = slot;  // order only decides which wavefront serves a row
    }
    hi = lo;
  }
  softmax_row<G, kSoftmaxRegs, false>(lo, hi, t, vals, scale, out, softmax_shuffle_reduce<G>);
  __syncthreads();
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  const int n_quarter = s_count[0], n_wave = s_count[1], n_block = s_count[2];
  if (G < kSoftmaxQuarter) {
    constexpr int kTeams = kBlockThreads / kSoftmaxQuarter;
    for (int base = 0; base < n_quarter; base += kTeams) {  // uniform over the workgroup
      const int i = base + (int)threadIdx.x / kSoftmaxQuarter;
      int l = 0, h = 0;
      if (i < n_quarter) {
        const int k = s_list[0][i];
        l = s_lo[k];
        h = s_hi[k];
      }
      softmax_row<kSoftmaxQuarter, kSoftmaxRegs, false>(l, h, lane % kSoftmaxQuarter, vals, scale, out,
                                                        softmax_shuffle_reduce<kSoftmaxQuarter>);
    }
  }
  if (G < kWaveSize) {
    for (int i = w; i < n_wave; i += kWavesPerBlock) {
      const int k = s_list[1][i];
      softmax_row<kWaveSize, kSoftmaxRegs, false>(s_lo[k], s_hi[k], lane, vals, scale, out,
                                                  softmax_shuffle_reduce<kWaveSize>);
    }
  }
  for (int i = 0; i < n_block; ++i) {  // uniform over the workgroup
    const int k = s_list[2][i];
    softmax_row<kBlockThreads, kSoftmaxBlockRegs, false>(
        s_lo[k], s_hi[k], (int)threadIdx.x, vals, scale, out, [&](float v, bool take_max) {
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

__global__ __launch_bounds__(kSoftmaxGiantThreads) void softmax_csr_giant_kernel(
    int M, const int *__restrict__ row_ptr, const float *vals, float scale, float *out) {
  constexpr int kWaves = kSoftmaxGiantThreads / kWaveSize;
  __shared__ float s_red[kWaves];
  __shared__ int s_lo[kSoftmaxGiantThreads], s_hi[kSoftmaxGiantThreads];
  __shared__ int s_count;
  if (threadIdx.x == 0) s_count = 0;
  __syncthreads();
  const int64_t row = (int64_t)blockIdx.x * kSoftmaxGiantThreads + threadIdx.x;
  if (row < M) {
    const int lo = row_ptr[row], hi = row_ptr[row + 1];
    if (hi - lo > kSoftmaxBlockRowMax) {
      const int k = atomicAdd(&s_count, 1);  // rows are independent: their order is free
      s_lo[k] = lo;
      s_hi[k] = hi;
    }
  }
  __syncthreads();
  const int n = s_count;
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
  for (int i = 0; i < n; ++i) {  // uniform over the workgroup
    softmax_row<kSoftmaxGiantThreads, kSoftmaxBlockRegs, true>(
        s_lo[i], s_hi[i], (int)threadIdx.x, vals, scale, out, [&](float v, bool take_max) {
          v = softmax_shuffle_reduce<kWaveSize>(v, take_max);  // fixed order: lanes, then wavefronts
          __syncthreads();
          if (lane == 0) s_red[w] = v;
          __syncthreads();
          float r = s_red[0];
#pragma unroll
          for (int j = 1; j < kWaves; ++j) r = take_max ? fmaxf(r, s_red[j]) : r + s_red[j];
          return r;
        });
  }
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

}  // namespace scorch

extern "C" {

int scorch_hip_abi_version(void) { return SCORCH_HIP_ABI_VERSION; }

const char *scorch_hip_last_error(void) { return scorch::error_buffer(); }

int scorch_hip_softmax_csr_f32(int64_t M, int64_t nnz, const int32_t *row_ptr, const float *vals,
                               float scale, float *out, void *stream) {
  const char *fn = "scorch_hip_softmax_csr_f32";
  if (M < 0 || nnz < 0) return scorch::fail(SCORCH_HIP_EINVAL, "%s: negative size", fn);
  if (M >= INT32_MAX || nnz > INT32_MAX)
    return scorch::fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  SCORCH_REQUIRE(row_ptr != nullptr, "%s: row_ptr is NULL", fn);
  if (M == 0 || nnz == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(vals && out, "%s: NULL value array", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int g = scorch::softmax_group_width(M, nnz);
  const int64_t rows_per_block = scorch::kBlockThreads / g;
  const dim3 grid((unsigned)((M + rows_per_block - 1) / rows_per_block));
  const int m = (int)M;
  switch (g) {
    case 2: scorch::softmax_csr_kernel<2><<<grid, scorch::kBlockThreads, 0, s>>>(m, row_ptr, vals, scale, out); break;
    case 4: scorch::softmax_csr_kernel<4><<<grid, scorch::kBlockThreads, 0, s>>>(m, row_ptr, vals, scale, out); break;
    case 8: scorch::softmax_csr_kernel<8><<<grid, scorch::kBlockThreads, 0, s>>>(m, row_ptr, vals, scale, out); break;
    case 16: scorch::softmax_csr_kernel<16><<<grid, scorch::kBlockThreads, 0, s>>>(m, row_ptr, vals, scale, out); break;
    case 32: scorch::softmax_csr_kernel<32><<<grid, scorch::kBlockThreads, 0, s>>>(m, row_ptr, vals, scale, out); break;
    default: scorch::softmax_csr_kernel<64><<<grid, scorch::kBlockThreads, 0, s>>>(m, row_ptr, vals, scale, out); break;
  }
  SCORCH_HIP_CHECK(hipGetLastError());
  if (nnz > scorch::kSoftmaxBlockRowMax) {  // else no row can be that long
    const dim3 giant_grid((unsigned)((M + scorch::kSoftmaxGiantThreads - 1) / scorch::kSoftmaxGiantThreads));
    scorch::softmax_csr_giant_kernel<<<giant_grid, scorch::kSoftmaxGiantThreads, 0, s>>>(m, row_ptr, vals, scale, out);
    SCORCH_HIP_CHECK(hipGetLastError());
  }
  return SCORCH_HIP_OK;
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

}  // extern "C"
