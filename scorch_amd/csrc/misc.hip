// Smaller kernels around the SpMM/SDDMM path: CSR row softmax, the
// CSR -> coordinate row expansion, and the library's error/version calls.
#include "common.hpp"

namespace scorch {

char *error_buffer() {
  static thread_local char buf[kErrorBufferBytes] = {0};
  return buf;
}

// Lanes per row for the group-per-row kernels: the power of two nearest above
// the mean row length, between 2 and 64.
inline int group_width(int64_t M, int64_t nnz) {
  const int64_t mean = M > 0 ? (nnz + M - 1) / M : 0;
  int g = 2;
  while (g < kWaveSize && g < mean) g *= 2;
  return g;
}

// ---- CSR row softmax ----------------------------------------------------------
// One group of G lanes per row (rows of up to kSoftmaxLongRow entries); three
// sweeps over the row (maximum, sum of exponentials, normalised write).  The row is re-read from cache, not kept in
// registers, so any row length works.
constexpr int kSoftmaxLongRow = 256;   // longer rows get a whole workgroup
constexpr int kSoftmaxLongWorkgroups = 2048;

template <int G>
__global__ __launch_bounds__(kBlockThreads) void softmax_csr_kernel(int M,
                                                                    const int *__restrict__ row_ptr,
                                                                    const float *vals, float scale,
                                                                    float *out) {
  const int64_t group = ((int64_t)blockIdx.x * kBlockThreads + threadIdx.x) / G;
  const int t = threadIdx.x % G;
  const bool live = group < M;
  int lo = 0, hi = 0;
  if (live) {
    lo = row_ptr[group];
    hi = row_ptr[group + 1];
    if (hi - lo > kSoftmaxLongRow) hi = lo;  // softmax_csr_long_kernel owns this row
  }
  float mx = -3.402823466e38f;
  for (int p = lo + t; p < hi; p += G) mx = fmaxf(mx, vals[p] * scale);
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off));
  float sum = 0.0f;
  for (int p = lo + t; p < hi; p += G) sum += expf(vals[p] * scale - mx);
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off);
  for (int p = lo + t; p < hi; p += G) out[p] = expf(vals[p] * scale - mx) / sum;
}

// Rows longer than kSoftmaxLongRow: one workgroup per row, the same three sweeps
// with workgroup-wide reductions (fixed order: lanes, then wavefronts).  A fixed
// pool of workgroups scans the row pointer for such rows.
__device__ __forceinline__ float block_reduce(float v, float *scratch, bool take_max) {
  const int lane = wave_lane();
  const int w = threadIdx.x / kWaveSize;
#pragma unroll
  for (int off = kWaveSize / 2; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off);
    v = take_max ? fmaxf(v, o) : v + o;
  }
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  float r = scratch[0];
#pragma unroll
  for (int i = 1; i < kWavesPerBlock; ++i) r = take_max ? fmaxf(r, scratch[i]) : r + scratch[i];
  return r;
}

__global__ __launch_bounds__(kBlockThreads) void softmax_csr_long_kernel(int M,
                                                                         const int *__restrict__ row_ptr,
                                                                         const float *vals, float scale,
                                                                         float *out) {
  __shared__ float s_red[kWavesPerBlock];
  for (int row = blockIdx.x; row < M; row += gridDim.x) {
    const int lo = row_ptr[row], hi = row_ptr[row + 1];
    if (hi - lo <= kSoftmaxLongRow) continue;  // uniform across the workgroup
    float mx = -3.402823466e38f;
    for (int p = lo + threadIdx.x; p < hi; p += kBlockThreads) mx = fmaxf(mx, vals[p] * scale);
    mx = block_reduce(mx, s_red, true);
    float sum = 0.0f;
    for (int p = lo + threadIdx.x; p < hi; p += kBlockThreads) sum += expf(vals[p] * scale - mx);
    sum = block_reduce(sum, s_red, false);
    for (int p = lo + threadIdx.x; p < hi; p += kBlockThreads) out[p] = expf(vals[p] * scale - mx) / sum;
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
  const int g = scorch::group_width(M, nnz);
  const int64_t threads = M * g;
  const dim3 grid((unsigned)((threads + scorch::kBlockThreads - 1) / scorch::kBlockThreads));
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
  const unsigned pool = (unsigned)(M < scorch::kSoftmaxLongWorkgroups ? M : scorch::kSoftmaxLongWorkgroups);
  scorch::softmax_csr_long_kernel<<<pool, scorch::kBlockThreads, 0, s>>>(m, row_ptr, vals, scale, out);
  SCORCH_HIP_CHECK(hipGetLastError());
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

}  // extern "C"
