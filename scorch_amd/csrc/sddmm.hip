// SDDMM for gfx950: out[p] = mask[p] * <A[row_p, :], B[col_p, :]>.
//
// A wavefront owns kEntriesPerWave consecutive mask entries and handles them
// 64 at a time.  For each batch of 64, lane L first fetches the coordinates and
// mask value of entry L (coalesced).  The wavefront is then split into 64/GS
// groups of GS lanes; in step s, group g computes the dot product of entry
// g * GS + s: its GS lanes read the two K-vectors with one vector load each
// (GS * VEC elements per load, so a K = 64 fp32 row is one dwordx4 access by
// 16 lanes), multiply, and reduce with GS-wide butterfly shuffles.  After GS
// steps lane L keeps the result of entry L and the batch is written with one
// coalesced store.  Consecutive entries share their A row, which therefore
// comes from the vector cache after its first use.
//
// With a CSR mask the row of each entry is found by bisection of row_ptr; the
// wavefront first narrows the range to the rows its entries span, so the
// per-lane search is a few steps.  The same pass can write the row of every
// entry (the coordinate array of the result).
#include "common.hpp"

namespace scorch {

constexpr int kEntriesPerWave = 256;

// LONG: K exceeds what the group's lanes cover with one load each (GS * VEC
// elements); the vectors are then read four such pieces at a time, all eight
// loads requested before the first product.
template <int GS, int VEC, bool COO, bool LONG>
__global__ __launch_bounds__(kBlockThreads) void sddmm_kernel(
    int M, int K, int64_t nnz, const int *__restrict__ rows /* row_idx (COO) or row_ptr (CSR) */,
    const int *__restrict__ col_idx, const float *__restrict__ mask_vals,
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ out_vals,
    int *__restrict__ out_row_idx, int64_t batch_stride_a, int64_t batch_stride_b) {
  using VecT = Vec<float, VEC>;
  const int lane = wave_lane();
  // grid.y > 1: several products over one mask (one per attention head); problem h has its own A,
  // B and result values, the mask's values are shared and the row coordinates are written once
  if (blockIdx.y > 0) {
    A += blockIdx.y * batch_stride_a;
    B += blockIdx.y * batch_stride_b;
    out_vals += blockIdx.y * nnz;
    out_row_idx = nullptr;
  }
  // the grid is a multiple of 8 workgroups; every XCD takes a contiguous eighth of the entries
  const int64_t wave = xcd_contiguous(blockIdx.x, gridDim.x) * kWavesPerBlock + threadIdx.x / kWaveSize;
  const int64_t first = wave * kEntriesPerWave;
  if (first >= nnz) return;
  const int64_t last = first + kEntriesPerWave < nnz ? first + kEntriesPerWave : nnz;

  // Rows spanned by this wavefront's entries: row(p) = #{i : row_ptr[i+1] <= p}.
  int row_lo = 0, row_hi = 0;
  if (!COO) {
    auto end_key = [&](int i) { return (int64_t)rows[i + 1]; };
    row_lo = wave_count_below(M, first + 1, end_key);
    row_hi = wave_count_below(M, last, end_key);  // row of entry last - 1
  }

  const int t = lane % GS;  // position inside the group
  const int g = lane / GS;  // group

  for (int64_t base = first; base < last; base += kWaveSize) {
    const int64_t p = base + lane;
    const bool valid = p < last;
    int row = 0, col = 0;
    float scale = 0.0f;
    if (valid) {
      col = col_idx[p];
      scale = mask_vals[p];
      if (COO) {
        row = rows[p];
      } else {
        int lo = row_lo, hi = row_hi;  // answer in [lo, hi]
        while (lo < hi) {
          const int mid = (lo + hi) >> 1;
          if ((int64_t)rows[mid + 1] <= p) lo = mid + 1; else hi = mid;
        }
        row = lo;
      }
    }

    float mine = 0.0f;
#pragma unroll 4
    for (int s = 0; s < GS; ++s) {
      const int src = g * GS + s;
      const int r = __shfl(row, src);
      const int c = __shfl(col, src);
      const float *a = A + (size_t)r * (size_t)K;
      const float *b = B + (size_t)c * (size_t)K;
      float dot = 0.0f;
      if (!LONG) {
        for (int k = t * VEC; k < K; k += GS * VEC) {
          const VecT av = *reinterpret_cast<const VecT *>(a + k);
          const VecT bv = *reinterpret_cast<const VecT *>(b + k);
#pragma unroll
          for (int v = 0; v < VEC; ++v) dot += av.v[v] * bv.v[v];
        }
      } else {
        constexpr int kPieces = 4;
        for (int k0 = t * VEC; k0 < K; k0 += kPieces * GS * VEC) {
          VecT av[kPieces], bv[kPieces];
#pragma unroll
          for (int u = 0; u < kPieces; ++u) {
            const int k = k0 + u * GS * VEC;
            if (k < K) {
              av[u] = *reinterpret_cast<const VecT *>(a + k);
              bv[u] = *reinterpret_cast<const VecT *>(b + k);
            } else {
#pragma unroll
              for (int v = 0; v < VEC; ++v) av[u].v[v] = bv[u].v[v] = 0.0f;
            }
          }
#pragma unroll
          for (int u = 0; u < kPieces; ++u)
#pragma unroll
            for (int v = 0; v < VEC; ++v) dot += av[u].v[v] * bv[u].v[v];
        }
      }
#pragma unroll
      for (int off = GS / 2; off > 0; off >>= 1) dot += __shfl_xor(dot, off);
      if (t == s) mine = dot;
    }

    if (valid) {
      out_vals[p] = scale * mine;
      if (!COO && out_row_idx) out_row_idx[p] = row;
    }
  }
}

template <bool COO>
int launch_sddmm(int M, int K, int64_t nnz, const int *rows, const int *col_idx,
                 const float *mask_vals, const float *A, const float *B, float *out_vals,
                 int *out_row_idx, hipStream_t stream, int batch = 1, int64_t batch_stride_a = 0,
                 int64_t batch_stride_b = 0) {
  const int64_t waves = (nnz + kEntriesPerWave - 1) / kEntriesPerWave;
  const dim3 grid((unsigned)round_up_8((waves + kWavesPerBlock - 1) / kWavesPerBlock), (unsigned)batch);
  const bool vec4 = K % 4 == 0 && aligned_to(A, 16) && aligned_to(B, 16);
  const int per_lane = vec4 ? 4 : 1;
  const int64_t lanes_needed = (K + per_lane - 1) / per_lane;

  mark_launch(stream);
#define SCORCH_SDDMM_LAUNCH(GS, VEC, LONG)                                                         \
  sddmm_kernel<GS, VEC, COO, LONG><<<grid, kBlockThreads, 0, stream>>>(M, K, nnz, rows, col_idx,   \
                                                                      mask_vals, A, B, out_vals,  \
                                                                      out_row_idx, batch_stride_a,  \
                                                                      batch_stride_b)
#define SCORCH_SDDMM_PICK(VEC)                                              \
  do {                                                                      \
    if (lanes_needed <= 4) SCORCH_SDDMM_LAUNCH(4, VEC, false);              \
    else if (lanes_needed <= 8) SCORCH_SDDMM_LAUNCH(8, VEC, false);         \
    else if (lanes_needed <= 16) SCORCH_SDDMM_LAUNCH(16, VEC, false);       \
    else if (lanes_needed <= 32) SCORCH_SDDMM_LAUNCH(32, VEC, false);       \
    else if (lanes_needed <= 64) SCORCH_SDDMM_LAUNCH(64, VEC, false);       \
    else SCORCH_SDDMM_LAUNCH(64, VEC, true);                                \
  } while (0)

  if (vec4) SCORCH_SDDMM_PICK(4); else SCORCH_SDDMM_PICK(1);
#undef SCORCH_SDDMM_PICK
#undef SCORCH_SDDMM_LAUNCH
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(stream);
  return SCORCH_HIP_OK;
}

template <bool COO>
int sddmm_entry(const char *fn, int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                const int32_t *rows, const int32_t *col_idx, const float *mask_vals,
                const float *A, const float *B, float *out_vals, int32_t *out_row_idx,
                void *stream, int64_t batch = 1) {
  if (batch < 0 || batch > 65535)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: batch=%lld is outside [0, 65535]", fn, (long long)batch);
  if (batch == 0) return SCORCH_HIP_OK;
  if (M < 0 || n_cols < 0 || K < 0 || nnz < 0)
    return fail(SCORCH_HIP_EINVAL, "%s: negative size (M=%lld n_cols=%lld K=%lld nnz=%lld)", fn,
                (long long)M, (long long)n_cols, (long long)K, (long long)nnz);
  if (M >= INT32_MAX || n_cols > INT32_MAX || K > INT32_MAX || nnz > INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: sizes must fit int32 indices", fn);
  SCORCH_REQUIRE(COO || rows != nullptr, "%s: row_ptr is NULL", fn);
  if (nnz == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(M > 0 && n_cols > 0, "%s: nnz=%lld in an empty mask", fn, (long long)nnz);
  SCORCH_REQUIRE(rows && col_idx && mask_vals && out_vals, "%s: NULL index/value array", fn);
  SCORCH_REQUIRE(K == 0 || (A && B), "%s: NULL dense operand", fn);
  SCORCH_REQUIRE(aligned_to(rows, 4) && aligned_to(col_idx, 4) && aligned_to(mask_vals, 4) &&
                     aligned_to(out_vals, 4) && aligned_to(A, 4) && aligned_to(B, 4) &&
                     aligned_to(out_row_idx, 4),
                 "%s: arrays must be 4-byte aligned", fn);
  return launch_sddmm<COO>((int)M, (int)K, nnz, rows, col_idx, mask_vals, A, B, out_vals,
                           out_row_idx, static_cast<hipStream_t>(stream), (int)batch, M * K, n_cols * K);
}

}  // namespace scorch

extern "C" {

int scorch_hip_sddmm_coo_f32(int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                             const int32_t *row_idx, const int32_t *col_idx,
                             const float *mask_vals, const float *A, const float *B,
                             float *out_vals, void *stream) {
  return scorch::sddmm_entry<true>("scorch_hip_sddmm_coo_f32", M, n_cols, K, nnz, row_idx, col_idx,
                                   mask_vals, A, B, out_vals, nullptr, stream);
}

int scorch_hip_sddmm_csr_f32(int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                             const int32_t *row_ptr, const int32_t *col_idx,
                             const float *mask_vals, const float *A, const float *B,
                             float *out_vals, int32_t *out_row_idx, void *stream) {
  return scorch::sddmm_entry<false>("scorch_hip_sddmm_csr_f32", M, n_cols, K, nnz, row_ptr,
                                    col_idx, mask_vals, A, B, out_vals, out_row_idx, stream);
}

int scorch_hip_sddmm_csr_batched_f32(int64_t batch, int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                                     const int32_t *row_ptr, const int32_t *col_idx, const float *mask_vals,
                                     const float *A, const float *B, float *out_vals, int32_t *out_row_idx,
                                     void *stream) {
  return scorch::sddmm_entry<false>("scorch_hip_sddmm_csr_batched_f32", M, n_cols, K, nnz, row_ptr, col_idx,
                                    mask_vals, A, B, out_vals, out_row_idx, stream, batch);
}

}  // extern "C"
