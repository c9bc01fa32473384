/* A C host of libscorch_hip.so: what a binding of the reference's native module would do, with
 * nothing but the C ABI (include/scorch_hip.h) and the HIP runtime.  Builds a small power-law-ish
 * CSR matrix, multiplies it through the stateless call and through a plan handle, runs an SDDMM
 * and a row softmax through the same plan, and checks everything against plain loops on the host.
 * Prints "ok" and returns 0, or says what differed. */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "scorch_hip.h"

#define CHECK_HIP(call)                                                                  \
  do {                                                                                   \
    hipError_t e_ = (call);                                                              \
    if (e_ != hipSuccess) {                                                              \
      fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));                         \
      return 2;                                                                          \
    }                                                                                    \
  } while (0)
#define CHECK_SCORCH(call)                                                               \
  do {                                                                                   \
    int rc_ = (call);                                                                    \
    if (rc_ != SCORCH_HIP_OK) {                                                          \
      fprintf(stderr, "%s: status %d: %s\n", #call, rc_, scorch_hip_last_error());       \
      return 3;                                                                          \
    }                                                                                    \
  } while (0)

static unsigned int state = 12345u;
static unsigned int next_u32(void) {
  state = state * 1664525u + 1013904223u;
  return state >> 8;
}
static float next_unit(void) { return (float)(next_u32() % 20001) / 10000.0f - 1.0f; }

static void *to_device(const void *host, size_t bytes) {
  void *dev = NULL;
  if (bytes == 0) bytes = 4;
  if (hipMalloc(&dev, bytes) != hipSuccess) return NULL;
  if (host && hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice) != hipSuccess) return NULL;
  return dev;
}

static double worst(const float *got, const double *want, size_t n) {
  double num = 0.0, den = 0.0;
  for (size_t i = 0; i < n; ++i) {
    num += (got[i] - want[i]) * (got[i] - want[i]);
    den += want[i] * want[i];
  }
  return sqrt(num / (den > 0.0 ? den : 1.0));
}

int main(void) {
  enum { M = 3000, K = 2000, N = 96, D = 24 };
  /* rows of 0 to 40 entries, every 97th row 700 long: the plan takes the merge-path kernels */
  int32_t *row_ptr = (int32_t *)malloc(sizeof(int32_t) * (M + 1));
  row_ptr[0] = 0;
  for (int i = 0; i < M; ++i) row_ptr[i + 1] = row_ptr[i] + (i % 97 == 5 ? 700 : (int)(next_u32() % 41));
  const int nnz = row_ptr[M];
  int32_t *col_idx = (int32_t *)malloc(sizeof(int32_t) * nnz);
  float *vals = (float *)malloc(sizeof(float) * nnz);
  for (int i = 0; i < M; ++i) {
    /* increasing columns within a row */
    const int len = row_ptr[i + 1] - row_ptr[i];
    int c = 0;
    for (int p = 0; p < len; ++p) {
      const int room = K - c - (len - p);
      c += 1 + (room > 0 ? (int)(next_u32() % (unsigned)(room / (len - p) + 1)) : 0);
      col_idx[row_ptr[i] + p] = c - 1;
    }
  }
  for (int p = 0; p < nnz; ++p) vals[p] = next_unit();
  float *B = (float *)malloc(sizeof(float) * K * N), *Q = (float *)malloc(sizeof(float) * M * D),
        *Kd = (float *)malloc(sizeof(float) * K * D);
  for (int i = 0; i < K * N; ++i) B[i] = next_unit();
  for (int i = 0; i < M * D; ++i) Q[i] = next_unit();
  for (int i = 0; i < K * D; ++i) Kd[i] = next_unit();

  CHECK_SCORCH(scorch_hip_init());
  if (scorch_hip_abi_version() != SCORCH_HIP_ABI_VERSION) {
    fprintf(stderr, "header and library disagree on the ABI version\n");
    return 4;
  }
  int32_t *d_rp = (int32_t *)to_device(row_ptr, sizeof(int32_t) * (M + 1));
  int32_t *d_ci = (int32_t *)to_device(col_idx, sizeof(int32_t) * nnz);
  float *d_v = (float *)to_device(vals, sizeof(float) * nnz), *d_B = (float *)to_device(B, sizeof(float) * K * N);
  float *d_Q = (float *)to_device(Q, sizeof(float) * M * D), *d_K = (float *)to_device(Kd, sizeof(float) * K * D);
  float *d_C = (float *)to_device(NULL, sizeof(float) * M * N), *d_C2 = (float *)to_device(NULL, sizeof(float) * M * N);
  float *d_s = (float *)to_device(NULL, sizeof(float) * nnz), *d_p = (float *)to_device(NULL, sizeof(float) * nnz);
  int32_t *d_rows = (int32_t *)to_device(NULL, sizeof(int32_t) * nnz);
  const size_t ws_bytes = scorch_hip_spmm_csr_workspace_bytes(M, nnz, N, sizeof(float));
  void *d_ws = to_device(NULL, ws_bytes);
  if (!d_rp || !d_ci || !d_v || !d_B || !d_Q || !d_K || !d_C || !d_C2 || !d_s || !d_p || !d_rows || !d_ws) {
    fprintf(stderr, "device allocation failed\n");
    return 2;
  }

  /* the stateless call, and the same product through a plan */
  CHECK_SCORCH(scorch_hip_spmm_csr_f32(M, K, N, nnz, d_rp, d_ci, d_v, d_B, d_C, d_ws, ws_bytes, NULL));
  scorch_hip_csr_plan *plan = NULL;
  CHECK_SCORCH(scorch_hip_csr_plan_create(M, K, nnz, d_rp, d_ci, NULL, &plan));
  int64_t info[SCORCH_HIP_PLAN_INFO_INTS];
  CHECK_SCORCH(scorch_hip_csr_plan_info(plan, info));
  if (info[0] != M || info[1] != K || info[2] != nnz || info[3] != 700 || info[5] != 1) {
    fprintf(stderr, "plan info: M %lld K %lld nnz %lld longest %lld sorted %lld\n", (long long)info[0],
            (long long)info[1], (long long)info[2], (long long)info[3], (long long)info[5]);
    return 5;
  }
  CHECK_SCORCH(scorch_hip_csr_plan_prepare(plan, SCORCH_HIP_PLAN_SPMM_F32, N, NULL));
  CHECK_SCORCH(scorch_hip_spmm_csr_plan_f32(plan, N, d_v, d_B, NULL, SCORCH_HIP_ACT_NONE, d_C2, NULL));
  CHECK_SCORCH(scorch_hip_sddmm_csr_plan_f32(plan, D, d_v, d_Q, d_K, d_s, d_rows, NULL));
  CHECK_SCORCH(scorch_hip_softmax_csr_plan_f32(plan, d_s, 0.25f, d_p, NULL));
  CHECK_HIP(hipDeviceSynchronize());

  float *C = (float *)malloc(sizeof(float) * M * N), *C2 = (float *)malloc(sizeof(float) * M * N);
  float *s = (float *)malloc(sizeof(float) * nnz), *prob = (float *)malloc(sizeof(float) * nnz);
  int32_t *rows = (int32_t *)malloc(sizeof(int32_t) * nnz);
  CHECK_HIP(hipMemcpy(C, d_C, sizeof(float) * M * N, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(C2, d_C2, sizeof(float) * M * N, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(s, d_s, sizeof(float) * nnz, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(prob, d_p, sizeof(float) * nnz, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(rows, d_rows, sizeof(int32_t) * nnz, hipMemcpyDeviceToHost));

  /* the host's own loops, in double */
  double *want_C = (double *)calloc((size_t)M * N, sizeof(double)), *want_s = (double *)malloc(sizeof(double) * nnz),
         *want_p = (double *)malloc(sizeof(double) * nnz);
  int bad_rows = 0;
  for (int i = 0; i < M; ++i) {
    double top = -1e300, sum = 0.0;
    for (int p = row_ptr[i]; p < row_ptr[i + 1]; ++p) {
      const int j = col_idx[p];
      for (int n = 0; n < N; ++n) want_C[(size_t)i * N + n] += (double)vals[p] * B[(size_t)j * N + n];
      double dot = 0.0;
      for (int k = 0; k < D; ++k) dot += (double)Q[i * D + k] * Kd[j * D + k];
      want_s[p] = vals[p] * dot;
      if (0.25 * (double)s[p] > top) top = 0.25 * (double)s[p];
      bad_rows += rows[p] != i;
    }
    for (int p = row_ptr[i]; p < row_ptr[i + 1]; ++p) sum += exp(0.25 * (double)s[p] - top);
    for (int p = row_ptr[i]; p < row_ptr[i + 1]; ++p) want_p[p] = exp(0.25 * (double)s[p] - top) / sum;
  }
  const double e_c = worst(C, want_C, (size_t)M * N), e_c2 = worst(C2, want_C, (size_t)M * N);
  const double e_s = worst(s, want_s, nnz), e_p = worst(prob, want_p, nnz);
  const int same = memcmp(C, C2, sizeof(float) * M * N) == 0;
  printf("spmm %.2e  planned spmm %.2e (bit-identical: %d)  sddmm %.2e  softmax %.2e  wrong rows %d\n", e_c, e_c2,
         same, e_s, e_p, bad_rows);
  if (e_c > 1e-5 || e_c2 > 1e-5 || e_s > 1e-5 || e_p > 1e-5 || !same || bad_rows) return 1;

  /* a malformed index gets no plan, and nothing reads through it */
  col_idx[7] = K;
  CHECK_HIP(hipMemcpy(d_ci, col_idx, sizeof(int32_t) * nnz, hipMemcpyHostToDevice));
  scorch_hip_csr_plan *refused = NULL;
  if (scorch_hip_csr_plan_create(M, K, nnz, d_rp, d_ci, NULL, &refused) != SCORCH_HIP_EINVAL || refused != NULL) {
    fprintf(stderr, "a column index of K was accepted\n");
    return 6;
  }
  CHECK_SCORCH(scorch_hip_csr_plan_destroy(plan));
  puts("ok");
  return 0;
}
