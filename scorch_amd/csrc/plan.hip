// The plan handle of scorch_hip.h: what is found out once about a CSR pattern (that it is well
// formed, its longest row, its empty rows; per dense width the merge-path chunk boundaries; the
// SDDMM's per-XCD entry lists) and the device memory those products need, kept behind one
// pointer.  Host code only: every kernel is reached through the library's own step-by-step
// entry points (scorch_hip_unstable.h), so a planned product runs exactly the kernels, and gives
// exactly the bits, of the steps called one by one.
//
// The reference has no such object: its dispatch looks at nothing but the dtype
// (src/scorch/prebuilt_kernels.py:198-224).
#include <new>

#include "common.hpp"

namespace scorch {
hipError_t preload_attn();
hipError_t preload_attn_f32();
hipError_t preload_blockdesc();
hipError_t preload_blocked();
hipError_t preload_misc();
hipError_t preload_sddmm();
hipError_t preload_spgemm();
hipError_t preload_spmm();
hipError_t preload_spmm_rows();
hipError_t preload_spmm_tiled();
}  // namespace scorch

namespace {

constexpr int kPlanWidths = 8;              // chunk boundaries kept for this many values of N
constexpr int64_t kRowsKernelMaxRow = 256;  // longest row the row-split kernel is chosen for
constexpr int64_t kSoftmaxShortRow = 4096;  // rows up to this length: the one-launch softmax
constexpr int64_t kFillFirstBytes = (int64_t)32 << 20;
constexpr int64_t kListsMinDense = (int64_t)8 << 20, kListsMaxDense = (int64_t)20 << 20;

struct Boundaries {
  int64_t N = -1;
  void *data = nullptr;
  size_t bytes = 0;
  uint64_t last_use = 0;
};

}  // namespace

struct scorch_hip_csr_plan {
  int device = 0;
  int64_t M = 0, n_cols = 0, nnz = 0;
  const int32_t *row_ptr = nullptr, *col_idx = nullptr;
  int32_t report[SCORCH_HIP_INSPECT_REPORT_INTS] = {};
  Boundaries widths[kPlanWidths];
  uint64_t uses = 0;
  void *workspace = nullptr;  // carries of the merge-path kernels, rows of the softmax: one product at a time
  size_t workspace_bytes = 0;
  void *lists = nullptr;      // the SDDMM's entry lists
  size_t lists_bytes = 0;
  bool lists_built = false;

  int64_t longest_row() const { return report[2]; }
  int64_t empty_rows() const { return report[3]; }
  size_t held() const {
    size_t total = workspace_bytes + lists_bytes;
    for (const Boundaries &b : widths) total += b.bytes;
    return total;
  }
};

struct scorch_hip_dense_plan {
  int device = 0;
  int64_t K = 0, N = 0;
  const float *B = nullptr;
  float *tiles = nullptr;  // B stored by column tiles, or null where that layout does not pay
  size_t tiles_bytes = 0;
};

namespace {

using scorch::fail;

int check_plan(const char *fn, const scorch_hip_csr_plan *plan) {
  if (!plan) return fail(SCORCH_HIP_EINVAL, "%s: plan is NULL", fn);
  int device = -1;
  SCORCH_HIP_CHECK(hipGetDevice(&device));
  if (device != plan->device)
    return fail(SCORCH_HIP_EINVAL, "%s: the plan was made on device %d, the current device is %d", fn,
                plan->device, device);
  return SCORCH_HIP_OK;
}

// The workspace grows and is never shrunk; work enqueued earlier may still use the old one, so
// the stream is waited for before it is freed.
int reserve_workspace(scorch_hip_csr_plan *plan, size_t bytes, hipStream_t stream) {
  if (bytes <= plan->workspace_bytes) return SCORCH_HIP_OK;
  if (plan->workspace) {
    SCORCH_HIP_CHECK(hipStreamSynchronize(stream));
    SCORCH_HIP_CHECK(hipFree(plan->workspace));
    plan->workspace = nullptr;
    plan->workspace_bytes = 0;
  }
  SCORCH_HIP_CHECK(hipMalloc(&plan->workspace, bytes));
  plan->workspace_bytes = bytes;
  return SCORCH_HIP_OK;
}

bool spmm_fills_first(const scorch_hip_csr_plan *plan, int64_t N, bool has_bias) {
  return !has_bias && 2 * plan->empty_rows() >= plan->M && plan->M * N * 4 >= kFillFirstBytes;
}
bool spmm_by_rows(const scorch_hip_csr_plan *plan, int64_t N, bool has_bias) {
  return plan->M == 0 || N == 0 ||
         (!spmm_fills_first(plan, N, has_bias) && plan->longest_row() <= kRowsKernelMaxRow);
}

// Boundaries and workspace of the merge-path kernels for dense width N (nothing for a product
// the row-split kernel serves with and without a bias).
int prepare_spmm(scorch_hip_csr_plan *plan, int64_t N, hipStream_t stream, Boundaries **found,
                 bool whatever_the_rows = false) {
  if (found) *found = nullptr;
  if (N < 0) return fail(SCORCH_HIP_EINVAL, "scorch_hip_csr_plan: negative N");
  if (!whatever_the_rows && spmm_by_rows(plan, N, false) && spmm_by_rows(plan, N, true)) return SCORCH_HIP_OK;
  if (int rc = reserve_workspace(plan, scorch_hip_spmm_csr_workspace_bytes(plan->M, plan->nnz, N, 4), stream))
    return rc;
  Boundaries *slot = nullptr;
  for (Boundaries &b : plan->widths)
    if (b.N == N) slot = &b;
  if (!slot) {
    slot = &plan->widths[0];
    for (Boundaries &b : plan->widths)
      if (b.last_use < slot->last_use) slot = &b;
    if (slot->data) {  // the oldest width makes room
      SCORCH_HIP_CHECK(hipStreamSynchronize(stream));
      SCORCH_HIP_CHECK(hipFree(slot->data));
      *slot = Boundaries();
    }
    const size_t bytes = scorch_hip_spmm_csr_bounds_bytes(plan->M, plan->nnz, N, 4);
    if (bytes > 0) {
      SCORCH_HIP_CHECK(hipMalloc(&slot->data, bytes));
      slot->bytes = bytes;
      if (int rc = scorch_hip_spmm_csr_bounds(plan->M, plan->nnz, N, 4, plan->row_ptr, slot->data, bytes, stream)) {
        (void)hipFree(slot->data);
        *slot = Boundaries();
        return rc;
      }
    }
    slot->N = N;
  }
  slot->last_use = ++plan->uses;
  if (found) *found = slot;
  return SCORCH_HIP_OK;
}

bool sddmm_by_lists(const scorch_hip_csr_plan *plan, int64_t K) {
  const int64_t dense = plan->n_cols * K * 4;
  return K > 0 && K <= 256 && plan->nnz > 0 && dense >= kListsMinDense && dense <= kListsMaxDense &&
         plan->nnz >= 4 * plan->n_cols;
}

int prepare_sddmm(scorch_hip_csr_plan *plan, int64_t K, hipStream_t stream) {
  if (K < 0) return fail(SCORCH_HIP_EINVAL, "scorch_hip_csr_plan: negative K");
  if (!sddmm_by_lists(plan, K) || plan->lists_built) return SCORCH_HIP_OK;
  const size_t bytes = scorch_hip_sddmm_csr_lists_bytes(plan->nnz);
  SCORCH_HIP_CHECK(hipMalloc(&plan->lists, bytes));
  plan->lists_bytes = bytes;
  if (int rc = scorch_hip_sddmm_csr_lists(plan->M, plan->n_cols, plan->nnz, plan->row_ptr, plan->col_idx,
                                          plan->lists, bytes, stream)) {
    (void)hipFree(plan->lists);
    plan->lists = nullptr;
    plan->lists_bytes = 0;
    return rc;
  }
  plan->lists_built = true;
  return SCORCH_HIP_OK;
}

int prepare_softmax(scorch_hip_csr_plan *plan, hipStream_t stream) {
  if (plan->longest_row() <= kSoftmaxShortRow) return SCORCH_HIP_OK;
  return reserve_workspace(plan, scorch_hip_softmax_csr_workspace_bytes(plan->M, plan->nnz), stream);
}

}  // namespace

extern "C" {

int scorch_hip_init(void) {
  hipError_t (*const loaders[])() = {scorch::preload_attn,      scorch::preload_attn_f32, scorch::preload_blockdesc,
                                     scorch::preload_blocked,   scorch::preload_misc,     scorch::preload_sddmm,
                                     scorch::preload_spgemm,    scorch::preload_spmm,     scorch::preload_spmm_rows,
                                     scorch::preload_spmm_tiled};
  for (auto load : loaders) SCORCH_HIP_CHECK(load());
  return SCORCH_HIP_OK;
}

int scorch_hip_csr_plan_create(int64_t M, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                               const int32_t *col_idx, void *stream, scorch_hip_csr_plan **out) {
  if (!out) return fail(SCORCH_HIP_EINVAL, "scorch_hip_csr_plan_create: plan is NULL");
  *out = nullptr;
  // (the value array is not a plan's business: any non-null pointer satisfies the shared check)
  if (int rc = scorch::check_csr_args("scorch_hip_csr_plan_create", M, n_cols, nnz, row_ptr, col_idx, row_ptr))
    return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  int device = -1;
  SCORCH_HIP_CHECK(hipGetDevice(&device));
  int32_t *report = nullptr;
  SCORCH_HIP_CHECK(hipMalloc(reinterpret_cast<void **>(&report), sizeof(int32_t) * SCORCH_HIP_INSPECT_REPORT_INTS));
  scorch_hip_csr_plan *plan = new (std::nothrow) scorch_hip_csr_plan();
  int rc = plan ? SCORCH_HIP_OK : fail(SCORCH_HIP_ERUNTIME, "scorch_hip_csr_plan_create: out of host memory");
  if (!rc) rc = scorch_hip_csr_inspect(M, n_cols, nnz, row_ptr, col_idx, report, stream);
  if (!rc) {
    hipError_t err = hipMemcpyAsync(plan->report, report, sizeof(plan->report), hipMemcpyDeviceToHost, s);
    if (err == hipSuccess) err = hipStreamSynchronize(s);
    if (err != hipSuccess)
      rc = fail(SCORCH_HIP_ERUNTIME, "scorch_hip_csr_plan_create: reading the inspection back failed: %s",
                hipGetErrorString(err));
  }
  (void)hipFree(report);
  if (!rc && (plan->report[0] || plan->report[1]))
    rc = fail(SCORCH_HIP_EINVAL, "scorch_hip_csr_plan_create: malformed CSR index:%s%s",
              plan->report[0] ? " row_ptr must start at 0, never decrease and end at nnz;" : "",
              plan->report[1] ? " a column index lies outside [0, n_cols)" : "");
  if (rc) {
    delete plan;
    return rc;
  }
  plan->device = device;
  plan->M = M;
  plan->n_cols = n_cols;
  plan->nnz = nnz;
  plan->row_ptr = row_ptr;
  plan->col_idx = col_idx;
  *out = plan;
  return SCORCH_HIP_OK;
}

int scorch_hip_csr_plan_destroy(scorch_hip_csr_plan *plan) {
  if (!plan) return SCORCH_HIP_OK;
  // work that still reads the plan's memory may be in flight on any stream of its device
  int current = -1;
  hipError_t err = hipGetDevice(&current);
  if (err == hipSuccess && current != plan->device) err = hipSetDevice(plan->device);
  if (err == hipSuccess) err = hipDeviceSynchronize();
  for (Boundaries &b : plan->widths)
    if (b.data) (void)hipFree(b.data);
  if (plan->workspace) (void)hipFree(plan->workspace);
  if (plan->lists) (void)hipFree(plan->lists);
  if (current >= 0 && current != plan->device) (void)hipSetDevice(current);
  delete plan;
  if (err != hipSuccess)
    return fail(SCORCH_HIP_ERUNTIME, "scorch_hip_csr_plan_destroy: %s", hipGetErrorString(err));
  return SCORCH_HIP_OK;
}

int scorch_hip_csr_plan_info(const scorch_hip_csr_plan *plan, int64_t *info) {
  if (!plan || !info) return fail(SCORCH_HIP_EINVAL, "scorch_hip_csr_plan_info: NULL argument");
  info[0] = plan->M;
  info[1] = plan->n_cols;
  info[2] = plan->nnz;
  info[3] = plan->longest_row();
  info[4] = plan->empty_rows();
  info[5] = plan->report[4] == 0;
  info[6] = (int64_t)plan->held();
  info[7] = 0;
  return SCORCH_HIP_OK;
}

int scorch_hip_csr_plan_prepare(scorch_hip_csr_plan *plan, int op, int64_t width, void *stream) {
  if (int rc = check_plan("scorch_hip_csr_plan_prepare", plan)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (op) {
    case SCORCH_HIP_PLAN_SPMM_F32: return prepare_spmm(plan, width, s, nullptr);
    case SCORCH_HIP_PLAN_SDDMM_F32: return prepare_sddmm(plan, width, s);
    case SCORCH_HIP_PLAN_SOFTMAX_F32: return prepare_softmax(plan, s);
    case SCORCH_HIP_PLAN_SPMM_DENSE_F32: return prepare_spmm(plan, width, s, nullptr, true);
    default: return fail(SCORCH_HIP_EINVAL, "scorch_hip_csr_plan_prepare: op %d is not a scorch_hip_plan_op", op);
  }
}

int scorch_hip_spmm_csr_plan_f32(scorch_hip_csr_plan *plan, int64_t N, const float *vals, const float *B,
                                 const float *bias, int act, float *C, void *stream) {
  if (int rc = check_plan("scorch_hip_spmm_csr_plan_f32", plan)) return rc;
  if (act != SCORCH_HIP_ACT_NONE && act != SCORCH_HIP_ACT_RELU)
    return fail(SCORCH_HIP_EINVAL, "scorch_hip_spmm_csr_plan_f32: act %d is not a scorch_hip_act", act);
  if (N < 0) return fail(SCORCH_HIP_EINVAL, "scorch_hip_spmm_csr_plan_f32: negative N");
  if (spmm_by_rows(plan, N, bias != nullptr))
    return scorch_hip_spmm_csr_rows_f32(plan->M, plan->n_cols, N, plan->nnz, plan->row_ptr, plan->col_idx, vals, B,
                                        bias, act, C, stream);
  Boundaries *bounds = nullptr;
  if (int rc = prepare_spmm(plan, N, static_cast<hipStream_t>(stream), &bounds)) return rc;
  const int hint = spmm_fills_first(plan, N, bias != nullptr) ? SCORCH_HIP_HINT_MOSTLY_EMPTY_ROWS : 0;
  return scorch_hip_spmm_csr_planned_f32(plan->M, plan->n_cols, N, plan->nnz, plan->row_ptr, plan->col_idx, vals, B,
                                         bias, act | hint, C, bounds ? bounds->data : nullptr,
                                         bounds ? bounds->bytes : 0, plan->workspace, plan->workspace_bytes, stream);
}

int scorch_hip_sddmm_csr_plan_f32(scorch_hip_csr_plan *plan, int64_t K, const float *mask_vals, const float *A,
                                  const float *B, float *out_vals, int32_t *out_row_idx, void *stream) {
  if (int rc = check_plan("scorch_hip_sddmm_csr_plan_f32", plan)) return rc;
  if (int rc = prepare_sddmm(plan, K, static_cast<hipStream_t>(stream))) return rc;
  if (sddmm_by_lists(plan, K))
    return scorch_hip_sddmm_csr_listed_f32(1, plan->M, plan->n_cols, K, plan->nnz, plan->lists, plan->lists_bytes,
                                           mask_vals, nullptr, A, B, out_vals, out_row_idx, stream);
  return scorch_hip_sddmm_csr_f32(plan->M, plan->n_cols, K, plan->nnz, plan->row_ptr, plan->col_idx, mask_vals, A, B,
                                  out_vals, out_row_idx, stream);
}

int scorch_hip_softmax_csr_plan_f32(scorch_hip_csr_plan *plan, const float *vals, float scale, float *out,
                                    void *stream) {
  if (int rc = check_plan("scorch_hip_softmax_csr_plan_f32", plan)) return rc;
  if (plan->longest_row() <= kSoftmaxShortRow)
    return scorch_hip_softmax_csr_known_rows_f32(1, plan->M, plan->nnz, plan->longest_row(), plan->row_ptr, vals,
                                                 scale, out, nullptr, 0, stream);
  if (int rc = prepare_softmax(plan, static_cast<hipStream_t>(stream))) return rc;
  return scorch_hip_softmax_csr_known_rows_f32(1, plan->M, plan->nnz, plan->longest_row(), plan->row_ptr, vals,
                                               scale, out, plan->workspace, plan->workspace_bytes, stream);
}

int scorch_hip_dense_plan_create(int64_t K, int64_t N, const float *B, void *stream, scorch_hip_dense_plan **out) {
  const char *fn = "scorch_hip_dense_plan_create";
  if (!out) return fail(SCORCH_HIP_EINVAL, "%s: plan is NULL", fn);
  *out = nullptr;
  if (K < 0 || N < 0) return fail(SCORCH_HIP_EINVAL, "%s: negative size (K=%lld N=%lld)", fn, (long long)K, (long long)N);
  if (K > INT32_MAX || N > INT32_MAX) return fail(SCORCH_HIP_EUNSUPPORTED, "%s: K and N must fit int32", fn);
  if (K > 0 && N > 0 && !B) return fail(SCORCH_HIP_EINVAL, "%s: B is NULL", fn);
  if (!scorch::aligned_to(B, 4)) return fail(SCORCH_HIP_EINVAL, "%s: B must be 4-byte aligned", fn);
  int device = -1;
  SCORCH_HIP_CHECK(hipGetDevice(&device));
  scorch_hip_dense_plan *plan = new (std::nothrow) scorch_hip_dense_plan();
  if (!plan) return fail(SCORCH_HIP_ERUNTIME, "%s: out of host memory", fn);
  plan->device = device;
  plan->K = K;
  plan->N = N;
  plan->B = B;
  // (whether a product gathers the rows of B more than once is known only with its sparse operand:
  // the layout is prepared for every shape it can pay for, and each product decides)
  if (scorch_hip_dense_tiled_recommended(K, N, INT32_MAX, 4)) {
    plan->tiles_bytes = scorch_hip_dense_tiled_bytes(K, N, 4);
    hipError_t err = hipMalloc(reinterpret_cast<void **>(&plan->tiles), plan->tiles_bytes);
    int rc = err == hipSuccess ? scorch_hip_dense_to_tiled_f32(K, N, B, plan->tiles, plan->tiles_bytes, stream)
                               : fail(SCORCH_HIP_ERUNTIME, "%s: hipMalloc of %zu bytes failed: %s", fn,
                                      plan->tiles_bytes, hipGetErrorString(err));
    if (rc) {
      if (plan->tiles) (void)hipFree(plan->tiles);
      delete plan;
      return rc;
    }
  }
  *out = plan;
  return SCORCH_HIP_OK;
}

int scorch_hip_dense_plan_update(scorch_hip_dense_plan *plan, void *stream) {
  if (!plan) return fail(SCORCH_HIP_EINVAL, "scorch_hip_dense_plan_update: plan is NULL");
  int device = -1;
  SCORCH_HIP_CHECK(hipGetDevice(&device));
  if (device != plan->device)
    return fail(SCORCH_HIP_EINVAL, "scorch_hip_dense_plan_update: the plan was made on device %d, the current device is %d",
                plan->device, device);
  if (!plan->tiles) return SCORCH_HIP_OK;
  return scorch_hip_dense_to_tiled_f32(plan->K, plan->N, plan->B, plan->tiles, plan->tiles_bytes, stream);
}

int scorch_hip_dense_plan_destroy(scorch_hip_dense_plan *plan) {
  if (!plan) return SCORCH_HIP_OK;
  hipError_t err = hipSuccess;
  if (plan->tiles) {
    int current = -1;
    err = hipGetDevice(&current);
    if (err == hipSuccess && current != plan->device) err = hipSetDevice(plan->device);
    if (err == hipSuccess) err = hipDeviceSynchronize();  // products that read the tiles may be in flight
    (void)hipFree(plan->tiles);
    if (current >= 0 && current != plan->device) (void)hipSetDevice(current);
  }
  delete plan;
  if (err != hipSuccess)
    return fail(SCORCH_HIP_ERUNTIME, "scorch_hip_dense_plan_destroy: %s", hipGetErrorString(err));
  return SCORCH_HIP_OK;
}

int scorch_hip_spmm_csr_plan_dense_f32(scorch_hip_csr_plan *plan, const float *vals, const scorch_hip_dense_plan *dense,
                                       const float *bias, int act, float *C, void *stream) {
  const char *fn = "scorch_hip_spmm_csr_plan_dense_f32";
  if (int rc = check_plan(fn, plan)) return rc;
  if (!dense) return fail(SCORCH_HIP_EINVAL, "%s: the dense plan is NULL", fn);
  if (dense->device != plan->device || dense->K != plan->n_cols)
    return fail(SCORCH_HIP_EINVAL, "%s: the dense plan is %lld x %lld on device %d, the sparse one %lld x %lld on %d",
                fn, (long long)dense->K, (long long)dense->N, dense->device, (long long)plan->M,
                (long long)plan->n_cols, plan->device);
  const int64_t N = dense->N;
  if (!dense->tiles || plan->M == 0 || !scorch_hip_dense_tiled_recommended(dense->K, N, plan->nnz, 4))
    return scorch_hip_spmm_csr_plan_f32(plan, N, vals, dense->B, bias, act, C, stream);
  Boundaries *bounds = nullptr;
  if (int rc = prepare_spmm(plan, N, static_cast<hipStream_t>(stream), &bounds, true)) return rc;
  return scorch_hip_spmm_csr_tiled_f32(plan->M, plan->n_cols, N, plan->nnz, plan->row_ptr, plan->col_idx, vals,
                                       dense->tiles, dense->tiles_bytes, bias, act, C, bounds ? bounds->data : nullptr,
                                       bounds ? bounds->bytes : 0, plan->workspace, plan->workspace_bytes,
                                       plan->longest_row(), stream);
}

}  // extern "C"
