/*
 * scorch_hip.h -- C ABI of libscorch_hip.so: Scorch's prebuilt CSR
 * sparse x dense kernels (SpMM, SDDMM and their neighbours) for AMD MI355X
 * (gfx950).  This header is the stable surface: one call per operation, and
 * a plan handle for patterns that are reused.  The single steps underneath
 * (scorch_hip_unstable.h) are the library's own business.
 *
 * The library replaces, for device-resident operands only, the reference's
 * pybind11 module `scorch_ops` (csrc/ops.cpp, csrc/spmm.h, csrc/kernels.h).
 * Where the reference passes (shape, mode_indices, values) triples of torch
 * tensors, this ABI passes the arrays underneath them:
 *
 *   CSR  "d,s":  row_ptr  int32[M + 1]   (mode_indices[1][0], "pos")
 *                col_idx  int32[nnz]     (mode_indices[1][1], "crd")
 *                vals     T[nnz]
 *   COO  "o,o":  row_idx  int32[nnz]     (mode_indices[0][0])
 *                col_idx  int32[nnz]     (mode_indices[1][0])
 *   dense "d,d": flat row-major T[rows * cols]
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer on the current HIP device unless it
 *     says "host".  The caller owns all memory, outputs included (the
 *     reference mallocs its outputs; here the caller's allocator does).
 *   - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL is
 *     the default stream) and the call returns without waiting for it.
 *   - Return value: SCORCH_HIP_OK (0), or one of the positive error codes below; the
 *     message for the calling thread's last failure is in
 *     scorch_hip_last_error().  Arguments are validated on the host before
 *     anything is launched; index CONTENTS are not (as in the reference, an
 *     out-of-range column index is undefined behaviour).
 *   - row_ptr must be non-decreasing with row_ptr[0] == 0 and
 *     row_ptr[M] == nnz.  Column indices within a row may be in any order
 *     and may repeat.
 *   - No global mutable state (a plan handle holds its own): calls from
 *     several host threads on different streams do not interfere, provided
 *     their workspaces and plans are distinct.
 *   - Integer kernels wrap on overflow, like the reference's.
 */
#ifndef SCORCH_HIP_H_
#define SCORCH_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SCORCH_HIP_ABI_VERSION 3

/* Every function below is exported from libscorch_hip.so. */
#if defined(__GNUC__)
#define SCORCH_HIP_API __attribute__((visibility("default")))
#else
#define SCORCH_HIP_API
#endif

enum scorch_hip_status {
  SCORCH_HIP_OK = 0,
  SCORCH_HIP_EINVAL = 1,       /* bad argument (null pointer, negative size, misaligned...) */
  SCORCH_HIP_EWORKSPACE = 2,   /* workspace missing or too small */
  SCORCH_HIP_ERUNTIME = 3,     /* a HIP runtime call failed */
  SCORCH_HIP_EUNSUPPORTED = 4  /* shape outside what the kernels handle */
};

/* Epilogue selector of scorch_hip_spmm_csr_bias_act_f32. */
enum scorch_hip_act { SCORCH_HIP_ACT_NONE = 0, SCORCH_HIP_ACT_RELU = 1 };

/* ABI version of the loaded library (SCORCH_HIP_ABI_VERSION at build time). */
SCORCH_HIP_API int scorch_hip_abi_version(void);

/* Message of the calling thread's most recent failed call ("" if none). */
SCORCH_HIP_API const char *scorch_hip_last_error(void);

/* Optional.  Loads the library's device code for the current device now.  Otherwise the HIP
 * runtime loads it piece by piece, when the first kernel of each of the library's source files
 * is launched: about a millisecond added to the first product of each kind.  Launches nothing;
 * SCORCH_HIP_ERUNTIME without a usable device.  No counterpart in the reference. */
SCORCH_HIP_API int scorch_hip_init(void);

/* ------------------------------------------------------------------------
 * SpMM: C[M,N] = A_csr[M,K] * B[K,N], all of one dtype.
 *
 * Replaces spmm_csr_float_v2 (csrc/spmm.h:2007-2089; the fp32 symbol
 * scorch.matmul resolves first, src/scorch/prebuilt_kernels.py:45) and
 * spmm_csr_typed<T> (csrc/spmm.h:91-150), bound as
 * prebuilt_spmm_csr_{f32,f64,i32,i64} (csrc/ops.cpp:30-39,92-98).  The
 * reference's tile_size argument has no counterpart.
 *
 * Every element of C is written (rows without entries become zero); C need
 * not be initialised.  `workspace` holds partial sums of rows that are split
 * between wavefronts; it must be at least
 * scorch_hip_spmm_csr_workspace_bytes(M, nnz, N, sizeof(T)) bytes, 256-byte
 * aligned, and must not be shared by calls that may run concurrently.
 * Results are bit-reproducible from run to run for a given shape.
 * ---------------------------------------------------------------------- */
SCORCH_HIP_API size_t scorch_hip_spmm_csr_workspace_bytes(int64_t M, int64_t nnz, int64_t N, size_t elem_size);

SCORCH_HIP_API int scorch_hip_spmm_csr_f32(int64_t M, int64_t K, int64_t N, int64_t nnz,
                            const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                            const float *B, float *C,
                            void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_f64(int64_t M, int64_t K, int64_t N, int64_t nnz,
                            const int32_t *row_ptr, const int32_t *col_idx, const double *vals,
                            const double *B, double *C,
                            void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_i32(int64_t M, int64_t K, int64_t N, int64_t nnz,
                            const int32_t *row_ptr, const int32_t *col_idx, const int32_t *vals,
                            const int32_t *B, int32_t *C,
                            void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_i64(int64_t M, int64_t K, int64_t N, int64_t nnz,
                            const int32_t *row_ptr, const int32_t *col_idx, const int64_t *vals,
                            const int64_t *B, int64_t *C,
                            void *workspace, size_t workspace_bytes, void *stream);

/* scorch_hip_spmm_csr_f32 for callers that cannot allocate device memory or
 * hand over a workspace: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.
 * Same kernels and bit-identical results; the carry records live in a static
 * device array of SCORCH_HIP_STATIC_SCRATCH_BYTES inside the library (every
 * GPU the library has run on holds its copy until the process ends) instead of
 * a workspace argument, and the call makes no hipMalloc / hipFree.
 *   - Shapes whose scorch_hip_spmm_csr_workspace_bytes(M, nnz, N, 4) exceeds
 *     SCORCH_HIP_STATIC_SCRATCH_BYTES are refused with SCORCH_HIP_EWORKSPACE
 *     (the 1,048,576-row, 17.8 M-entry, N = 128 product needs 38 MB and fits).
 *   - All calls on one GPU share that GPU's array: calls that may overlap in
 *     time on one GPU (two streams, two host threads) race on it.  Calls on one
 *     stream are ordered and safe.
 *   - The first call on a device looks the array's address up
 *     (hipGetSymbolAddress); make that call outside a graph capture. */
#define SCORCH_HIP_STATIC_SCRATCH_BYTES ((size_t)48 << 20)
SCORCH_HIP_API int scorch_hip_spmm_csr_f32_static(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                   const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                                   const float *B, float *C, void *stream);

/* Fused C = act(A * B + bias), bias is T[N] broadcast over rows.
 * Replaces spmm_csr_bias_act<float, relu> (csrc/spmm.h:28-89), bound as
 * spmm_csr_bias_float and spmm_csr_bias_relu_float (csrc/ops.cpp:167-208).
 * `act` is a scorch_hip_act.  Workspace as for scorch_hip_spmm_csr_f32. */
SCORCH_HIP_API int scorch_hip_spmm_csr_bias_act_f32(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                     const int32_t *row_ptr, const int32_t *col_idx,
                                     const float *vals, const float *B, const float *bias,
                                     int act, float *C,
                                     void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * SDDMM: out_vals[p] = mask_vals[p] * <A[i_p, 0:K], B[j_p, 0:K]> for every
 * stored entry p = (i_p, j_p) of the mask.  A is [M, K], B is [n_cols, K]:
 * B is indexed [j, k], i.e. the dense product is A * B^T.
 *
 * _coo replaces sddmm_coo_float_prebuilt (csrc/kernels.h:508-570, bound at
 * csrc/ops.cpp:210-217): the result's index arrays are the mask's own, so
 * only values are produced; entries may be in any order.
 *
 * _csr covers the "d,s" mask of einsum("ij,ik,jk->ij"), which the reference
 * serves with generated code whose result is a coordinate tensor with one
 * entry per mask entry, in mask order, explicit zeros kept
 * (src/scorch/ops.py:638-666, src/scorch/compiler/cin_lowerer.py:2286-2326).
 * out_row_idx, when not NULL, receives the row of every entry (the result's
 * mode_indices[0][0]); its mode_indices[1][0] is col_idx itself.
 *
 * mask_vals may be NULL in every SDDMM entry point: every stored entry of the
 * mask is then taken to be 1 (an attention mask, the mask of this benchmark's
 * SDDMM configuration) and nothing is read for it.
 * ---------------------------------------------------------------------- */
SCORCH_HIP_API int scorch_hip_sddmm_coo_f32(int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                             const int32_t *row_idx, const int32_t *col_idx,
                             const float *mask_vals, const float *A, const float *B,
                             float *out_vals, void *stream);
SCORCH_HIP_API int scorch_hip_sddmm_csr_f32(int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                             const int32_t *row_ptr, const int32_t *col_idx,
                             const float *mask_vals, const float *A, const float *B,
                             float *out_vals, int32_t *out_row_idx, void *stream);

/* ------------------------------------------------------------------------
 * SpMV: y[M] = A_csr[M,K] * x[K].
 * Replaces spmv_csr<T> (csrc/kernels.h:13-49), bound as
 * prebuilt_spmv_csr_{f32,f64,i32,i64} (csrc/ops.cpp:52-61,100-101).
 * Every element of y is written.  `workspace` (partial sums of rows split
 * between wavefronts): scorch_hip_spmv_csr_workspace_bytes(M, nnz, sizeof(T))
 * bytes, 256-byte aligned.  Results are bit-reproducible from run to run.
 * ---------------------------------------------------------------------- */
SCORCH_HIP_API size_t scorch_hip_spmv_csr_workspace_bytes(int64_t M, int64_t nnz, size_t elem_size);

SCORCH_HIP_API int scorch_hip_spmv_csr_f32(int64_t M, int64_t K, int64_t nnz, const int32_t *row_ptr,
                            const int32_t *col_idx, const float *vals, const float *x,
                            float *y, void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmv_csr_f64(int64_t M, int64_t K, int64_t nnz, const int32_t *row_ptr,
                            const int32_t *col_idx, const double *vals, const double *x,
                            double *y, void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmv_csr_i32(int64_t M, int64_t K, int64_t nnz, const int32_t *row_ptr,
                            const int32_t *col_idx, const int32_t *vals, const int32_t *x,
                            int32_t *y, void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmv_csr_i64(int64_t M, int64_t K, int64_t nnz, const int32_t *row_ptr,
                            const int32_t *col_idx, const int64_t *vals, const int64_t *x,
                            int64_t *y, void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * SpGEMM: C_csr[M,N] = A_csr[M,K] * B_csr[K,N], in two calls.
 * Replaces spmspm_csr<T> (csrc/kernels.h:52-202), bound as
 * prebuilt_spmspm_csr_{f32,f64,i32,i64} and spmspm_csr_float
 * (csrc/ops.cpp:41-50,99,113).  The reference allocates the result inside one
 * call; here the caller owns it, so the call is split where the size becomes
 * known:
 *   1. _symbolic writes c_row_ptr[M + 1] (device).  The caller reads
 *      c_row_ptr[M] back (that read synchronises) and allocates c_col_idx
 *      and c_vals of that length.  c_row_ptr[M] == -1 means that the result
 *      has 2^31 entries or more, which its int32 row pointer cannot hold: the
 *      rest of c_row_ptr is then meaningless and _numeric must not be called.
 *   2. _numeric_<T> fills c_col_idx and c_vals.
 * As in the reference, column indices are ascending within each row and every
 * structurally reachable entry is stored, also when its value sums to zero.
 * The structure is exact and the same on every run; floating-point sums are
 * accumulated atomically, so their last bits may vary between runs.
 * `workspace`: scorch_hip_spgemm_csr_workspace_bytes(M, N, sizeof(T)) bytes,
 * 256-byte aligned (the symbolic call needs no more than elem_size = 1).
 * ---------------------------------------------------------------------- */
SCORCH_HIP_API size_t scorch_hip_spgemm_csr_workspace_bytes(int64_t M, int64_t N, size_t elem_size);

SCORCH_HIP_API int scorch_hip_spgemm_csr_symbolic(int64_t M, int64_t K, int64_t N,
                                   const int32_t *a_row_ptr, const int32_t *a_col_idx,
                                   const int32_t *b_row_ptr, const int32_t *b_col_idx,
                                   int32_t *c_row_ptr,
                                   void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spgemm_csr_numeric_f32(int64_t M, int64_t K, int64_t N,
                                   const int32_t *a_row_ptr, const int32_t *a_col_idx, const float *a_vals,
                                   const int32_t *b_row_ptr, const int32_t *b_col_idx, const float *b_vals,
                                   const int32_t *c_row_ptr, int32_t *c_col_idx, float *c_vals,
                                   void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spgemm_csr_numeric_f64(int64_t M, int64_t K, int64_t N,
                                   const int32_t *a_row_ptr, const int32_t *a_col_idx, const double *a_vals,
                                   const int32_t *b_row_ptr, const int32_t *b_col_idx, const double *b_vals,
                                   const int32_t *c_row_ptr, int32_t *c_col_idx, double *c_vals,
                                   void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spgemm_csr_numeric_i32(int64_t M, int64_t K, int64_t N,
                                   const int32_t *a_row_ptr, const int32_t *a_col_idx, const int32_t *a_vals,
                                   const int32_t *b_row_ptr, const int32_t *b_col_idx, const int32_t *b_vals,
                                   const int32_t *c_row_ptr, int32_t *c_col_idx, int32_t *c_vals,
                                   void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spgemm_csr_numeric_i64(int64_t M, int64_t K, int64_t N,
                                   const int32_t *a_row_ptr, const int32_t *a_col_idx, const int64_t *a_vals,
                                   const int32_t *b_row_ptr, const int32_t *b_col_idx, const int64_t *b_vals,
                                   const int32_t *c_row_ptr, int32_t *c_col_idx, int64_t *c_vals,
                                   void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * Row softmax over the stored values of a CSR matrix:
 * out[p] = exp(scale * v[p] - m_i) / sum_q exp(scale * v[q] - m_i), q over
 * row i, m_i the row maximum of scale * v.  out may alias vals.
 * The reference composes this step from torch scatter ops in its attention
 * benchmark (_sparse_softmax_csr_vectorized,
 * bench/bench_sparse_transformer.py:277-297, applied to scores * scale at
 * :362-368); it has no native kernel for it.
 * `workspace` (256-byte aligned, scorch_hip_softmax_csr_workspace_bytes; 0
 * bytes, and then it may be NULL, for nnz <= 4096) holds the list of rows
 * longer than 4096 entries between the two kernels; not to be shared by calls
 * that may overlap in time.
 * ---------------------------------------------------------------------- */
SCORCH_HIP_API size_t scorch_hip_softmax_csr_workspace_bytes(int64_t M, int64_t nnz);
SCORCH_HIP_API int scorch_hip_softmax_csr_f32(int64_t M, int64_t nnz, const int32_t *row_ptr,
                               const float *vals, float scale, float *out, void *workspace,
                               size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * A plan: what can be found out once about a CSR pattern that is multiplied by again and again,
 * kept by the library behind an opaque handle.  The reference's dispatch is stateless
 * (src/scorch/prebuilt_kernels.py:198-224), but its callers multiply by one matrix many times (a
 * graph's normalised adjacency in every layer and iteration, bench/bench_gcn.py:314-329; an
 * attention mask for every head, bench/bench_sparse_transformer.py:354-372).
 *
 * scorch_hip_csr_plan_create inspects the index arrays (one kernel, one read of 32 bytes: it
 * waits for `stream`) and refuses a malformed index with SCORCH_HIP_EINVAL before any kernel
 * dereferences it: row_ptr that does not start at 0, end at nnz or decreases, a column index
 * outside [0, n_cols).  The plan keeps the two POINTERS, not copies: the arrays must stay where
 * they are, unchanged, until the plan is destroyed.  A plan belongs to the device that was
 * current when it was made and to one host thread at a time; the products of one plan share its
 * scratch memory, so they must not overlap in time (one stream, or the caller orders them).
 *
 * scorch_hip_spmm_csr_plan_f32      C = act(A * B + bias) like scorch_hip_spmm_csr_bias_act_f32
 *                                   (bias may be NULL with act = SCORCH_HIP_ACT_NONE): the
 *                                   row-split kernel when all rows are short, else the merge-path
 *                                   kernels reading chunk boundaries computed once per N, with the
 *                                   result zero-filled in one pass when most rows are empty.
 *                                   The merge-path results are those of scorch_hip_spmm_csr_f32 /
 *                                   _bias_act_f32 bit for bit; the row-split kernel adds a row's
 *                                   terms up in another grouping (equal to rounding).  Both are
 *                                   bit-reproducible from call to call.
 * scorch_hip_sddmm_csr_plan_f32     like scorch_hip_sddmm_csr_f32 (mask_vals and out_row_idx may
 *                                   be NULL); a mask with a dense right operand of 8 to 20 MB is
 *                                   served from per-XCD entry lists built once.  Bit-identical.
 * scorch_hip_softmax_csr_plan_f32   like scorch_hip_softmax_csr_f32; one launch when no row is
 *                                   longer than 4096.  Bit-identical.
 *
 * The first product of a kind and width allocates device memory (hipMalloc: not under graph
 * capture); scorch_hip_csr_plan_prepare does that ahead of time, after which the product calls
 * of that kind and width allocate nothing and do not synchronise.  `width` is N for
 * SCORCH_HIP_PLAN_SPMM_F32 and SCORCH_HIP_PLAN_SPMM_DENSE_F32, K for SCORCH_HIP_PLAN_SDDMM_F32
 * and ignored for SCORCH_HIP_PLAN_SOFTMAX_F32.  A plan holds boundaries for at most 8 widths of N; a ninth
 * replaces the oldest.
 *
 * scorch_hip_csr_plan_info writes SCORCH_HIP_PLAN_INFO_INTS int64 to `info` (host): M, n_cols,
 * nnz, the longest row, the number of empty rows, 1 if every row's column indices increase
 * strictly else 0, bytes of device memory the plan holds, 0.
 * ---------------------------------------------------------------------- */
typedef struct scorch_hip_csr_plan scorch_hip_csr_plan;
enum scorch_hip_plan_op {
  SCORCH_HIP_PLAN_SPMM_F32 = 0,
  SCORCH_HIP_PLAN_SDDMM_F32 = 1,
  SCORCH_HIP_PLAN_SOFTMAX_F32 = 2,
  SCORCH_HIP_PLAN_SPMM_DENSE_F32 = 3 /* products through a scorch_hip_dense_plan N wide */
};
#define SCORCH_HIP_PLAN_INFO_INTS 8
SCORCH_HIP_API int scorch_hip_csr_plan_create(int64_t M, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                               const int32_t *col_idx, void *stream, scorch_hip_csr_plan **plan /* host */);
SCORCH_HIP_API int scorch_hip_csr_plan_destroy(scorch_hip_csr_plan *plan);
SCORCH_HIP_API int scorch_hip_csr_plan_info(const scorch_hip_csr_plan *plan, int64_t *info /* host, [8] */);
SCORCH_HIP_API int scorch_hip_csr_plan_prepare(scorch_hip_csr_plan *plan, int op, int64_t width, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_plan_f32(scorch_hip_csr_plan *plan, int64_t N, const float *vals,
                                 const float *B, const float *bias, int act, float *C, void *stream);
SCORCH_HIP_API int scorch_hip_sddmm_csr_plan_f32(scorch_hip_csr_plan *plan, int64_t K, const float *mask_vals,
                                  const float *A, const float *B, float *out_vals, int32_t *out_row_idx,
                                  void *stream);
SCORCH_HIP_API int scorch_hip_softmax_csr_plan_f32(scorch_hip_csr_plan *plan, const float *vals, float scale,
                                    float *out, void *stream);

/* The dense side of the same idea: a dense fp32 operand B[K, N] that many products use unchanged
 * (a weight matrix: the reference's weight-sparse autoencoder multiplies every batch by the same
 * decoder weight, bench/bench_sparse_autoencoder.py:250-276, and converts weights once outside its
 * loop, bench/README_sparse_autoencoder.md:86).  For shapes where it pays (rows of B of 2 KiB and
 * more, K * 128 bytes within an L2's reach) scorch_hip_dense_plan_create stores B a second time by
 * column tiles (hipMalloc of the size of B, one read and one write of B on `stream`); for other
 * shapes the handle only names B.  It keeps the POINTER B: the array must stay in place until the
 * plan is destroyed, and after its VALUES have changed scorch_hip_dense_plan_update copies them
 * again -- a product issued in between would use the old values, and nothing could notice.
 * scorch_hip_spmm_csr_plan_dense_f32 is scorch_hip_spmm_csr_plan_f32 with B named by its plan:
 * with the tile copy, and a sparse operand that gathers the rows of B twice or more on average,
 * every XCD keeps one tile of the copy in its L2 while all rows of A gather from it, so B comes
 * from memory once (the decoder shape, 4096 x 16,384 with 32 entries per row times 16,384 x 4096:
 * 0.10 ms against 0.25 ms); otherwise it is that call.  Results agree with the other SpMM entry
 * points to rounding and are bit-reproducible.  scorch_hip_csr_plan_prepare with
 * SCORCH_HIP_PLAN_SPMM_DENSE_F32 and width N allocates ahead of time what these products need. */
typedef struct scorch_hip_dense_plan scorch_hip_dense_plan;
SCORCH_HIP_API int scorch_hip_dense_plan_create(int64_t K, int64_t N, const float *B, void *stream,
                                 scorch_hip_dense_plan **plan /* host */);
SCORCH_HIP_API int scorch_hip_dense_plan_update(scorch_hip_dense_plan *plan, void *stream);
SCORCH_HIP_API int scorch_hip_dense_plan_destroy(scorch_hip_dense_plan *plan);
SCORCH_HIP_API int scorch_hip_spmm_csr_plan_dense_f32(scorch_hip_csr_plan *plan, const float *vals,
                                       const scorch_hip_dense_plan *dense, const float *bias, int act,
                                       float *C, void *stream);

/* ------------------------------------------------------------------------
 * Fused block-sparse attention, bf16 in / bf16 out, fp32 accumulation:
 * O[h] = softmax_rows(scale * Q[h] K[h]^T, restricted to the mask) V[h].
 * Q, K, V, O are [H, S, D] row-major bf16.  The mask is shared by all heads and
 * given as a block-CSR pattern over (S / block)^2 blocks of block x block
 * entries: block_row_ptr int32[S / block + 1], block_col_idx
 * int32[n_active_blocks]; every entry of an active block is live.  Query rows
 * whose block row has no active block give zeros.
 * Built for D = 32, 64 and 128 and block = 64 (other values:
 * SCORCH_HIP_EUNSUPPORTED).
 * One kernel does what the reference's attention benchmark composes per head
 * from SDDMM, a row softmax and SpMM (bench/bench_sparse_transformer.py:354-372);
 * the reference has no fused or bf16 counterpart.
 *
 * The _masked form serves masks that are not unions of whole blocks (the
 * reference's Longformer pattern, a sliding window plus global tokens,
 * bench/bench_sparse_transformer.py:117-141; a causal diagonal): active block i
 * is fully live when block_mask_index[i] < 0, and otherwise restricted to the
 * 64 x 64 bit mask block_masks[64 * block_mask_index[i] .. + 63], where bit j
 * of word r says that query r of the block row attends to key j of the block.
 * block_mask_index is int32[n_active_blocks], block_masks uint64[64 * n_masks]
 * (several blocks may share one mask).  Queries without any live key give zeros.
 * ---------------------------------------------------------------------- */
SCORCH_HIP_API int scorch_hip_attn_blocksparse_bf16(int64_t H, int64_t S, int64_t D, int64_t block,
                                     int64_t n_active_blocks,
                                     const int32_t *block_row_ptr, const int32_t *block_col_idx,
                                     const void *Q, const void *K, const void *V, float scale,
                                     void *O, void *stream);
SCORCH_HIP_API int scorch_hip_attn_blocksparse_masked_bf16(
    int64_t H, int64_t S, int64_t D, int64_t block, int64_t n_active_blocks,
    const int32_t *block_row_ptr, const int32_t *block_col_idx, const int32_t *block_mask_index,
    int64_t n_masks, const uint64_t *block_masks, const void *Q, const void *K, const void *V,
    float scale, void *O, void *stream);

/* Rows of a CSR matrix's entries: row_idx[p] = i for row_ptr[i] <= p < row_ptr[i+1].
 * The device-side counterpart of the "d,s" -> "o,o" index conversion the
 * reference performs on the host (STensor.from_coo / to_sparse,
 * src/scorch/stensor.py:318-365). */
SCORCH_HIP_API int scorch_hip_csr_row_indices(int64_t M, int64_t nnz, const int32_t *row_ptr,
                               int32_t *row_idx, void *stream);

/* The other direction: the CSR row pointer (M + 1 entries) of coordinates sorted
 * by row, row_ptr[r] = number of entries in rows below r.  *unsorted, which the
 * caller has set to 0, is set to 1 if a row coordinate lies outside [0, M) or
 * below its predecessor; row_ptr is then meaningless.  With it a coordinate
 * ("o,o") operand is handed to the CSR kernels, which is how this build serves
 * the reference's spmm_coo_float (csrc/spmm.h:247-372) and spmspm_coo_float
 * (csrc/kernels.h:397-497, bound at csrc/ops.cpp:140-143). */
SCORCH_HIP_API int scorch_hip_coo_row_ptr(int64_t M, int64_t nnz, const int32_t *row_idx,
                           int32_t *row_ptr, int32_t *unsorted, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SCORCH_HIP_H_ */