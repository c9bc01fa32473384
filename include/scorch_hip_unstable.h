/*
 * scorch_hip_unstable.h -- the steps underneath scorch_hip.h: INTERNAL AND UNSTABLE.
 *
 * Everything declared here is exported from libscorch_hip.so for the library's own Python host
 * layer, its tests and its benchmark: the single steps of a planned product (inspection, chunk
 * boundaries, entry lists, block descriptions, work-item lists), kernels pinned to one path, and
 * timing aids.  Their signatures and meanings may change with any SCORCH_HIP_ABI_VERSION, and
 * nothing outside this repository should bind them: a binding of the reference needs none of them
 * -- scorch_hip.h declares one call per operation, and its plan handle does inspection and
 * boundaries by itself.  The conventions of scorch_hip.h apply (device pointers, `stream`,
 * return codes).
 */
#ifndef SCORCH_HIP_UNSTABLE_H_
#define SCORCH_HIP_UNSTABLE_H_

#include "scorch_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* May be or-ed into the `act` argument of scorch_hip_spmm_csr_planned_<T>: the caller knows
 * (scorch_hip_csr_inspect reports it) that most rows of A are empty.  C is then zeroed with one
 * streaming fill and only the rows that have entries are written, as the reference does
 * (csrc/spmm.h:2024-2025, 2052: memset, then empty rows skipped), instead of a row-sized store of
 * zeros per empty row between the gathers.  Same result; ignored with a bias. */
#define SCORCH_HIP_HINT_MOSTLY_EMPTY_ROWS 0x100

/* Benchmarking aid: per-kernel durations of the calls made in between, on the
 * calling host thread.  After scorch_hip_timing_begin() the SpMM, SDDMM and
 * attention entry points record a HIP event on their stream before their first
 * kernel, between their kernels and after their last (16 events at most; later
 * ones are dropped).  scorch_hip_timing_end() waits for the last event and
 * writes the time between consecutive events, in milliseconds, to
 * interval_ms[0 .. min(*count, capacity)); *count is the number of intervals.
 * One call per bracket gives one interval per kernel, in launch order.  The
 * reference's only timing is wall-clock around a whole call
 * (src/scorch/prebuilt_kernels.py:217-222). */
SCORCH_HIP_API int scorch_hip_timing_begin(void);
SCORCH_HIP_API int scorch_hip_timing_end(float *interval_ms /* host */, int capacity, int *count /* host */);

/* Benchmarking aid: scorch_hip_spmm_csr_f32 with each of its two kernels
 * bracketed by HIP events on `stream`.  Waits for the work to finish and
 * reports the durations in milliseconds: kernel_ms[0] the merge-path SpMM
 * kernel, kernel_ms[1] the carry fix-up kernel (host array of two floats).
 * Same results as scorch_hip_spmm_csr_f32.  It synchronises, so it is not
 * meant for production loops.  No counterpart in the reference, whose only
 * timing is wall-clock around the whole call
 * (src/scorch/prebuilt_kernels.py:217-222). */
SCORCH_HIP_API int scorch_hip_spmm_csr_f32_timed(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                  const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                                  const float *B, float *C,
                                  void *workspace, size_t workspace_bytes, void *stream,
                                  float *kernel_ms /* host, [2] */);

/* ------------------------------------------------------------------------
 * What a caller can compute once per sparse operand and reuse in every later
 * product with it.  The reference has no such step: its dispatch is stateless
 * (src/scorch/prebuilt_kernels.py:198-224), but its callers multiply by one
 * matrix many times (a graph's normalised adjacency in every layer and
 * iteration, bench/bench_gcn.py:314-329; weights converted once outside the
 * loop, bench/README_sparse_autoencoder.md:86).  All of it lives in memory the
 * caller owns; the library keeps no state.
 *
 * scorch_hip_csr_inspect writes SCORCH_HIP_INSPECT_REPORT_INTS int32 to `report` (device):
 *   [0] 1 if row_ptr is malformed (row_ptr[0] != 0, row_ptr[M] != nnz, or a
 *       pointer below its predecessor), else 0
 *   [1] 1 if a column index lies outside [0, K), else 0
 *   [2] the longest row
 *   [3] the number of empty rows
 *   [4] the number of entries that do not exceed the entry before them in their
 *       row (0: every row's column indices increase strictly)
 *   [5] the number of runs: maximal stretches of a row's entries that increase
 *       and lie in one aligned group of 64 columns.  nnz / (64 * runs) bounds
 *       from above the share of stored positions in the 64 x 64 blocks the
 *       pattern touches: a graph is told from a mask made of blocks without
 *       looking at blocks
 *   [6], [7] 0 (reserved)
 * ([4] and [5] mean what they say only when [0] is 0.)
 * It reads row_ptr[0..M] and col_idx[0..nnz) only, so it is safe on malformed
 * input; a caller that reads the report back (one synchronisation) can refuse
 * the operand before any kernel dereferences it, and knows whether all rows
 * are short.
 * ---------------------------------------------------------------------- */
#define SCORCH_HIP_INSPECT_REPORT_INTS 8
SCORCH_HIP_API int scorch_hip_csr_inspect(int64_t M, int64_t K, int64_t nnz, const int32_t *row_ptr,
                           const int32_t *col_idx, int32_t *report /* device, [8] */, void *stream);

/* Row-split SpMM for matrices whose rows are all short: C = act(A * B + bias)
 * in one launch, without workspace (a team of lanes per row; no rows are cut,
 * so there are no carries to fold).  Same contraction as
 * scorch_hip_spmm_csr_<T> / _bias_act_f32 (csrc/spmm.h:28-150,2007-2089); bias
 * may be NULL (then act must be SCORCH_HIP_ACT_NONE).  Correct for rows of any
 * length but slow when one is long (a row is walked by one team): meant for
 * operands whose longest row, as scorch_hip_csr_inspect reports it, is a few
 * hundred entries at most.  Bit-reproducible. */
SCORCH_HIP_API int scorch_hip_spmm_csr_rows_f32(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                 const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                                 const float *B, const float *bias, int act, float *C, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_rows_f64(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                 const int32_t *row_ptr, const int32_t *col_idx, const double *vals,
                                 const double *B, const double *bias, int act, double *C, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_rows_i32(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                 const int32_t *row_ptr, const int32_t *col_idx, const int32_t *vals,
                                 const int32_t *B, const int32_t *bias, int act, int32_t *C, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_rows_i64(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                 const int32_t *row_ptr, const int32_t *col_idx, const int64_t *vals,
                                 const int64_t *B, const int64_t *bias, int act, int64_t *C, void *stream);

/* Merge-path SpMM with its chunk boundaries computed beforehand.
 * scorch_hip_spmm_csr_bounds fills `bounds` (device, 8-byte aligned,
 * scorch_hip_spmm_csr_bounds_bytes(M, nnz, N, sizeof(T)) bytes) from row_ptr;
 * the boundaries depend on row_ptr, N and the element size only.
 * scorch_hip_spmm_csr_planned_<T> is scorch_hip_spmm_csr_<T> (with the
 * optional bias / activation of _bias_act_f32) whose wavefronts read their two
 * boundaries from `bounds` instead of searching row_ptr; bounds may be NULL,
 * and the call is then the unplanned one.  Same results bit for bit.  The
 * caller vouches that `bounds` was built from this row_ptr with these M, nnz,
 * N and element size. */
SCORCH_HIP_API size_t scorch_hip_spmm_csr_bounds_bytes(int64_t M, int64_t nnz, int64_t N, size_t elem_size);
SCORCH_HIP_API int scorch_hip_spmm_csr_bounds(int64_t M, int64_t nnz, int64_t N, size_t elem_size,
                               const int32_t *row_ptr, void *bounds, size_t bounds_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_planned_f32(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                    const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                                    const float *B, const float *bias, int act, float *C,
                                    const void *bounds, size_t bounds_bytes,
                                    void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_planned_f64(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                    const int32_t *row_ptr, const int32_t *col_idx, const double *vals,
                                    const double *B, const double *bias, int act, double *C,
                                    const void *bounds, size_t bounds_bytes,
                                    void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_planned_i32(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                    const int32_t *row_ptr, const int32_t *col_idx, const int32_t *vals,
                                    const int32_t *B, const int32_t *bias, int act, int32_t *C,
                                    const void *bounds, size_t bounds_bytes,
                                    void *workspace, size_t workspace_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_planned_i64(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                    const int32_t *row_ptr, const int32_t *col_idx, const int64_t *vals,
                                    const int64_t *B, const int64_t *bias, int act, int64_t *C,
                                    const void *bounds, size_t bounds_bytes,
                                    void *workspace, size_t workspace_bytes, void *stream);

/* SpMM against a wide dense operand that is reused (a weight matrix), stored
 * once by column tiles.  The reference's weight-sparse autoencoder multiplies
 * every batch by the same dense decoder weight (bench/bench_sparse_autoencoder.py:
 * 250-276); with B row-major each stored entry of A gathers a whole row of B
 * from memory, although every row of B is gathered several times.
 *   Bt[tile][k][c]: tile t holds columns [32 t, 32 t + 32) of B (fp32; 128-byte
 *   tile rows), K rows contiguous, zero padded past N;
 *   scorch_hip_dense_tiled_bytes(K, N, 4) bytes, 128-byte aligned.
 * scorch_hip_dense_to_tiled_f32 builds Bt from a row-major B (one read and one
 * write of B).  scorch_hip_spmm_csr_tiled_f32 is scorch_hip_spmm_csr_planned_f32
 * with Bt in place of B: every XCD keeps one tile of Bt in its L2 while all rows
 * of A gather from it, so B comes from memory about once.  Results agree with
 * the other SpMM entry points to rounding (rows of more than 64 entries are
 * summed in another grouping) and are bit-reproducible from run to run.
 * longest_row is the longest row of A if the caller knows it (scorch_hip_csr_inspect reports it), else
 * 0: with no row beyond 32 to 64 entries (depending on the shape) no row is shared between wavefronts,
 * and the launch that folds shared rows' partial sums is left out.
 * scorch_hip_dense_tiled_recommended is 1 when the layout pays: rows of B of
 * 2 KiB and more, K * 128 bytes within an L2's reach (3 MiB), and nnz >= 2 K. */
SCORCH_HIP_API size_t scorch_hip_dense_tiled_bytes(int64_t K, int64_t N, size_t elem_size);
SCORCH_HIP_API int scorch_hip_dense_tiled_recommended(int64_t K, int64_t N, int64_t nnz, size_t elem_size);
SCORCH_HIP_API int scorch_hip_dense_to_tiled_f32(int64_t K, int64_t N, const float *B, float *Bt,
                                  size_t bt_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_tiled_f32(int64_t M, int64_t K, int64_t N, int64_t nnz,
                                  const int32_t *row_ptr, const int32_t *col_idx, const float *vals,
                                  const float *Bt, size_t bt_bytes, const float *bias, int act, float *C,
                                  const void *bounds, size_t bounds_bytes,
                                  void *workspace, size_t workspace_bytes, int64_t longest_row, void *stream);

/* SDDMM for a CSR mask whose pattern is used again and again (an attention mask
 * serves every head, layer and step), with B larger than one of the GPU's eight
 * L2 caches but not than all of them together.  The reference has no such step.
 * scorch_hip_sddmm_csr_lists sorts the mask's entries once into eight lists by
 * the eighth of the column range they fall in (`lists`: device, 256-byte aligned,
 * scorch_hip_sddmm_csr_lists_bytes(nnz) bytes; it depends on row_ptr, col_idx and
 * n_cols only, and a list holds its entries in the mask's order, the same on every
 * build).  scorch_hip_sddmm_csr_listed_f32 is scorch_hip_sddmm_csr_batched_f32
 * computed list by list, each list on one XCD, whose L2 then keeps that eighth of
 * B: the same products, the same results bit for bit.  K <= 256.
 * scorch_hip_sddmm_csr_list_values_f32 copies the mask's values into the lists' order
 * (listed_vals[e] = vals[position of list entry e]); handed to the listed kernel as `listed_vals`
 * they are read with the entries, coalesced, instead of one scattered load per entry (mask_vals is
 * then not read).  The copy is the caller's to redo when the values change.  listed_vals may be
 * NULL, and so may mask_vals (a mask of ones). */
SCORCH_HIP_API size_t scorch_hip_sddmm_csr_lists_bytes(int64_t nnz);
SCORCH_HIP_API int scorch_hip_sddmm_csr_lists(int64_t M, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                               const int32_t *col_idx, void *lists, size_t lists_bytes, void *stream);
SCORCH_HIP_API int scorch_hip_sddmm_csr_list_values_f32(int64_t nnz, const void *lists, size_t lists_bytes,
                                         const float *vals, float *listed_vals /* [nnz] */, void *stream);
SCORCH_HIP_API int scorch_hip_sddmm_csr_listed_f32(int64_t batch, int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                                    const void *lists, size_t lists_bytes, const float *mask_vals,
                                    const float *listed_vals, const float *A, const float *B, float *out_vals,
                                    int32_t *out_row_idx, void *stream);

/* The same for `batch` value arrays over one pattern, for a caller that knows the pattern's longest
 * row (scorch_hip_csr_inspect reports it): with longest_row <= 4096 one launch and no workspace
 * (NULL, 0); with longest_row <= 16,384 the two launches that serve longer rows in stretches are
 * left out; the workspace is that of scorch_hip_softmax_csr_workspace_bytes otherwise.  The entries
 * of `out` that belong to a row longer than stated may be left unwritten. */
SCORCH_HIP_API int scorch_hip_softmax_csr_known_rows_f32(int64_t batch, int64_t M, int64_t nnz,
                               int64_t longest_row, const int32_t *row_ptr, const float *vals,
                               float scale, float *out, void *workspace, size_t workspace_bytes,
                               void *stream);

/* The same with long block rows shared out among workgroups (a mask with a global token has a
 * block row that holds every key block: as one workgroup's work it sets the time of the whole
 * launch).  The work is a list of items, longest first, 4 int32 each (16-byte aligned): block row,
 * begin and end of its stretch within block_col_idx, and the slot its partial result goes to, or
 * -1 for a whole block row, which writes O itself.  The stretches of a shared-out row have
 * consecutive slots; split_rows lists those rows, 4 int32 each: block row, first slot, number of
 * stretches, 0.  Partial results (unnormalised sums, reference maximum, row sum per query) go
 * through `workspace` (256-byte aligned, scorch_hip_attn_blocksparse_split_workspace_bytes(H,
 * n_slots, D) bytes; not to be shared by calls that may overlap in time) and a second kernel
 * combines them.  block_mask_index may be NULL (every block fully live).  With pair_items != 0 a
 * workgroup takes two items, the k-th longest and then the k-th shortest of the list, so that all
 * workgroups carry about the same work and half as many start: it pays where the items differ in
 * length (or are very short) and the launch is about one to four times what the chip holds at
 * once, and costs a few per cent elsewhere; same results bit for bit.  With priority_step > 0 a
 * wavefront's priority on its SIMD follows the key blocks its workgroup has left to do (this item's
 * and, before the second item of a pair, that item's), in four levels of priority_step blocks: the
 * wavefronts that were dispatched first win a SIMD's arbitration otherwise, two of a CU's four
 * workgroups finish a quarter of the launch ahead of the other two and the CU runs half empty from
 * there on.  It pays where a CU holds two workgroups or more at a time; a quarter of the most any
 * workgroup has to do is the step to give.  Same results bit for bit.  No counterpart in the
 * reference, like the two entry points above. */
SCORCH_HIP_API size_t scorch_hip_attn_blocksparse_split_workspace_bytes(int64_t H, int64_t n_slots, int64_t D);
SCORCH_HIP_API int scorch_hip_attn_blocksparse_split_bf16(
    int64_t H, int64_t S, int64_t D, int64_t block, int64_t n_active_blocks, int64_t n_items,
    const int32_t *items, int pair_items, int priority_step, int64_t n_split_rows, const int32_t *split_rows,
    int64_t n_slots, const int32_t *block_col_idx, const int32_t *block_mask_index, int64_t n_masks,
    const uint64_t *block_masks, const void *Q, const void *K, const void *V, float scale, void *O,
    void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------
 * Fused block-sparse attention in fp32: the same computation as
 * scorch_hip_attn_blocksparse_masked_bf16 / _split_bf16 with fp32 Q, K, V, O
 * (H, S, D), fp32 probabilities and fp32 accumulation on the fp32 matrix
 * instruction: the per-head SDDMM -> row softmax -> SpMM composition of
 * bench/bench_sparse_transformer.py:354-372 in one kernel and at that
 * composition's precision.  D = 32, 64 or 128, 64 x 64 blocks.
 * block_mask_index may be NULL (every listed block fully live).  With
 * n_items = 0 every block row is one workgroup's (block_row_ptr is read); with
 * n_items > 0 the work items are `items` (4 x int32 each: block row, first and
 * one-past-last position in block_col_idx, partial slot or -1), the block rows
 * that were shared out are `split_rows` (block row, first slot, stretches, 0)
 * and `workspace` (256-byte aligned,
 * scorch_hip_attn_blocksparse_f32_workspace_bytes(H, n_slots, D)) takes their
 * partial results; block_row_ptr is then not read.  The reference has no fused
 * kernel.
 * ---------------------------------------------------------------------- */
SCORCH_HIP_API size_t scorch_hip_attn_blocksparse_f32_workspace_bytes(int64_t H, int64_t n_slots, int64_t D);
SCORCH_HIP_API int scorch_hip_attn_blocksparse_f32(
    int64_t H, int64_t S, int64_t D, int64_t block, int64_t n_active_blocks, const int32_t *block_row_ptr,
    const int32_t *block_col_idx, const int32_t *block_mask_index, int64_t n_masks, const uint64_t *block_masks,
    int64_t n_items, const int32_t *items, int64_t n_split_rows, const int32_t *split_rows, int64_t n_slots,
    const float *Q, const float *K, const float *V, float scale, float *O, void *workspace, size_t workspace_bytes,
    void *stream);

/* ------------------------------------------------------------------------
 * SDDMM and SpMM in fp32 for a CSR operand whose entries cluster in 64 x 64
 * blocks (attention masks), on the fp32 matrix instruction: the same results
 * as scorch_hip_sddmm_csr_batched_f32 and scorch_hip_spmm_csr_batched_f32 (the
 * reference's csrc/kernels.h:508-570 and csrc/spmm.h:2007-2089 for every head,
 * as bench/bench_sparse_transformer.py:354-372 composes them), up to the order
 * of the fp32 sums, for a pattern the caller has described by blocks:
 *   block_col_idx[n_active_blocks]    block column of every active block, block
 *                                     row major;
 *   block_words[n_active_blocks * 64] bit c of word r of a block: column c of
 *                                     the block is stored in row r of it;
 *   block_off[n_active_blocks * 64]   position in the CSR arrays of the first
 *                                     stored entry of row r inside the block;
 *   block_cols[n_active_blocks]       (SpMM; may be NULL) bit c: some row of the
 *                                     block stores column c.  A row of B that
 *                                     no entry of a block refers to is then not
 *                                     used for that block, whatever it holds.
 * Every row's column indices must increase strictly (the entry of bit c is
 * then block_off + the number of set bits below c); the arrays are trusted.
 * M and the sparse operand's column count must be multiples of 64, the dense
 * operands 32, 64 or 128 wide.  `items` (4 x int32 each: block row, first and
 * one-past-last position in block_col_idx, 0) are the work items: for the
 * SDDMM any cover of the active blocks by stretches of block rows (the fourth
 * integer is not read); for the SpMM every block row either once and whole
 * (fourth integer -1; a block row without blocks gives zero rows) or as
 * consecutive stretches whose fourth integers are consecutive slots of
 * `workspace` (256-byte aligned,
 * scorch_hip_spmm_csr_blocked_workspace_bytes(H, n_slots, N)), named in
 * `split_rows` (block row, first slot, stretches, 0): a second kernel adds a
 * row's stretches up in their order, so the result does not depend on timing.  A is (H, M, K), B is (H, n_cols, K) [SDDMM] or (H, K, N)
 * [SpMM], mask_vals is [nnz] (shared by the heads; NULL: every value is 1, an
 * attention mask, and nothing is read for it), vals and out_vals are (H, nnz),
 * C is (H, M, N).  out_row_idx (may be NULL) receives the row of
 * every entry.
 * ---------------------------------------------------------------------- */
SCORCH_HIP_API int scorch_hip_sddmm_csr_blocked_f32(
    int64_t H, int64_t M, int64_t n_cols, int64_t K, int64_t nnz, int64_t n_active_blocks,
    const int32_t *block_col_idx, const uint64_t *block_words, const int32_t *block_off, int64_t n_items,
    const int32_t *items, const float *mask_vals, const float *A, const float *B, float *out_vals,
    int32_t *out_row_idx, void *stream);
SCORCH_HIP_API size_t scorch_hip_spmm_csr_blocked_workspace_bytes(int64_t H, int64_t n_slots, int64_t N);
SCORCH_HIP_API int scorch_hip_spmm_csr_blocked_f32(
    int64_t H, int64_t M, int64_t K, int64_t N, int64_t nnz, int64_t n_active_blocks, const int32_t *block_col_idx,
    const uint64_t *block_words, const int32_t *block_off, const uint64_t *block_cols, int64_t n_items,
    const int32_t *items, int64_t n_split_rows, const int32_t *split_rows, int64_t n_slots, const float *vals,
    const float *B, float *C, void *workspace, size_t workspace_bytes, void *stream);

/* The block description of a CSR pattern, built on the device in two calls with one host read
 * between them.  The reference's attention loop wraps fresh operands for every head and call
 * (bench/bench_sparse_transformer.py:354-372), so describing a pattern must cost about what one
 * product costs.  M and n_cols multiples of 64, at most 131,072 block columns.
 *   _block_count  block_row_ptr[M / 64 + 1]: running count of the active blocks (those that hold
 *                 a stored entry) per block row.  The caller reads block_row_ptr[M / 64] back,
 *                 the number of active blocks, and allocates the arrays of the second call.
 *   _block_fill   block_col_idx, block_words, block_off, block_cols as described above, and
 *                 block_nnz[n_active_blocks], the number of stored positions of every block
 *                 (4096: fully stored).  Entries may repeat and rows need not be sorted for
 *                 block_words / block_cols / block_nnz to be right; block_off is what the block
 *                 kernels need only when every row's columns increase strictly
 *                 (scorch_hip_csr_inspect, report[4] == 0).  Column indices outside [0, n_cols)
 *                 are skipped by both calls. */
SCORCH_HIP_API int scorch_hip_csr_block_count(int64_t M, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                                              const int32_t *col_idx, int32_t *block_row_ptr, void *stream);
SCORCH_HIP_API int scorch_hip_csr_block_fill(int64_t M, int64_t n_cols, int64_t nnz, const int32_t *row_ptr,
                                             const int32_t *col_idx, const int32_t *block_row_ptr,
                                             int64_t n_active_blocks, int32_t *block_col_idx,
                                             uint64_t *block_words, int32_t *block_off, uint64_t *block_cols,
                                             int32_t *block_nnz, void *stream);

/* ------------------------------------------------------------------------
 * One sparsity pattern, `batch` value arrays: the three steps of the reference's
 * sparse attention -- SDDMM, row softmax, SpMM, which its benchmark runs head by
 * head from a Python loop (bench/bench_sparse_transformer.py:325,354-372) -- each
 * as one launch over all heads (grid.y = head).  For any CSR mask and any head
 * dimension and in fp32; the fused kernel above is bf16, for D = 32, 64 or 128.
 * Problem h uses A + h M K, B + h n_cols K (resp. vals + h nnz, B + h K N) and
 * writes out + h nnz (resp. C + h M N); the pattern and, for SDDMM, the mask's
 * values are shared.  batch <= 65535.  Results are those of `batch` separate
 * calls, bit for bit.
 *   _sddmm_csr_batched: out_row_idx (may be NULL) is written once, nnz entries.
 *   _softmax_csr_batched: workspace as for scorch_hip_softmax_csr_f32.
 *   _spmm_csr_rows_batched: the row-split kernel (short rows), no workspace.
 *   _spmm_csr_batched: the merge-path kernels; workspace of
 *     scorch_hip_spmm_csr_batched_workspace_bytes(batch, M, nnz, N) bytes;
 *     `bounds` as for scorch_hip_spmm_csr_planned_f32 (may be NULL).
 * ---------------------------------------------------------------------- */
SCORCH_HIP_API int scorch_hip_sddmm_csr_batched_f32(int64_t batch, int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                                     const int32_t *row_ptr, const int32_t *col_idx,
                                     const float *mask_vals /* [nnz] */, const float *A /* [batch, M, K] */,
                                     const float *B /* [batch, n_cols, K] */, float *out_vals /* [batch, nnz] */,
                                     int32_t *out_row_idx /* [nnz] or NULL */, void *stream);
SCORCH_HIP_API int scorch_hip_softmax_csr_batched_f32(int64_t batch, int64_t M, int64_t nnz, const int32_t *row_ptr,
                                       const float *vals /* [batch, nnz] */, float scale,
                                       float *out /* [batch, nnz] */, void *workspace, size_t workspace_bytes,
                                       void *stream);
SCORCH_HIP_API int scorch_hip_spmm_csr_rows_batched_f32(int64_t batch, int64_t M, int64_t K, int64_t N, int64_t nnz,
                                         const int32_t *row_ptr, const int32_t *col_idx,
                                         const float *vals /* [batch, nnz] */, const float *B /* [batch, K, N] */,
                                         float *C /* [batch, M, N] */, void *stream);
SCORCH_HIP_API size_t scorch_hip_spmm_csr_batched_workspace_bytes(int64_t batch, int64_t M, int64_t nnz, int64_t N);
SCORCH_HIP_API int scorch_hip_spmm_csr_batched_f32(int64_t batch, int64_t M, int64_t K, int64_t N, int64_t nnz,
                                    const int32_t *row_ptr, const int32_t *col_idx,
                                    const float *vals /* [batch, nnz] */, const float *B /* [batch, K, N] */,
                                    float *C /* [batch, M, N] */, const void *bounds, size_t bounds_bytes,
                                    void *workspace, size_t workspace_bytes, void *stream);

/* Whether a value array holds anything but `value`: *differ (device) is set to 1 if some vals[i]
 * != value (a NaN differs from everything), else to 0.  The host layer asks it of an SDDMM mask's
 * values once, to pass mask_vals = NULL from then on when they are all 1; an attention mask's are.
 * No counterpart in the reference. */
SCORCH_HIP_API int scorch_hip_values_differ_f32(int64_t n, const float *vals, float value,
                                 int32_t *differ /* device */, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SCORCH_HIP_UNSTABLE_H_ */
