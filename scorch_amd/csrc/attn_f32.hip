// Fused block-sparse attention in fp32 for gfx950: O = softmax(scale * Q K^T restricted to
// a mask of 64 x 64 blocks, optionally with per-block bit masks) V, fp32 operands, fp32
// probabilities, fp32 accumulation.
//
// This is the three-step pipeline SDDMM -> row softmax -> SpMM that the reference runs per head
// in fp32 (bench/bench_sparse_transformer.py:354-372) in one kernel and at the reference's own
// precision: the scores never reach memory.  The structure is that of the bf16 kernel in
// attn.hip (one workgroup = one head x one block row or one stretch of one, a wavefront = 16
// queries, S^T = K Q^T and O^T += V^T P^T so that an MFMA result is the next MFMA's operand
// without any exchange between lanes); what differs is the matrix instruction,
// v_mfma_f32_16x16x4_f32, which contracts four values per lane group at a sixteenth of the bf16
// rate, so the kernel is bound by the matrix cores and everything around them is kept simple:
// tiles go through registers into LDS rows padded by 16 bytes (no bank conflicts for either
// operand), one tile in LDS and the next in registers, the accumulators are rescaled whenever a
// query's running maximum rises.
//
// Lane (g, n) = (lane / 16, lane % 16).  An MFMA takes A[i = n][k = g] and B[k = g][j = n] and
// adds to C[4g .. 4g+3][n].  Which four values of the contraction index a group of four MFMAs
// takes is free as long as both operands agree: step c of slab j uses d = 16 j + 4 g + c, so a
// lane's operands for four steps are 16 contiguous bytes of a row of K (one ds_read_b128) and of
// its query's row of Q (kept in registers).
#include "common.hpp"

namespace scorch {
namespace attn32 {

constexpr int kBlock = 64;  // mask block edge: queries per workgroup, keys per step
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Combine a value over the four lanes that share a query (lanes n, n + 16, n + 32, n + 48).
template <typename Op>
__device__ __forceinline__ float combine_query_lanes(float x, Op op) {
  const unsigned bits = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  x = op(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
  const unsigned bits2 = __builtin_bit_cast(unsigned, x);
  auto q = __builtin_amdgcn_permlane32_swap(bits2, bits2, false, false);
  return op(__builtin_bit_cast(float, (unsigned)q[0]), __builtin_bit_cast(float, (unsigned)q[1]));
}

template <int D>
struct Tile {
  // A row of a tile takes D + 4 floats in LDS.  Readers of K (lane n reads 16 bytes of row
  // 16 t + n) then start 4 n banks apart, eight lanes cover the 32 banks; readers of V (lane
  // (g, n) reads one float of row 16 t + 4 g + r at column 16 dt + n) fall on bank
  // n + 16 g mod 32, two lanes per bank, which is what 64 lanes on 32 banks cost anyway.
  static constexpr int kStride = D + 4;
  static constexpr int kFloats = kBlock * kStride;
  static constexpr int kChunksPerRow = D / 4;  // 16-byte chunks
  static constexpr int kChunksPerThread = kBlock * kChunksPerRow / kBlockThreads;
};

constexpr float kDead = -3.0e38f;  // score of an entry the mask leaves out; also "no maximum yet"

template <int D>
__global__ __launch_bounds__(kBlockThreads)
__attribute__((amdgpu_waves_per_eu(D == 128 ? 2 : 4))) void attn_f32_kernel(
    int S, int n_blocks, int n_heads, const int *__restrict__ block_row_ptr,
    const int *__restrict__ block_col_idx, const int *__restrict__ block_mask_index,
    const unsigned long long *__restrict__ block_masks, const float *__restrict__ Q,
    const float *__restrict__ K, const float *__restrict__ V, float scale_log2e, float *__restrict__ O,
    int n_items, const int4 *__restrict__ items, int n_slots, float *__restrict__ partials) {
  using T = Tile<D>;
  constexpr int kStride = T::kStride;
  constexpr int kSlabs = D / 16;  // contraction slabs of the first product (four MFMA steps each)
  constexpr int kFeat = D / 16;   // 16-feature tiles of the second product
  constexpr int kCpt = T::kChunksPerThread;
  __shared__ __attribute__((aligned(16))) float s_k[T::kFloats];
  __shared__ __attribute__((aligned(16))) float s_v[T::kFloats];

  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int w = uniform(tid / kWaveSize);
  const int g = lane >> 4;
  const int n = lane & 15;
  int head, rank;
  {
    // all workgroups of a head on one XCD when the head count allows it (workgroup ids go round
    // the 8 XCDs): a head's K and V are then fetched into one L2 only
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
  // work item: a block row, or with `items` a stretch of one (x: block row, y and z: the stretch
  // within block_col_idx, w: where its partial result goes, -1 = it writes O itself)
  int qb, kb_begin, kb_end, part_slot = -1;
  if (items) {
    const int4 item = items[rank];
    qb = uniform(item.x);
    kb_begin = uniform(item.y);
    kb_end = uniform(item.z);
    part_slot = uniform(item.w);
  } else {
    qb = n_blocks - 1 - rank;
    kb_begin = block_row_ptr[qb];
    kb_end = block_row_ptr[qb + 1];
  }
  const size_t head_off = (size_t)head * (size_t)S * D;
  const float *Kh = K + head_off, *Vh = V + head_off;
  const int query = qb * kBlock + w * 16 + n;

  // The query's row, scaled once: scores then come out of the matrix cores in base-2 exponent
  // units (a negative or zero scale needs nothing special).
  floatx4 q_op[kSlabs];
#pragma unroll
  for (int j = 0; j < kSlabs; ++j) {
    q_op[j] = *reinterpret_cast<const floatx4 *>(Q + head_off + (size_t)query * D + 16 * j + 4 * g);
#pragma unroll
    for (int c = 0; c < 4; ++c) q_op[j][c] *= scale_log2e;
  }

  floatx4 o_acc[kFeat];
#pragma unroll
  for (int dt = 0; dt < kFeat; ++dt) o_acc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = kDead;
  float l_run = 0.0f;  // this lane's share of the row sum (its 16 keys of every block)

  // Tile traffic: thread `tid` moves chunks tid, tid + 256, ... (16 bytes each) of a 64 x D tile.
  floatx4 k_next[kCpt], v_next[kCpt];
  auto fetch_k = [&](int it) {
    const size_t tile = (size_t)uniform(block_col_idx[it]) * kBlock * D;
#pragma unroll
    for (int u = 0; u < kCpt; ++u)
      k_next[u] = *reinterpret_cast<const floatx4 *>(Kh + tile + (size_t)(tid + u * kBlockThreads) * 4);
  };
  auto fetch_v = [&](int it) {
    const size_t tile = (size_t)uniform(block_col_idx[it]) * kBlock * D;
#pragma unroll
    for (int u = 0; u < kCpt; ++u)
      v_next[u] = *reinterpret_cast<const floatx4 *>(Vh + tile + (size_t)(tid + u * kBlockThreads) * 4);
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int u = 0; u < kCpt; ++u) {
      const int chunk = tid + u * kBlockThreads;
      const int at = (chunk / T::kChunksPerRow) * kStride + (chunk % T::kChunksPerRow) * 4;
      *reinterpret_cast<floatx4 *>(&s_k[at]) = k_next[u];
      *reinterpret_cast<floatx4 *>(&s_v[at]) = v_next[u];
    }
  };
  const int my_query_in_block = w * 16 + n;

  if (kb_begin < kb_end) {
    fetch_k(kb_begin);
    fetch_v(kb_begin);
    store_tile();
  }
  __syncthreads();

  for (int it = kb_begin; it < kb_end; ++it) {
    const bool more = it + 1 < kb_end;
    if (more) fetch_k(it + 1);  // in flight while this block is computed (V follows after the scores:
                                // the two sets of staging registers are then not live at once with
                                // the K operands)

    // S^T = K Q^T: tile t holds keys 16 t + 4 g + r (r = 0 .. 3) against query n
    floatx4 st[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) st[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < kSlabs; ++j) {
      floatx4 k_op[4];
#pragma unroll
      for (int t = 0; t < 4; ++t)
        k_op[t] = *reinterpret_cast<const floatx4 *>(&s_k[(16 * t + n) * kStride + 16 * j + 4 * g]);
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int t = 0; t < 4; ++t)
          st[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(k_op[t][c], q_op[j][c], st[t], 0, 0, 0);
    }

    if (more) fetch_v(it + 1);

    // a block that is only partly live: bit j of word i of its mask says whether query i of the
    // block row attends to key j of the block
    unsigned long long live = ~0ull;
    bool partly_live = false;  // the same for the whole workgroup
    if (block_mask_index) {
      const int mask_at = uniform(block_mask_index[it]);
      if (mask_at >= 0) {
        partly_live = true;
        live = block_masks[(size_t)mask_at * kBlock + my_query_in_block] >> (4 * g);
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (!((live >> (16 * t + r)) & 1ull)) st[t][r] = kDead;
      }
    }

    // online softmax, base 2
    float mx = st[0][0];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, st[t][r]);
    mx = combine_query_lanes(mx, [](float a, float b) { return fmaxf(a, b); });
    if (__any(mx > m_run)) {  // some query's maximum rises: after a row's first key blocks, seldom
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // (no maximum yet: the sums are 0)
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < kFeat; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_acc[dt][r] *= alpha;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) st[t][r] = __builtin_amdgcn_exp2f(st[t][r] - m_run);
    if (partly_live) {
      // an entry the mask leaves out: exp2(kDead - m_run) is 0 already unless the query has had no
      // live key so far (m_run = kDead), so it is set
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (!((live >> (16 * t + r)) & 1ull)) st[t][r] = 0.0f;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) l_run += st[t][r];

    // O^T += V^T P^T: step (t, r) contracts keys 16 t + 4 g + r, whose probabilities lane (g, n)
    // holds for query n; the V^T operand is V[that key][16 dt + n]
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float *v_row = &s_v[(16 * t + 4 * g + r) * kStride + n];
#pragma unroll
        for (int dt = 0; dt < kFeat; ++dt)
          o_acc[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(v_row[16 * dt], st[t][r], o_acc[dt], 0, 0, 0);
      }

    __syncthreads();  // every wavefront is done with this tile
    if (more) store_tile();
    __syncthreads();
  }

  const float l = combine_query_lanes(l_run, [](float a, float b) { return a + b; });
  if (part_slot >= 0) {
    // a stretch of a block row: unnormalised sums, their reference maximum and the row sum
    float *part = partials + (((size_t)head * n_slots + part_slot) * kBlock + (w * 16 + n)) * (D + 4);
#pragma unroll
    for (int dt = 0; dt < kFeat; ++dt) *reinterpret_cast<floatx4 *>(part + 16 * dt + 4 * g) = o_acc[dt];
    if (g == 0) {
      part[D] = m_run;
      part[D + 1] = l;
    }
    return;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;  // queries without a live key give zeros
  float *out = O + head_off + (size_t)query * D;
#pragma unroll
  for (int dt = 0; dt < kFeat; ++dt) {
    floatx4 o = o_acc[dt];
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] *= inv;
    *reinterpret_cast<floatx4 *>(out + 16 * dt + 4 * g) = o;
  }
}

// Combines the stretches of a block row that was shared out: with m* the largest of the
// stretches' reference maxima, O = sum_p 2^(m_p - m*) O_p / sum_p 2^(m_p - m*) l_p.
// One workgroup per (split row, head); thread t takes query t / 4 and a quarter of the features.
template <int D>
__global__ __launch_bounds__(kBlockThreads) void attn_f32_merge_kernel(int S, int n_slots,
                                                                       const int4 *__restrict__ split_rows,
                                                                       const float *__restrict__ partials,
                                                                       float *__restrict__ O) {
  const int4 row = split_rows[blockIdx.x];  // x: block row, y: first slot, z: number of stretches
  const int head = blockIdx.y;
  const int q = threadIdx.x >> 2, quarter = threadIdx.x & 3;
  constexpr int kMine = D / 4;
  const float *base = partials + (((size_t)head * n_slots + row.y) * kBlock + q) * (D + 4);
  const size_t part_stride = (size_t)kBlock * (D + 4);
  float m_star = kDead;
  for (int p = 0; p < row.z; ++p) m_star = fmaxf(m_star, base[p * part_stride + D]);
  float acc[kMine];
#pragma unroll
  for (int j = 0; j < kMine; ++j) acc[j] = 0.0f;
  float l = 0.0f;
  for (int p = 0; p < row.z; ++p) {
    const float *part = base + p * part_stride;
    const float weight = __builtin_amdgcn_exp2f(part[D] - m_star);
    l += weight * part[D + 1];
#pragma unroll
    for (int j = 0; j < kMine; j += 4) {
      const floatx4 o = *reinterpret_cast<const floatx4 *>(part + quarter * kMine + j);
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[j + r] += weight * o[r];
    }
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;
  float *out = O + ((size_t)head * S + (size_t)row.x * kBlock + q) * D + quarter * kMine;
#pragma unroll
  for (int j = 0; j < kMine; j += 4) {
    floatx4 o;
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = acc[j + r] * inv;
    *reinterpret_cast<floatx4 *>(out + j) = o;
  }
}

template <int D>
static int launch(dim3 grid, hipStream_t s, int S, int n_blocks, int H, const int32_t *block_row_ptr,
                  const int32_t *block_col_idx, const int32_t *block_mask_index,
                  const unsigned long long *block_masks, const float *q, const float *k, const float *v,
                  float scale_log2e, float *o, int n_items, const int4 *items, int n_slots, float *partials,
                  int n_split_rows, const int4 *split_rows) {
  mark_launch(s);
  attn_f32_kernel<D><<<grid, kBlockThreads, 0, s>>>(S, n_blocks, H, block_row_ptr, block_col_idx, block_mask_index,
                                                    block_masks, q, k, v, scale_log2e, o, n_items, items, n_slots,
                                                    partials);
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(s);
  if (n_split_rows > 0) {
    attn_f32_merge_kernel<D><<<dim3((unsigned)n_split_rows, (unsigned)H), kBlockThreads, 0, s>>>(S, n_slots, split_rows,
                                                                                               partials, o);
    SCORCH_HIP_CHECK(hipGetLastError());
    mark_launch(s);
  }
  return SCORCH_HIP_OK;
}

}  // namespace attn32
}  // namespace scorch

extern "C" size_t scorch_hip_attn_blocksparse_f32_workspace_bytes(int64_t H, int64_t n_slots, int64_t D) {
  if (H <= 0 || n_slots <= 0 || D <= 0) return 0;
  return (size_t)H * (size_t)n_slots * scorch::attn32::kBlock * (size_t)(D + 4) * sizeof(float);
}

extern "C" int scorch_hip_attn_blocksparse_f32(
    int64_t H, int64_t S, int64_t D, int64_t block, int64_t n_active_blocks, const int32_t *block_row_ptr,
    const int32_t *block_col_idx, const int32_t *block_mask_index, int64_t n_masks, const uint64_t *block_masks,
    int64_t n_items, const int32_t *items, int64_t n_split_rows, const int32_t *split_rows, int64_t n_slots,
    const float *Q, const float *K, const float *V, float scale, float *O, void *workspace, size_t workspace_bytes,
    void *stream) {
  using namespace scorch;
  const char *fn = "scorch_hip_attn_blocksparse_f32";
  if (H < 0 || S < 0 || D < 0 || block <= 0 || n_active_blocks < 0 || n_masks < 0 || n_items < 0 ||
      n_split_rows < 0 || n_slots < 0)
    return fail(SCORCH_HIP_EINVAL, "%s: negative size (H=%lld S=%lld D=%lld block=%lld)", fn, (long long)H,
                (long long)S, (long long)D, (long long)block);
  if ((D != 32 && D != 64 && D != 128) || block != attn32::kBlock)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: only head dimensions 32, 64 and 128 and %d x %d mask blocks are "
                "built (got D=%lld block=%lld)", fn, attn32::kBlock, attn32::kBlock, (long long)D, (long long)block);
  if (S % attn32::kBlock != 0)
    return fail(SCORCH_HIP_EINVAL, "%s: S=%lld is not a multiple of the block size", fn, (long long)S);
  if (H * (S / attn32::kBlock) > INT32_MAX || S * D > INT32_MAX || n_items * H > INT32_MAX || n_slots > INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: H=%lld, S=%lld or the item count too large", fn, (long long)H,
                (long long)S);
  if (H == 0 || S == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(n_items > 0 || block_row_ptr != nullptr, "%s: block_row_ptr is NULL", fn);
  SCORCH_REQUIRE(n_active_blocks == 0 || block_col_idx != nullptr, "%s: block_col_idx is NULL", fn);
  SCORCH_REQUIRE(Q && K && V && O, "%s: NULL Q/K/V/O", fn);
  SCORCH_REQUIRE(aligned_to(Q, 16) && aligned_to(K, 16) && aligned_to(V, 16) && aligned_to(O, 16),
                 "%s: Q, K, V and O must be 16-byte aligned", fn);
  if (block_mask_index) {
    SCORCH_REQUIRE(n_masks == 0 || block_masks != nullptr, "%s: block_masks is NULL", fn);
    SCORCH_REQUIRE(aligned_to(block_masks, 8), "%s: block_masks must be 8-byte aligned", fn);
  }
  const int n_blocks = (int)(S / attn32::kBlock);
  int work = n_blocks;
  const int4 *item_list = nullptr, *rows = nullptr;
  float *partials = nullptr;
  if (n_items > 0) {
    SCORCH_REQUIRE(items != nullptr && aligned_to(items, 16), "%s: items must be 16-byte aligned", fn);
    SCORCH_REQUIRE(n_split_rows == 0 || (split_rows != nullptr && aligned_to(split_rows, 16)),
                   "%s: split_rows must be 16-byte aligned", fn);
    const size_t need = scorch_hip_attn_blocksparse_f32_workspace_bytes(H, n_slots, D);
    if (need > 0 && (!workspace || workspace_bytes < need || !aligned_to(workspace, 256)))
      return fail(SCORCH_HIP_EWORKSPACE, "%s: a 256-byte aligned workspace of %zu bytes is needed, %zu given", fn,
                  need, workspace ? workspace_bytes : (size_t)0);
    work = (int)n_items;
    item_list = reinterpret_cast<const int4 *>(items);
    rows = reinterpret_cast<const int4 *>(split_rows);
    partials = static_cast<float *>(workspace);
  } else if (n_split_rows > 0 || n_slots > 0) {
    return fail(SCORCH_HIP_EINVAL, "%s: split rows without items", fn);
  }
  const dim3 grid((unsigned)((int64_t)work * H));
  const float scale_log2e = scale * 1.4426950408889634f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned long long *masks = reinterpret_cast<const unsigned long long *>(block_masks);
#define SCORCH_ATTN32(DIM)                                                                                     \
  return attn32::launch<DIM>(grid, s, (int)S, n_blocks, (int)H, block_row_ptr, block_col_idx, block_mask_index, \
                             masks, Q, K, V, scale_log2e, O, work, item_list, (int)n_slots, partials,          \
                             (int)n_split_rows, rows)
  if (D == 32) SCORCH_ATTN32(32);
  if (D == 64) SCORCH_ATTN32(64);
  SCORCH_ATTN32(128);
#undef SCORCH_ATTN32
}

SCORCH_DEFINE_PRELOAD(attn_f32)
