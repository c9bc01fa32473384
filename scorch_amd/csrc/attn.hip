// Fused block-sparse attention for gfx950: O = softmax(scale * Q K^T restricted
// to a block mask) V, bf16 operands, fp32 accumulation, one pass over the mask.
//
// It replaces, for a mask made of 64 x 64 blocks, the three-step pipeline
// SDDMM -> row softmax -> SpMM that the reference runs per head
// (bench/bench_sparse_transformer.py:354-372): the scores are never written to
// memory.  The contraction inside a block is dense, so it runs on the matrix
// cores (v_mfma_f32_16x16x32_bf16).
//
// Work split.  One workgroup (4 wavefronts) owns one head and one block row of
// the mask, i.e. 64 queries; each wavefront owns 16 of them.  The workgroup
// walks the block row's active key blocks.  For each, the 64 x 64 K tile and
// the 64 x 64 V tile are staged in LDS once for all four wavefronts, both
// row-major; the next tile's global loads are in flight while the current one
// is consumed (two LDS buffers, one barrier per key block).  The second
// product needs V by columns (eight keys of one feature per lane): that
// operand is read with ds_read_b64_tr_b16, which hands each lane of a 16-lane
// group one column of a 4 x 16 block whose rows the group's lanes address.
//
// Per wavefront and key block, everything stays in registers:
//   S^T = K Q^T        (keys x queries: 4 tiles of 16 keys, contraction over D)
//   online softmax     (running max / sum per query, base-2 exponent)
//   O^T += V^T P^T     (features x queries: 4 tiles of 16 features, contraction over keys)
// Working with the transposes makes the layouts chain without any shuffle: an
// MFMA result tile holds, in lane (g, n) (g = lane / 16, n = lane % 16), rows
// 4g .. 4g+3 of column n.  Column n is query n throughout, so each lane owns
// the softmax state of its query; the 16 probabilities it holds after the
// first product (4 tiles x 4 keys) are exactly the B operand of the second
// one, provided the V^T operand is gathered with the same key order.
#include "common.hpp"

namespace scorch {

constexpr int kAttnBlock = 64;  // mask block edge: queries per workgroup, keys per step
constexpr int kAttnDim = 64;    // head dimension
constexpr int kLdsRow = 72;     // LDS row length in bf16 (64 + 8 padding against bank conflicts)

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef short4v __attribute__((address_space(3))) lds_short4v;

// Combine a value over the four lanes that share a query (lanes n, n + 16,
// n + 32, n + 48) with the row-swap instructions of gfx950: they stay in the
// vector ALU, where a shuffle through LDS (ds_bpermute) would put two LDS round
// trips into the middle of every key block's dependent chain.
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the
// even rows of its second, v_permlane32_swap the upper half of the first with the
// lower half of the second; fed the same value twice, the two results hold, in
// every lane, the value of the lane and of its partner.
template <typename Op>
__device__ __forceinline__ float combine_query_lanes(float x, Op op) {
  const unsigned bits = __builtin_bit_cast(unsigned, x);
  auto r = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  x = op(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
  const unsigned bits2 = __builtin_bit_cast(unsigned, x);
  auto q = __builtin_amdgcn_permlane32_swap(bits2, bits2, false, false);
  return op(__builtin_bit_cast(float, (unsigned)q[0]), __builtin_bit_cast(float, (unsigned)q[1]));
}

template <bool NEGATIVE_SCALE>
__global__ __launch_bounds__(kBlockThreads) void attn_blocksparse_kernel(
    int S, int n_blocks, int n_heads, const int *__restrict__ block_row_ptr,
    const int *__restrict__ block_col_idx, const __bf16 *__restrict__ Q,
    const __bf16 *__restrict__ K, const __bf16 *__restrict__ V, float scale_log2e,
    __bf16 *__restrict__ O) {
  __shared__ __attribute__((aligned(16))) __bf16 s_k[2][kAttnBlock][kLdsRow];   // [key][feature]
  __shared__ __attribute__((aligned(16))) __bf16 s_v[2][kAttnBlock][kLdsRow];   // [key][feature]

  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int w = tid / kWaveSize;
  const int g = lane >> 4;  // 16-lane group: which keys / features of a tile this lane holds
  const int n = lane & 15;  // query within the wavefront's 16
  // Workgroup -> (head, block row).  Workgroups are dealt to the 8 XCDs round
  // robin by their linear id, and every XCD has its own 4 MB L2.  When the head
  // count allows it, all workgroups of a head are given ids of one residue mod
  // 8, so that a head's K and V (2 * S * 128 bytes) are fetched into one L2 only
  // and an XCD works through its heads one after the other.
  int head, rank;
  {
    const int id = blockIdx.x;
    if (n_heads % 8 == 0) {
      const int xcd = id & 7, slot = id >> 3;
      head = xcd + 8 * (slot / n_blocks);
      rank = slot % n_blocks;
    } else {
      head = id / n_blocks;
      rank = id % n_blocks;
    }
  }
  const int qb = n_blocks - 1 - rank;  // longest block rows first
  const size_t head_off = (size_t)head * (size_t)S * kAttnDim;
  const __bf16 *Qh = Q + head_off, *Kh = K + head_off, *Vh = V + head_off;

  // B operand of S^T = K Q^T: this lane's query row, features 8g + 32s .. + 7.
  const int query = qb * kAttnBlock + w * 16 + n;
  bf16x8 q_op[2];
#pragma unroll
  for (int s = 0; s < 2; ++s)
    q_op[s] = *reinterpret_cast<const bf16x8 *>(Qh + (size_t)query * kAttnDim + 8 * g + 32 * s);

  floatx4 o_acc[4];  // O^T tiles: o_acc[dt][r] = O[query][16 dt + 4g + r]
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) o_acc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -3.0e38f;  // running maximum of scale * log2(e) * score, equal in the 4 lanes of a query
  // Running sum of the (bf16-rounded) probabilities of query n, kept by the matrix
  // core: a row of ones appended to V^T makes the second product add up P as
  // well.  Matrix and vector instructions do not overlap on this chip, so two
  // more matrix instructions (32 cycles) are cheaper than the sixteen additions
  // (64 cycles) they replace.  Every element of l_acc holds the same value.
  floatx4 l_acc = floatx4{0.f, 0.f, 0.f, 0.f};
  bf16x8 ones;
#pragma unroll
  for (int j = 0; j < 8; ++j) ones[j] = (__bf16)1.0f;

  const int kb_begin = block_row_ptr[qb];
  const int kb_end = block_row_ptr[qb + 1];

  // Staging: a thread handles two 16-byte pieces of each tile; piece c covers
  // row c / 8 (a key), features 8 (c % 8) .. + 7.  Tiles alternate between two
  // register sets and two LDS buffers by parity: while tile `it` is consumed
  // from LDS, tile it + 1 waits in registers and tile it + 2 is being fetched,
  // so a fetch has a whole key block of work to hide behind.
  bf16x8 k_stage[2][2], v_stage[2][2];
  auto load_tile = [&](auto set_tag, int it) {
    constexpr int kSet = decltype(set_tag)::value;
    // tile base: the same for every thread (scalar arithmetic); piece offset: fixed per thread
    const size_t tile = (size_t)uniform(block_col_idx[it]) * (kAttnBlock * kAttnDim);
    const __bf16 *k_tile = Kh + tile, *v_tile = Vh + tile;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int piece = (tid + u * kBlockThreads) * 8;  // tiles are contiguous: piece c starts at element 8 c
      k_stage[kSet][u] = *reinterpret_cast<const bf16x8 *>(k_tile + piece);
      v_stage[kSet][u] = *reinterpret_cast<const bf16x8 *>(v_tile + piece);
    }
  };
  auto store_tile = [&](auto set_tag) {  // register set p -> LDS buffer p
    constexpr int kSet = decltype(set_tag)::value;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = tid + u * kBlockThreads;
      const int key = c >> 3, f0 = (c & 7) * 8;
      *reinterpret_cast<bf16x8 *>(&s_k[kSet][key][f0]) = k_stage[kSet][u];
      *reinterpret_cast<bf16x8 *>(&s_v[kSet][key][f0]) = v_stage[kSet][u];
    }
  };
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;

  if (kb_begin < kb_end) {
    load_tile(Even{}, kb_begin);
    store_tile(Even{});
    if (kb_begin + 1 < kb_end) load_tile(Odd{}, kb_begin + 1);
  }
  __syncthreads();

  // One key block: tile `it` has parity P = decltype(tag)::value.
  auto key_block = [&](auto tag, int it) {
    constexpr int buf = decltype(tag)::value;
    using Other = std::integral_constant<int, buf ^ 1>;
    if (it + 2 < kb_end) load_tile(tag, it + 2);  // this parity's registers are free again

    // S^T tile t: keys 16t .. 16t+15 (rows) x 16 queries (columns).
    floatx4 st[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const bf16x8 k_lo = *reinterpret_cast<const bf16x8 *>(&s_k[buf][16 * t + n][8 * g]);
      const bf16x8 k_hi = *reinterpret_cast<const bf16x8 *>(&s_k[buf][16 * t + n][8 * g + 32]);
      st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_lo, q_op[0], floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
      st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_hi, q_op[1], st[t], 0, 0, 0);
    }

    // Online softmax for query n, in base 2: this lane holds keys 16t + 4g + r.
    // With scale > 0 the maximum of the scaled scores is the scaled maximum.
    float mx = st[0][0];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = NEGATIVE_SCALE ? fminf(mx, st[t][r]) : fmaxf(mx, st[t][r]);
    mx *= scale_log2e;
    mx = combine_query_lanes(mx, [](float a, float b) { return fmaxf(a, b); });
    const float m_new = fmaxf(m_run, mx);
    // Rescale what has been accumulated only when some query's maximum moved
    // (after the first few key blocks it rarely does).
    if (__any(m_new > m_run)) {
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      l_acc[0] *= alpha;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_acc[dt][r] *= alpha;
    }
    m_run = m_new;

    // P^T as the B operand of the second product: slot j of step s is key
    // 32s + 16 (j / 4) + 4g + (j % 4).
    bf16x8 p_op[2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[t][r], scale_log2e, -m_new));
        p_op[t >> 1][(t & 1) * 4 + r] = (__bf16)p;
      }

    // O^T tile dt: features 16dt .. 16dt+15 (rows) x 16 queries, contraction over
    // the 64 keys.  A operand: lane (g, n) needs V[key][16dt + n] for the eight
    // keys of its slots.  One transposing read covers four consecutive keys:
    // lane i of the group addresses row key0 + i / 4, features 16dt + 4 (i % 4) .. + 3,
    // and receives V[key0 .. key0 + 3][16dt + i].
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int key0 = 32 * s + 4 * g + (n >> 2);
        const int f0 = 16 * dt + 4 * (n & 3);
        const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4v *)&s_v[buf][key0][f0]);
        const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4v *)&s_v[buf][key0 + 16][f0]);
        const short8v packed = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        const bf16x8 v_op = __builtin_bit_cast(bf16x8, packed);
        o_acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_op, p_op[s], o_acc[dt], 0, 0, 0);
      }
#pragma unroll
    for (int s = 0; s < 2; ++s) l_acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, p_op[s], l_acc, 0, 0, 0);

    if (it + 1 < kb_end) store_tile(Other{});
    __syncthreads();
  };

  for (int it = kb_begin; it < kb_end; it += 2) {
    key_block(Even{}, it);
    if (it + 1 < kb_end) key_block(Odd{}, it + 1);
  }

  // Normalise and store O[query][16dt + 4g .. + 3] (8 bytes per tile and lane).
  const float l = l_acc[0];
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;  // block rows without key blocks give zeros
  __bf16 *out = O + head_off + (size_t)query * kAttnDim;
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) {
    bf16x4 o;
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = (__bf16)(o_acc[dt][r] * inv);
    *reinterpret_cast<bf16x4 *>(out + 16 * dt + 4 * g) = o;
  }
}

}  // namespace scorch

extern "C" int scorch_hip_attn_blocksparse_bf16(int64_t H, int64_t S, int64_t D, int64_t block,
                                                int64_t n_active_blocks,
                                                const int32_t *block_row_ptr,
                                                const int32_t *block_col_idx, const void *Q,
                                                const void *K, const void *V, float scale, void *O,
                                                void *stream) {
  using namespace scorch;
  const char *fn = "scorch_hip_attn_blocksparse_bf16";
  if (H < 0 || S < 0 || D < 0 || block <= 0 || n_active_blocks < 0)
    return fail(SCORCH_HIP_EINVAL, "%s: negative size (H=%lld S=%lld D=%lld block=%lld)", fn,
                (long long)H, (long long)S, (long long)D, (long long)block);
  if (D != kAttnDim || block != kAttnBlock)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: only head dimension %d and %d x %d mask blocks are built "
                "(got D=%lld block=%lld)", fn, kAttnDim, kAttnBlock, kAttnBlock, (long long)D,
                (long long)block);
  if (S % kAttnBlock != 0)
    return fail(SCORCH_HIP_EINVAL, "%s: S=%lld is not a multiple of the block size", fn, (long long)S);
  if (H * (S / kAttnBlock) > INT32_MAX || S * D > INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: H=%lld or S=%lld too large", fn, (long long)H, (long long)S);
  SCORCH_REQUIRE(block_row_ptr != nullptr, "%s: block_row_ptr is NULL", fn);
  if (H == 0 || S == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(n_active_blocks == 0 || block_col_idx != nullptr, "%s: block_col_idx is NULL", fn);
  SCORCH_REQUIRE(Q && K && V && O, "%s: NULL Q/K/V/O", fn);
  SCORCH_REQUIRE(aligned_to(Q, 16) && aligned_to(K, 16) && aligned_to(V, 16) && aligned_to(O, 16),
                 "%s: Q, K, V and O must be 16-byte aligned", fn);
  const int n_blocks = (int)(S / kAttnBlock);
  const dim3 grid((unsigned)(n_blocks * H));
  const float scale_log2e = scale * 1.4426950408889634f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const __bf16 *q = static_cast<const __bf16 *>(Q), *k = static_cast<const __bf16 *>(K),
               *v = static_cast<const __bf16 *>(V);
  if (scale < 0.0f)
    attn_blocksparse_kernel<true><<<grid, kBlockThreads, 0, s>>>(
        (int)S, n_blocks, (int)H, block_row_ptr, block_col_idx, q, k, v, scale_log2e,
        static_cast<__bf16 *>(O));
  else
    attn_blocksparse_kernel<false><<<grid, kBlockThreads, 0, s>>>(
        (int)S, n_blocks, (int)H, block_row_ptr, block_col_idx, q, k, v, scale_log2e,
        static_cast<__bf16 *>(O));
  SCORCH_HIP_CHECK(hipGetLastError());
  return SCORCH_HIP_OK;
}
