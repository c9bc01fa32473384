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
// the 64 x 64 V tile are put in LDS once for all four wavefronts, both
// row-major; the next tile's loads are in flight while the current one is
// consumed (two LDS buffers, one barrier per key block).  The second
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
constexpr float kRescaleSlack = 8.0f;  // see the online softmax in the kernel

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

// One 16-byte-per-lane load from a buffer straight into LDS: the address is the buffer's base
// (scalar) + a scalar byte offset + the lane's byte offset, the LDS target a scalar base + 16 x
// lane.  (The buffer descriptor is built here, inside a device function: its type does not exist
// in the host pass, which still has to instantiate the kernel templates' launch stubs.)
__device__ __forceinline__ void load_to_lds_16(const void *buffer, int buffer_bytes, unsigned lane_offset,
                                               int scalar_offset, __attribute__((address_space(3))) void *lds) {
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(buffer), 0, buffer_bytes, 0x00020000);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, lds, 16, lane_offset, scalar_offset, 0, 0);
}

// K and V tiles are written to LDS by the load itself (buffer_load_dwordx4 ... lds):
// no staging registers, no LDS store instructions; at D = 64, with 127 VGPRs and
// 32 KB of LDS per workgroup, four workgroups share a CU.  Such a load puts lane L's 16
// bytes at (wave-uniform base) + 16 L, so a wavefront instruction fills eight
// whole 128-byte rows and rows cannot be padded against bank conflicts.  Instead
// the 16-byte chunks of a row are permuted: chunk c of row r lies at position
// c ^ (r & 7).  The permutation is applied on the way in (each lane fetches the
// chunk that belongs at its LDS position) and undone by the readers' address
// arithmetic.  (Staging through registers with padded rows measured 12 % slower.)
//
// Head dimension D is 32, 64 or 128: a tile row is RB = 2 D bytes, i.e. CPR = D / 8 chunks of 16
// bytes, a tile 64 RB bytes.  The permutation is chunk c of row r at position c ^ swizzle(r) with
// swizzle(r) = r & 7 (for D = 32, where a row has only four chunks, (r >> 1) & 3): what matters
// is that the eight lanes the LDS serves together, which read the same chunk of eight
// consecutive rows, fall into eight different 16-byte bank groups.
template <int D>
struct AttnTile {
  static constexpr int kRowBytes = 2 * D;
  static constexpr int kChunksPerRow = D / 8;
  static constexpr int kBytes = kAttnBlock * kRowBytes;
  static constexpr int kRowsPerLoad = 1024 / kRowBytes;     // rows one wavefront load instruction fills
  static constexpr int kLoadsPerWave = 16 / kRowsPerLoad;   // a wavefront fills 16 rows of a tile
  __device__ static __forceinline__ int swizzle(int row) { return D == 32 ? (row >> 1) & 3 : row & 7; }
  // Wavefronts per SIMD the kernel is compiled for: the register budget is 512 / this.
  static constexpr int kWavesPerSimd = D == 128 ? 2 : 4;
};

template <int D, bool NEGATIVE_SCALE, bool MASKED>
__global__ __launch_bounds__(kBlockThreads)
__attribute__((amdgpu_waves_per_eu(AttnTile<D>::kWavesPerSimd))) void attn_blocksparse_kernel(
    int S, int n_blocks, int n_heads, const int *__restrict__ block_row_ptr,
    const int *__restrict__ block_col_idx, const int *__restrict__ block_mask_index,
    const unsigned long long *__restrict__ block_masks, const __bf16 *__restrict__ Q,
    const __bf16 *__restrict__ K, const __bf16 *__restrict__ V, float scale_log2e,
    __bf16 *__restrict__ O, int n_items, const int4 *__restrict__ items, int n_slots,
    float *__restrict__ partials, int pairs, int prio_step) {
  using Tile = AttnTile<D>;
  constexpr int kTileBytes = Tile::kBytes;
  constexpr int kRowBytes = Tile::kRowBytes;
  constexpr int kSteps = D / 32;   // MFMA steps of the first product (contraction over D)
  constexpr int kFeat = D / 16;    // 16-feature tiles of the second product
  // Two buffers each for K and V, as four separate arrays: the compiler then sees that the
  // loads which fill one buffer (they write LDS asynchronously) cannot touch the buffer being
  // read, and does not make the reads wait for them.  (As halves of one array, every second key
  // block waited for its own prefetch before its first LDS read.)
  __shared__ __attribute__((aligned(1024))) unsigned char s_k0[kTileBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_k1[kTileBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_v0[kTileBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char s_v1[kTileBytes];

  const int tid = threadIdx.x;
  const int lane = tid & (kWaveSize - 1);
  const int w = uniform(tid / kWaveSize);  // a scalar: the LDS targets of the tile loads are then scalar too
  const int g = lane >> 4;
  const int n = lane & 15;
  int head, rank;
  {
    // Workgroups are dealt to the 8 XCDs round robin by their linear id, and every
    // XCD has its own 4 MB L2.  When the head count allows it, all workgroups of a
    // head are given ids of one residue mod 8, so that a head's K and V
    // (2 * S * 128 bytes) are fetched into one L2 only and an XCD works through its
    // heads one after the other.
    const int id = blockIdx.x;
    const int n_ranks = pairs ? (n_items + 1) >> 1 : n_items;
    if (n_heads % 8 == 0) {
      const int xcd = id & 7, slot = id >> 3;
      head = xcd + 8 * (slot / n_ranks);
      rank = slot % n_ranks;
    } else {
      head = id / n_ranks;
      rank = id % n_ranks;
    }
  }
  // pairs: a workgroup takes two items, the rank-th longest and the rank-th shortest, one after
  // the other, so that all workgroups carry about the same work and fit the chip in one round
  for (int pass = 0; pass < (pairs ? 2 : 1); ++pass) {
  const int item_rank = pass == 0 ? rank : n_items - 1 - rank;
  if (pass == 1 && item_rank <= rank) break;
  // A workgroup's work item is a block row, or -- when `items` is given -- a stretch of a block
  // row's key blocks (x: block row, y and z: the stretch within block_col_idx, w: where its
  // partial result goes, or -1 for a whole row that writes O itself).  Items come longest first.
  int qb, kb_begin, kb_end, part_slot = -1;
  if (items) {
    const int4 item = items[item_rank];
    qb = uniform(item.x);
    kb_begin = uniform(item.y);
    kb_end = uniform(item.z);
    part_slot = uniform(item.w);
  } else {
    qb = n_blocks - 1 - item_rank;  // (masks with longer block rows further down: longest first)
    kb_begin = block_row_ptr[qb];
    kb_end = block_row_ptr[qb + 1];
  }
  // prio_step > 0: a wavefront's priority on its SIMD follows what its workgroup has left to do
  // (this item's remaining key blocks and, in the first pass of a pair, the second item's), in four
  // levels of prio_step blocks.  The wavefronts that were dispatched first win the SIMD's
  // arbitration otherwise: of the four workgroups of a CU two then finish a quarter of the launch
  // ahead of the other two, and the CU runs half empty from there on.
  int later_blocks = 0;
  if (prio_step > 0 && pairs && pass == 0 && n_items - 1 - rank > rank) {
    const int second = uniform(n_items - 1 - rank);
    if (items) {
      const int *words = reinterpret_cast<const int *>(items) + 4 * (size_t)second;  // (scalar loads)
      later_blocks = words[2] - words[1];
    } else {
      const int qb2 = n_blocks - 1 - second;
      later_blocks = block_row_ptr[qb2 + 1] - block_row_ptr[qb2];
    }
  }
  const size_t head_off = (size_t)head * (size_t)S * D;
  const __bf16 *Qh = Q + head_off;
  const unsigned char *Kb = reinterpret_cast<const unsigned char *>(K + head_off);
  const unsigned char *Vb = reinterpret_cast<const unsigned char *>(V + head_off);

  const int query = qb * kAttnBlock + w * 16 + n;
  bf16x8 q_op[kSteps];
#pragma unroll
  for (int s = 0; s < kSteps; ++s)
    q_op[s] = *reinterpret_cast<const bf16x8 *>(Qh + (size_t)query * D + 8 * g + 32 * s);

  floatx4 o_acc[kFeat];
#pragma unroll
  for (int dt = 0; dt < kFeat; ++dt) o_acc[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m_run = -3.0e38f;
  // (scale 0: every score counts as 0, nothing ever needs rescaling beyond the first block)
  const float inv_scale_log2e = scale_log2e != 0.0f ? 1.0f / scale_log2e : 0.0f;
  float raise_at = NEGATIVE_SCALE ? 3.0e38f : -3.0e38f;  // the first key block always sets m_run
  floatx4 l_acc = floatx4{0.f, 0.f, 0.f, 0.f};  // row sums of P, taken by the matrix core (ones row)
  bf16x8 ones;
#pragma unroll
  for (int j = 0; j < 8; ++j) ones[j] = (__bf16)1.0f;



  // Loading: wavefront w fills rows 16w .. 16w + 15 of a tile with kLoadsPerWave instructions of
  // kRowsPerLoad rows each.  Lane L of instruction u lands at row 16w + u kRowsPerLoad + L / CPR,
  // position L % CPR, which holds chunk (L % CPR) ^ swizzle(row).
  // The loads go through buffer descriptors of the head's K and V: the tile's byte offset is the
  // instruction's scalar offset, the lane's place in the tile its vector offset, the LDS target
  // comes from M0 -- a tile request costs no vector instructions at all.
  unsigned src_in_tile[Tile::kLoadsPerWave];
#pragma unroll
  for (int u = 0; u < Tile::kLoadsPerWave; ++u) {
    const int row = 16 * w + u * Tile::kRowsPerLoad + lane / Tile::kChunksPerRow;
    src_in_tile[u] = (unsigned)(row * kRowBytes + (((lane % Tile::kChunksPerRow) ^ Tile::swizzle(row)) * 16));
  }
  const int head_bytes = (int)(unsigned)((size_t)S * D * 2);  // (the host has checked that it fits 32 bits)
  auto load_tile = [&](auto buf_tag, int it) {
    constexpr int kBuf = decltype(buf_tag)::value;
    unsigned char *k_dst = kBuf ? s_k1 : s_k0;
    unsigned char *v_dst = kBuf ? s_v1 : s_v0;
    const int tile = (int)((unsigned)uniform(block_col_idx[it]) * (unsigned)kTileBytes);
#pragma unroll
    for (int u = 0; u < Tile::kLoadsPerWave; ++u) {
      load_to_lds_16(Kb, head_bytes, src_in_tile[u], tile,
                     (__attribute__((address_space(3))) void *)(&k_dst[(16 * w + u * Tile::kRowsPerLoad) * kRowBytes]));
      load_to_lds_16(Vb, head_bytes, src_in_tile[u], tile,
                     (__attribute__((address_space(3))) void *)(&v_dst[(16 * w + u * Tile::kRowsPerLoad) * kRowBytes]));
    }
  };
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;

  // Readers' offsets inside a tile.  K: row 16t + n, chunk 4s + g for contraction step s (its
  // swizzle depends on n only).  V^T: row 32s + 16h + 4g + n / 4, 8 bytes at feature
  // 16dt + 4 (n % 4), i.e. chunk 2dt + (n % 4) / 2, half (n % 4) % 2 (swizzle: on 4g + n / 4).
  const int k_swz = Tile::swizzle(n);
  const int k_row = n * kRowBytes;
  const int v_row = 4 * g + (n >> 2);
  const int v_swz = Tile::swizzle(v_row);
  const int v_off = v_row * kRowBytes + (n & 1) * 8;
  const int v_chunk = (n & 3) >> 1;
  const int my_query_in_block = w * 16 + n;

  if (kb_begin < kb_end) load_tile(Even{}, kb_begin);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  auto key_block = [&](auto tag, int it) {
    constexpr int buf = decltype(tag)::value;
    using Other = std::integral_constant<int, buf ^ 1>;
    const unsigned char *k_src = buf ? s_k1 : s_k0;
    const unsigned char *v_src = buf ? s_v1 : s_v0;
    if (it + 1 < kb_end) load_tile(Other{}, it + 1);  // its last readers passed the previous barrier

    floatx4 st[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      st[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < kSteps; ++s) {
        const bf16x8 k_op = *reinterpret_cast<const bf16x8 *>(
            &k_src[16 * kRowBytes * t + k_row + (((4 * s + g) ^ k_swz) * 16)]);
        st[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_op, q_op[s], st[t], 0, 0, 0);
      }
    }

    // The V^T operands of the second product are requested now, all of them, so that they arrive
    // while the vector ALU does the softmax; requested one by one just before their MFMAs, every
    // MFMA of the second product waits an LDS round trip.  (The masked kernel at D = 64 has no
    // registers left for that and requests them after the softmax.)
    constexpr bool kEarlyV = !(MASKED && D == 64);
    bf16x8 v_ops[kFeat][2];
    auto request_v_operands = [&]() {
#pragma unroll
      for (int dt = 0; dt < kFeat; ++dt)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const int at = 32 * kRowBytes * s + v_off + (((2 * dt + v_chunk) ^ v_swz) * 16);
          const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v *)&v_src[at]);
          const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v *)&v_src[at + 16 * kRowBytes]);
          const short8v packed = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          v_ops[dt][s] = __builtin_bit_cast(bf16x8, packed);
        }
    };
    if constexpr (kEarlyV) request_v_operands();
    __builtin_amdgcn_sched_barrier(0);  // (the scheduler would move the reads back down to their uses)

    // A block that is only partly live brings a 64 x 64 bit mask: bit j of word i says whether
    // query i of the block row attends to key j of the block.  A lane holds the scores of its
    // query against keys 16t + 4g + r (bit 16t + r of the word shifted down by 4g); dead ones are
    // kept out of the maximum here and get probability zero below.
    int mask_at = -1;
    unsigned long long live = ~0ull;
    if constexpr (MASKED) {
      mask_at = uniform(block_mask_index[it]);
      if (mask_at >= 0) {
        live = block_masks[(size_t)mask_at * kAttnBlock + my_query_in_block] >> (4 * g);
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (!((live >> (16 * t + r)) & 1ull)) st[t][r] = NEGATIVE_SCALE ? 3.0e38f : -3.0e38f;
      }
    }

    float mx = st[0][0];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = NEGATIVE_SCALE ? fminf(mx, st[t][r]) : fmaxf(mx, st[t][r]);
    // The running maximum only has to keep the exponentials in range, so it is raised (and the
    // accumulators rescaled) only when a score exceeds it by more than kRescaleSlack in the
    // base-2 exponent: probabilities then reach 2^kRescaleSlack at most, which fp32 sums and bf16
    // operands hold with the same relative precision, and the final division by the row sum
    // cancels the common factor.  Whether that is the case is decided on each lane's own 16 raw
    // scores against `raise_at` = (m_run + kRescaleSlack) / scale: a query's four lanes share its
    // m_run, so one of them sees any score that matters, and the exchange between lanes that the
    // true maximum needs is paid only when the branch is taken -- after a row's first key blocks
    // hardly ever.
    if (__any(NEGATIVE_SCALE ? mx < raise_at : mx > raise_at)) {
      mx = combine_query_lanes(mx * scale_log2e, [](float a, float b) { return fmaxf(a, b); });
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      l_acc[0] *= alpha;
#pragma unroll
      for (int dt = 0; dt < kFeat; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_acc[dt][r] *= alpha;
      m_run = m_new;
      raise_at = (m_run + kRescaleSlack) * inv_scale_log2e;
    }

    bf16x8 p_op[2];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[t][r], scale_log2e, -m_run));
        if constexpr (MASKED) {
          if (!((live >> (16 * t + r)) & 1ull)) p = 0.0f;
        }
        p_op[t >> 1][(t & 1) * 4 + r] = (__bf16)p;
      }

    if constexpr (!kEarlyV) request_v_operands();
#pragma unroll
    for (int dt = 0; dt < kFeat; ++dt)
#pragma unroll
      for (int s = 0; s < 2; ++s)
        o_acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_ops[dt][s], p_op[s], o_acc[dt], 0, 0, 0);
#pragma unroll
    for (int s = 0; s < 2; ++s) l_acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, p_op[s], l_acc, 0, 0, 0);

    // the tile requested above must have landed in LDS before any wavefront reads it: the wait
    // is stated here and not left to the compiler's bookkeeping of asynchronous LDS writes
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // ... and lets the next block overwrite this buffer
  };

  for (int it = kb_begin; it < kb_end; it += 2) {
    if (prio_step > 0) {
      const int left = kb_end - it + later_blocks;  // (all of it in scalar registers)
      if (left >= 3 * prio_step) __builtin_amdgcn_s_setprio(3);
      else if (left >= 2 * prio_step) __builtin_amdgcn_s_setprio(2);
      else if (left >= prio_step) __builtin_amdgcn_s_setprio(1);
      else __builtin_amdgcn_s_setprio(0);
    }
    key_block(Even{}, it);
    if (it + 1 < kb_end) key_block(Odd{}, it + 1);
  }

  const float l = l_acc[0];
  if (part_slot >= 0) {
    // a stretch of a block row: the unnormalised sums, the reference maximum they are relative to
    // and the row sum go to the workspace; attn_merge_kernel combines the row's stretches
    float *part = partials + (((size_t)head * n_slots + part_slot) * kAttnBlock + (w * 16 + n)) * (D + 4);
#pragma unroll
    for (int dt = 0; dt < kFeat; ++dt) *reinterpret_cast<floatx4 *>(part + 16 * dt + 4 * g) = o_acc[dt];
    if (g == 0) {
      part[D] = m_run;
      part[D + 1] = l;
    }
    continue;
  }
  const float inv = l > 0.0f ? 1.0f / l : 0.0f;  // queries without a live key give zeros
  __bf16 *out = O + head_off + (size_t)query * D;
#pragma unroll
  for (int dt = 0; dt < kFeat; ++dt) {
    bf16x4 o;
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = (__bf16)(o_acc[dt][r] * inv);
    *reinterpret_cast<bf16x4 *>(out + 16 * dt + 4 * g) = o;
  }
  }  // pass
}

// Combines the stretches of a block row that was shared out: with m* the largest of the
// stretches' reference maxima (base-2 exponents), O = sum_p 2^(m_p - m*) O_p / sum_p 2^(m_p - m*) l_p.
// One workgroup per (split row, head); thread t takes query t / 4 and a quarter of the features.
template <int D>
__global__ __launch_bounds__(kBlockThreads) void attn_merge_kernel(int S, int n_slots,
                                                                   const int4 *__restrict__ split_rows,
                                                                   const float *__restrict__ partials,
                                                                   __bf16 *__restrict__ O) {
  const int4 row = split_rows[blockIdx.x];  // x: block row, y: first slot, z: number of stretches
  const int head = blockIdx.y;
  const int q = threadIdx.x >> 2, quarter = threadIdx.x & 3;
  constexpr int kMine = D / 4;  // features per thread
  const float *base = partials + (((size_t)head * n_slots + row.y) * kAttnBlock + q) * (D + 4);
  const size_t part_stride = (size_t)kAttnBlock * (D + 4);
  float m_star = -3.0e38f;
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
  __bf16 *out = O + ((size_t)head * S + (size_t)row.x * kAttnBlock + q) * D + quarter * kMine;
#pragma unroll
  for (int j = 0; j < kMine; j += 4) {
    bf16x4 o;
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = (__bf16)(acc[j + r] * inv);
    *reinterpret_cast<bf16x4 *>(out + j) = o;
  }
}

}  // namespace scorch

namespace scorch {

template <int D>
static void attn_launch_dim(dim3 grid, hipStream_t s, bool negative, int S, int n_blocks, int H,
                            const int32_t *block_row_ptr, const int32_t *block_col_idx,
                            const int32_t *block_mask_index, const unsigned long long *block_masks,
                            const __bf16 *q, const __bf16 *k, const __bf16 *v, float scale_log2e,
                            __bf16 *o, int n_items, const int4 *items, int n_slots, float *partials, int pairs,
                            int prio_step) {
#define SCORCH_ATTN_LAUNCH(NEG, MASKED)                                                          \
  attn_blocksparse_kernel<D, NEG, MASKED><<<grid, kBlockThreads, 0, s>>>(                        \
      S, n_blocks, H, block_row_ptr, block_col_idx, block_mask_index, block_masks, q, k, v,      \
      scale_log2e, o, n_items, items, n_slots, partials, pairs, prio_step)
  const bool masked = block_mask_index != nullptr;
  if (negative) {
    if (masked) SCORCH_ATTN_LAUNCH(true, true); else SCORCH_ATTN_LAUNCH(true, false);
  } else {
    if (masked) SCORCH_ATTN_LAUNCH(false, true); else SCORCH_ATTN_LAUNCH(false, false);
  }
#undef SCORCH_ATTN_LAUNCH
}

// Block rows shared out among several workgroups (scorch_hip_attn_blocksparse_split_bf16).
struct AttnSplit {
  int64_t n_items = 0, n_split_rows = 0, n_slots = 0;
  bool pair_items = false;              // a workgroup takes the k-th longest and then the k-th shortest item
  int prio_step = 0;                    // > 0: wavefront priority by the blocks a workgroup has left, in levels of this many
  const int32_t *items = nullptr;       // 4 per item: block row, begin, end, slot (-1: writes O itself)
  const int32_t *split_rows = nullptr;  // 4 per split row: block row, first slot, stretches, 0
  void *workspace = nullptr;
  size_t workspace_bytes = 0;
};

inline size_t attn_split_workspace_bytes(int64_t H, int64_t n_slots, int64_t D) {
  return (size_t)H * (size_t)n_slots * kAttnBlock * (size_t)(D + 4) * sizeof(float);
}

// Shared by the entry points; block_mask_index == nullptr means every listed block is fully
// live, split == nullptr that every block row is one workgroup's.
static int attn_entry(const char *fn, int64_t H, int64_t S, int64_t D, int64_t block,
                      int64_t n_active_blocks, const int32_t *block_row_ptr,
                      const int32_t *block_col_idx, const int32_t *block_mask_index,
                      const uint64_t *block_masks, const void *Q, const void *K, const void *V,
                      float scale, void *O, void *stream, const AttnSplit *split = nullptr) {
  if (H < 0 || S < 0 || D < 0 || block <= 0 || n_active_blocks < 0)
    return fail(SCORCH_HIP_EINVAL, "%s: negative size (H=%lld S=%lld D=%lld block=%lld)", fn,
                (long long)H, (long long)S, (long long)D, (long long)block);
  if ((D != 32 && D != 64 && D != 128) || block != kAttnBlock)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: only head dimensions 32, 64 and 128 and %d x %d mask "
                "blocks are built (got D=%lld block=%lld)", fn, kAttnBlock, kAttnBlock, (long long)D,
                (long long)block);
  if (S % kAttnBlock != 0)
    return fail(SCORCH_HIP_EINVAL, "%s: S=%lld is not a multiple of the block size", fn, (long long)S);
  if (H * (S / kAttnBlock) > INT32_MAX || S * D > INT32_MAX)
    return fail(SCORCH_HIP_EUNSUPPORTED, "%s: H=%lld or S=%lld too large", fn, (long long)H, (long long)S);
  SCORCH_REQUIRE(split || block_row_ptr != nullptr, "%s: block_row_ptr is NULL", fn);
  if (H == 0 || S == 0) return SCORCH_HIP_OK;
  SCORCH_REQUIRE(n_active_blocks == 0 || block_col_idx != nullptr, "%s: block_col_idx is NULL", fn);
  SCORCH_REQUIRE(Q && K && V && O, "%s: NULL Q/K/V/O", fn);
  SCORCH_REQUIRE(aligned_to(Q, 16) && aligned_to(K, 16) && aligned_to(V, 16) && aligned_to(O, 16),
                 "%s: Q, K, V and O must be 16-byte aligned", fn);
  const int n_blocks = (int)(S / kAttnBlock);
  int n_items = n_blocks, n_slots = 0;
  const int4 *items = nullptr;
  float *partials = nullptr;
  if (split) {
    if (split->n_items < 0 || split->n_split_rows < 0 || split->n_slots < 0 || split->n_items * H > INT32_MAX ||
        split->n_slots > INT32_MAX)
      return fail(SCORCH_HIP_EINVAL, "%s: n_items=%lld n_split_rows=%lld n_slots=%lld", fn,
                  (long long)split->n_items, (long long)split->n_split_rows, (long long)split->n_slots);
    if (split->n_items == 0) return SCORCH_HIP_OK;
    SCORCH_REQUIRE(split->items != nullptr && aligned_to(split->items, 16), "%s: items must be 16-byte aligned", fn);
    SCORCH_REQUIRE(split->n_split_rows == 0 || (split->split_rows != nullptr && aligned_to(split->split_rows, 16)),
                   "%s: split_rows must be 16-byte aligned", fn);
    const size_t need = attn_split_workspace_bytes(H, split->n_slots, D);
    if (need > 0 && (!split->workspace || split->workspace_bytes < need || !aligned_to(split->workspace, 256)))
      return fail(SCORCH_HIP_EWORKSPACE, "%s: a 256-byte aligned workspace of %zu bytes is needed, %zu given", fn,
                  need, split->workspace ? split->workspace_bytes : (size_t)0);
    n_items = (int)split->n_items;
    n_slots = (int)split->n_slots;
    items = reinterpret_cast<const int4 *>(split->items);
    partials = static_cast<float *>(split->workspace);
  }
  // pairs: every workgroup takes two items, see the kernel (asked for through the work-list entry)
  const int pairs = split && split->pair_items && n_items >= 2;
  const int prio_step = split ? split->prio_step : 0;
  const dim3 grid((unsigned)((pairs ? (n_items + 1) / 2 : n_items) * H));
  const float scale_log2e = scale * 1.4426950408889634f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const __bf16 *q = static_cast<const __bf16 *>(Q), *k = static_cast<const __bf16 *>(K),
               *v = static_cast<const __bf16 *>(V);
  __bf16 *o = static_cast<__bf16 *>(O);
  const unsigned long long *masks = reinterpret_cast<const unsigned long long *>(block_masks);
  mark_launch(s);
  if (D == 32)
    attn_launch_dim<32>(grid, s, scale < 0.0f, (int)S, n_blocks, (int)H, block_row_ptr, block_col_idx,
                        block_mask_index, masks, q, k, v, scale_log2e, o, n_items, items, n_slots, partials, pairs, prio_step);
  else if (D == 64)
    attn_launch_dim<64>(grid, s, scale < 0.0f, (int)S, n_blocks, (int)H, block_row_ptr, block_col_idx,
                        block_mask_index, masks, q, k, v, scale_log2e, o, n_items, items, n_slots, partials, pairs, prio_step);
  else
    attn_launch_dim<128>(grid, s, scale < 0.0f, (int)S, n_blocks, (int)H, block_row_ptr, block_col_idx,
                         block_mask_index, masks, q, k, v, scale_log2e, o, n_items, items, n_slots, partials, pairs, prio_step);
  SCORCH_HIP_CHECK(hipGetLastError());
  mark_launch(s);
  if (split && split->n_split_rows > 0) {
    const dim3 merge_grid((unsigned)split->n_split_rows, (unsigned)H);
    const int4 *rows = reinterpret_cast<const int4 *>(split->split_rows);
    if (D == 32) attn_merge_kernel<32><<<merge_grid, kBlockThreads, 0, s>>>((int)S, n_slots, rows, partials, o);
    else if (D == 64) attn_merge_kernel<64><<<merge_grid, kBlockThreads, 0, s>>>((int)S, n_slots, rows, partials, o);
    else attn_merge_kernel<128><<<merge_grid, kBlockThreads, 0, s>>>((int)S, n_slots, rows, partials, o);
    SCORCH_HIP_CHECK(hipGetLastError());
    mark_launch(s);
  }
  return SCORCH_HIP_OK;
}

}  // namespace scorch

extern "C" int scorch_hip_attn_blocksparse_bf16(int64_t H, int64_t S, int64_t D, int64_t block,
                                                int64_t n_active_blocks,
                                                const int32_t *block_row_ptr,
                                                const int32_t *block_col_idx, const void *Q,
                                                const void *K, const void *V, float scale, void *O,
                                                void *stream) {
  return scorch::attn_entry("scorch_hip_attn_blocksparse_bf16", H, S, D, block, n_active_blocks,
                            block_row_ptr, block_col_idx, nullptr, nullptr, Q, K, V, scale, O,
                            stream);
}

extern "C" int scorch_hip_attn_blocksparse_masked_bf16(
    int64_t H, int64_t S, int64_t D, int64_t block, int64_t n_active_blocks,
    const int32_t *block_row_ptr, const int32_t *block_col_idx, const int32_t *block_mask_index,
    int64_t n_masks, const uint64_t *block_masks, const void *Q, const void *K, const void *V,
    float scale, void *O, void *stream) {
  using namespace scorch;
  const char *fn = "scorch_hip_attn_blocksparse_masked_bf16";
  if (n_masks < 0) return fail(SCORCH_HIP_EINVAL, "%s: n_masks=%lld", fn, (long long)n_masks);
  if (n_active_blocks > 0 && H > 0 && S > 0) {
    SCORCH_REQUIRE(block_mask_index != nullptr, "%s: block_mask_index is NULL", fn);
    SCORCH_REQUIRE(n_masks == 0 || block_masks != nullptr, "%s: block_masks is NULL", fn);
    SCORCH_REQUIRE(aligned_to(block_masks, 8), "%s: block_masks must be 8-byte aligned", fn);
  }
  return attn_entry(fn, H, S, D, block, n_active_blocks, block_row_ptr, block_col_idx,
                    n_active_blocks > 0 ? block_mask_index : nullptr, block_masks, Q, K, V, scale,
                    O, stream);
}

extern "C" size_t scorch_hip_attn_blocksparse_split_workspace_bytes(int64_t H, int64_t n_slots, int64_t D) {
  if (H <= 0 || n_slots <= 0 || D <= 0) return 0;
  return scorch::attn_split_workspace_bytes(H, n_slots, D);
}

extern "C" int scorch_hip_attn_blocksparse_split_bf16(
    int64_t H, int64_t S, int64_t D, int64_t block, int64_t n_active_blocks, int64_t n_items,
    const int32_t *items, int pair_items, int priority_step, int64_t n_split_rows, const int32_t *split_rows,
    int64_t n_slots, const int32_t *block_col_idx, const int32_t *block_mask_index, int64_t n_masks,
    const uint64_t *block_masks, const void *Q, const void *K, const void *V, float scale, void *O,
    void *workspace, size_t workspace_bytes, void *stream) {
  using namespace scorch;
  const char *fn = "scorch_hip_attn_blocksparse_split_bf16";
  if (n_masks < 0) return fail(SCORCH_HIP_EINVAL, "%s: n_masks=%lld", fn, (long long)n_masks);
  if (priority_step < 0) return fail(SCORCH_HIP_EINVAL, "%s: priority_step=%d", fn, priority_step);
  if (block_mask_index != nullptr) {
    SCORCH_REQUIRE(n_masks == 0 || block_masks != nullptr, "%s: block_masks is NULL", fn);
    SCORCH_REQUIRE(aligned_to(block_masks, 8), "%s: block_masks must be 8-byte aligned", fn);
  }
  AttnSplit split;
  split.n_items = n_items;
  split.pair_items = pair_items != 0;
  split.prio_step = priority_step;
  split.n_split_rows = n_split_rows;
  split.n_slots = n_slots;
  split.items = items;
  split.split_rows = split_rows;
  split.workspace = workspace;
  split.workspace_bytes = workspace_bytes;
  return attn_entry(fn, H, S, D, block, n_active_blocks, nullptr, block_col_idx, block_mask_index, block_masks,
                    Q, K, V, scale, O, stream, &split);
}

SCORCH_DEFINE_PRELOAD(attn)
