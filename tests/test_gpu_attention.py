"""Fused block-sparse attention (bf16 in/out, fp32 accumulation) on the MI355X
through the C ABI.

Tolerance: relative Frobenius error <= 1e-2 against an fp64 recomputation on
the same (bf16-representable) inputs -- the bar for the bf16 path.  The
reference has no bf16 or fused kernel, so nothing of its own pins this path:
the oracle here is the textbook masked softmax (the reference's "dense" mode,
bench/bench_sparse_transformer.py:330-335) in float64, and, as a second
witness, this package's own fp32 SDDMM -> softmax -> SpMM pipeline.
"""
import numpy as np
import pytest
import torch

import scorch_amd as scorch
from gpu_util import dev
from scorch_amd import STensor, workloads
from scorch_amd import scorch_ops_hip as H

pytestmark = pytest.mark.gpu
TOL_BF16 = 1e-2


def bf16_inputs(S, heads, D, seed, window=4, stride=8):
    w = workloads.attention_blocksparse(S=S, H=heads, D=D, seed=seed, window=window, stride=stride)
    q, k, v = (torch.from_numpy(w[n]).to(torch.bfloat16) for n in ("q", "k", "v"))
    return w, q, k, v


def run_fused(w, q, k, v):
    out = H.attn_blocksparse_bf16(q.cuda(), k.cuda(), v.cuda(), dev(w["block_row_ptr"]),
                                  dev(w["block_col_idx"]), float(w["scale"]))
    assert out.dtype == torch.bfloat16 and out.shape == q.shape
    return out


@pytest.mark.parametrize("S,heads,seed", [(64, 1, 0), (256, 2, 1), (1024, 3, 2)])
def test_against_fp64_oracle(oracle, S, heads, seed):
    w, q, k, v = bf16_inputs(S, heads, 64, seed)
    out = run_fused(w, q, k, v).float().cpu().numpy()
    ref = oracle.attention_blocksparse_fp64(q.float().numpy(), k.float().numpy(), v.float().numpy(),
                                            w["block_row_ptr"], w["block_col_idx"], 64, float(w["scale"]))
    assert oracle.rel_fro(out, ref) <= TOL_BF16
    # well inside the bar: bf16 rounding of P and of the output is ~2^-9
    assert oracle.rel_fro(out, ref) <= 5e-3


def test_arbitrary_block_pattern_with_empty_block_rows(oracle):
    S, nb = 512, 8
    rng = np.random.default_rng(3)
    active = rng.random((nb, nb)) < 0.4
    active[2, :] = False                      # a block row with nothing to attend to
    active[5, :] = True                       # a full block row
    r, c = np.nonzero(active)
    brp = np.concatenate([[0], np.cumsum(np.bincount(r, minlength=nb))]).astype(np.int32)
    bci = c.astype(np.int32)
    q, k, v = (torch.from_numpy(rng.standard_normal((2, S, 64)).astype(np.float32)).to(torch.bfloat16)
               for _ in range(3))
    out = H.attn_blocksparse_bf16(q.cuda(), k.cuda(), v.cuda(), dev(brp), dev(bci), 0.125)
    out = out.float().cpu().numpy()
    ref = oracle.attention_blocksparse_fp64(q.float().numpy(), k.float().numpy(), v.float().numpy(),
                                            brp, bci, 64, 0.125)
    assert not out[:, 128:192].any()          # queries of block row 2
    assert oracle.rel_fro(out, ref) <= TOL_BF16


def test_large_scores_do_not_overflow(oracle):
    w, q, k, v = bf16_inputs(256, 1, 64, 4)
    out = H.attn_blocksparse_bf16((q * 8).cuda(), (k * 8).cuda(), v.cuda(), dev(w["block_row_ptr"]),
                                  dev(w["block_col_idx"]), 1.0).float().cpu().numpy()
    ref = oracle.attention_blocksparse_fp64((q * 8).float().numpy(), (k * 8).float().numpy(),
                                            v.float().numpy(), w["block_row_ptr"], w["block_col_idx"],
                                            64, 1.0)
    assert np.isfinite(out).all() and oracle.rel_fro(out, ref) <= TOL_BF16


def test_matches_unfused_fp32_pipeline():
    """Same inputs through SDDMM -> CSR softmax -> SpMM in fp32 (one head)."""
    w, q, k, v = bf16_inputs(1024, 1, 64, 5)
    fused = run_fused(w, q, k, v).float()[0]
    rp, ci = workloads.blocks_to_csr(w["block_row_ptr"], w["block_col_idx"], 64)
    S = 1024
    mask = STensor.from_csr_arrays(dev(rp), dev(ci), torch.ones(ci.size, device="cuda"), (S, S))
    scores = scorch.einsum("ij,ik,jk->ij", mask, q[0].float().cuda(), k[0].float().cuda())
    probs = H.softmax_csr_float(dev(rp), scores.values, float(w["scale"]))
    unfused = scorch.matmul(STensor.from_csr_arrays(dev(rp), dev(ci), probs, (S, S)), v[0].float().cuda())
    err = (torch.linalg.norm(fused - unfused) / torch.linalg.norm(unfused)).item()
    assert err <= TOL_BF16


def test_runs_are_bit_reproducible():
    w, q, k, v = bf16_inputs(2048, 4, 64, 6)
    a = run_fused(w, q, k, v)
    b = run_fused(w, q, k, v)
    assert torch.equal(a, b)


def test_full_size_workload():
    """S = 8192, 16 heads, D = 64, 64 x 64 blocks (window 4 + every 8th): each
    head against the masked dense softmax in fp64 on the device."""
    w, q, k, v = bf16_inputs(8192, 16, 64, workloads.SEEDS["attention_blocksparse"])
    assert w["block_col_idx"].size == 1466
    out = run_fused(w, q, k, v)
    nb = 128
    blocks = torch.zeros(nb, nb, dtype=torch.bool)
    rows = np.repeat(np.arange(nb), np.diff(w["block_row_ptr"]))
    blocks[torch.from_numpy(rows), torch.from_numpy(w["block_col_idx"]).long()] = True
    mask = blocks.cuda().repeat_interleave(64, 0).repeat_interleave(64, 1)
    worst = 0.0
    for h in range(16):
        q64, k64, v64 = (t[h].cuda().double() for t in (q, k, v))
        s = (q64 @ k64.T) * float(w["scale"])
        s.masked_fill_(~mask, float("-inf"))
        ref = torch.softmax(s, dim=-1) @ v64
        err = (torch.linalg.norm(out[h].double() - ref) / torch.linalg.norm(ref)).item()
        worst = max(worst, err)
        del s, ref
    assert worst <= TOL_BF16, worst


def test_negative_scale(oracle):
    w, q, k, v = bf16_inputs(256, 2, 64, 7)
    out = H.attn_blocksparse_bf16(q.cuda(), k.cuda(), v.cuda(), dev(w["block_row_ptr"]),
                                  dev(w["block_col_idx"]), -0.25).float().cpu().numpy()
    ref = oracle.attention_blocksparse_fp64(q.float().numpy(), k.float().numpy(), v.float().numpy(),
                                            w["block_row_ptr"], w["block_col_idx"], 64, -0.25)
    assert oracle.rel_fro(out, ref) <= TOL_BF16


@pytest.mark.parametrize("blocks_per_row", [1, 2, 3, 5])
def test_short_and_odd_block_rows(oracle, blocks_per_row):
    """Every block row has the same small number of key blocks (the tile pipeline's start-up cases)."""
    S, nb = 512, 8
    rng = np.random.default_rng(blocks_per_row)
    cols = np.stack([np.sort(rng.choice(nb, blocks_per_row, replace=False)) for _ in range(nb)])
    brp = (np.arange(nb + 1) * blocks_per_row).astype(np.int32)
    bci = cols.reshape(-1).astype(np.int32)
    q, k, v = (torch.from_numpy(rng.standard_normal((8, S, 64)).astype(np.float32)).to(torch.bfloat16)
               for _ in range(3))
    out = H.attn_blocksparse_bf16(q.cuda(), k.cuda(), v.cuda(), dev(brp), dev(bci), 0.125).float().cpu().numpy()
    ref = oracle.attention_blocksparse_fp64(q.float().numpy(), k.float().numpy(), v.float().numpy(),
                                            brp, bci, 64, 0.125)
    assert oracle.rel_fro(out, ref) <= TOL_BF16


# ---- other head dimensions, and masks that are not unions of whole blocks ----

@pytest.mark.parametrize("D", [32, 128])
@pytest.mark.parametrize("S,heads,seed", [(64, 1, 10), (512, 3, 11)])
def test_other_head_dimensions(oracle, D, S, heads, seed):
    w, q, k, v = bf16_inputs(S, heads, D, seed)
    out = run_fused(w, q, k, v).float().cpu().numpy()
    ref = oracle.attention_blocksparse_fp64(q.float().numpy(), k.float().numpy(), v.float().numpy(),
                                            w["block_row_ptr"], w["block_col_idx"], 64, float(w["scale"]))
    assert oracle.rel_fro(out, ref) <= 5e-3


def csr_of(mask_bool):
    rp = np.concatenate([[0], np.cumsum(mask_bool.sum(1))]).astype(np.int32)
    return rp, np.nonzero(mask_bool)[1].astype(np.int32)


def masked_case(oracle, mask_bool, heads, D, seed, scale=None):
    S = mask_bool.shape[0]
    rng = np.random.default_rng(seed)
    q, k, v = (torch.from_numpy(rng.standard_normal((heads, S, D)).astype(np.float32)).to(torch.bfloat16)
               for _ in range(3))
    scale = D ** -0.5 if scale is None else scale
    rp, ci = csr_of(mask_bool)
    out = H.sparse_attention_bf16(q.cuda(), k.cuda(), v.cuda(), dev(rp), dev(ci), scale).float().cpu().numpy()
    ref = np.stack([oracle.attention_dense_fp64(q[h].float().numpy(), k[h].float().numpy(),
                                                v[h].float().numpy(), mask_bool, scale) for h in range(heads)])
    return out, ref


def test_block_mask_regrouping_of_a_csr_mask():
    """The block structure built from a CSR mask: every entry in exactly its block's bit mask,
    full blocks marked -1, equal masks shared."""
    S = 256
    rng = np.random.default_rng(20)
    mask = rng.random((S, S)) < 0.02
    mask[64:128, 128:192] = True                       # a full block
    mask[192:256, :] = False                           # an empty block row
    mask[0:64, 0:64] = np.tri(64, dtype=bool)          # two equal partial blocks
    mask[128:192, 64:128] = np.tri(64, dtype=bool)
    rp, ci = csr_of(mask)
    bm = H.block_mask_from_csr(dev(rp), dev(ci), S)
    brp, bci, bmi = (t.cpu().numpy() for t in (bm.block_row_ptr, bm.block_col_idx, bm.block_mask_index))
    words = bm.block_masks.cpu().numpy().view(np.uint64).reshape(-1, 64)
    assert bm.nnz == int(mask.sum()) and brp[-1] == bci.size and brp[4] == brp[3]
    rebuilt = np.zeros_like(mask)
    for br in range(4):
        for i in range(brp[br], brp[br + 1]):
            bits = (np.full((64, 64), True) if bmi[i] < 0 else
                    ((words[bmi[i]][:, None] >> np.arange(64, dtype=np.uint64)[None, :]) & np.uint64(1)).astype(bool))
            rebuilt[64 * br:64 * br + 64, 64 * bci[i]:64 * bci[i] + 64] = bits
    assert np.array_equal(rebuilt, mask)
    at = {(br, int(bci[i])): int(bmi[i]) for br in range(4) for i in range(brp[br], brp[br + 1])}
    assert at[(1, 2)] == -1 and at[(0, 0)] == at[(2, 1)] >= 0
    assert bm.n_masks < bci.size


@pytest.mark.parametrize("D", [32, 64, 128])
def test_random_entry_mask(oracle, D):
    S = 256
    rng = np.random.default_rng(21 + D)
    mask = rng.random((S, S)) < 0.1
    mask[7, :] = False                                 # a query without keys inside active blocks
    mask[64:128, :] = False                            # an empty block row
    mask[130, :] = False
    mask[130, 255] = True                              # one key only (bit 63 of its word)
    out, ref = masked_case(oracle, mask, 2, D, 22)
    assert not out[:, 7].any() and not out[:, 64:128].any()
    assert oracle.rel_fro(out, ref) <= 5e-3


@pytest.mark.parametrize("D", [32, 64])
def test_causal_mask(oracle, D):
    S = 512
    out, ref = masked_case(oracle, np.tri(S, dtype=bool), 2, D, 23)
    assert oracle.rel_fro(out, ref) <= 5e-3


def test_masked_negative_scale_and_large_scores(oracle):
    S = 256
    rng = np.random.default_rng(24)
    mask = rng.random((S, S)) < 0.3
    out, ref = masked_case(oracle, mask, 1, 32, 25, scale=-3.0)
    assert np.isfinite(out).all() and oracle.rel_fro(out, ref) <= TOL_BF16
    out, ref = masked_case(oracle, mask, 1, 32, 26, scale=4.0)
    assert np.isfinite(out).all() and oracle.rel_fro(out, ref) <= TOL_BF16


def test_longformer_mask_reference_shape(oracle):
    """The reference's attention benchmark at its own shape (bench/bench_sparse_transformer.py:117-141,
    README: S = 4096, 8 heads, D = 32, window 64 + one global token, 532,286 entries): every head
    against the dense masked softmax in fp64 on the device, and against the fp32 three-launch form."""
    S, heads, D = 4096, 8, 32
    rp, ci = workloads.longformer_mask(S)
    assert ci.size == 532286
    rng = np.random.default_rng(27)
    q, k, v = (torch.from_numpy(rng.standard_normal((heads, S, D)).astype(np.float32)).to(torch.bfloat16).cuda()
               for _ in range(3))
    scale = D ** -0.5
    drp, dci = dev(rp), dev(ci)
    out = H.sparse_attention_bf16(q, k, v, drp, dci, scale)
    assert torch.equal(out, H.sparse_attention_bf16(q, k, v, drp, dci, scale))      # cached plan, same bits
    dense = torch.zeros(S, S, dtype=torch.bool)
    dense[torch.from_numpy(np.repeat(np.arange(S), np.diff(rp))), torch.from_numpy(ci).long()] = True
    dense = dense.cuda()
    worst = 0.0
    for h in range(heads):
        s = (q[h].double() @ k[h].double().T) * scale
        s.masked_fill_(~dense, float("-inf"))
        ref = torch.softmax(s, dim=-1) @ v[h].double()
        worst = max(worst, (torch.linalg.norm(out[h].double() - ref) / torch.linalg.norm(ref)).item())
    assert worst <= TOL_BF16, worst
    unfused = H.sparse_attention_csr(drp, dci, q.float(), k.float(), v.float(), scale)
    err = (torch.linalg.norm(out.float() - unfused) / torch.linalg.norm(unfused)).item()
    assert err <= TOL_BF16


# ---- long block rows shared out among workgroups ----

@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("longest", [1, 3, 4])
def test_shared_out_block_rows(oracle, D, longest):
    """A mask with a global token and a few long rows: every stretch length, stretches in which a
    query has no live key, against the fp64 dense masked softmax and against the unsplit kernel."""
    S = 512
    rng = np.random.default_rng(30 + D + longest)
    mask = np.abs(np.arange(S)[:, None] - np.arange(S)[None, :]) <= 40
    mask[0, :] = True                                  # a global token: block row 0 holds all 8 blocks
    mask[:, 0] = True
    mask[300:310, ::7] = True                          # a few more long rows, sparse within their blocks
    mask[65, :] = False                                # a query without keys
    rp, ci = csr_of(mask)
    q, k, v = (torch.from_numpy(rng.standard_normal((3, S, D)).astype(np.float32)).to(torch.bfloat16).cuda()
               for _ in range(3))
    scale = D ** -0.5
    bm = H.block_mask_from_csr(dev(rp), dev(ci), S)
    whole = H.attn_blocksparse_bf16(q, k, v, bm.block_row_ptr, bm.block_col_idx, scale,
                                    block_mask_index=bm.block_mask_index, block_masks=bm.block_masks)
    H.split_long_block_rows(bm, longest)
    assert bm.items is not None and bm.n_slots >= 2
    # every key block is in exactly one item, and a shared-out row's stretches have consecutive slots
    items = bm.items.cpu().numpy().reshape(-1, 4)
    covered = np.zeros(bm.n_active_blocks, int)
    for row, lo, hi, slot in items:
        covered[lo:hi] += 1
    assert (covered == 1).all() and (np.diff(items[:, 2] - items[:, 1]) <= 0).all()
    out = H.attn_blocksparse_split_bf16(q, k, v, bm, scale)
    assert torch.equal(out, H.attn_blocksparse_split_bf16(q, k, v, bm, scale))
    ref = np.stack([oracle.attention_dense_fp64(q[h].float().cpu().numpy(), k[h].float().cpu().numpy(),
                                                v[h].float().cpu().numpy(), mask, scale) for h in range(3)])
    assert not out[:, 65].any()
    assert oracle.rel_fro(out.float().cpu().numpy(), ref) <= 5e-3
    err = ((out.float() - whole.float()).norm() / whole.float().norm()).item()
    assert err <= 5e-3


def test_shared_out_rows_with_negative_scale_and_unmasked_blocks(oracle):
    """Whole blocks only (no bit masks in use), negative scale."""
    w, q, k, v = bf16_inputs(1024, 2, 64, 31)
    rp, ci = workloads.blocks_to_csr(w["block_row_ptr"], w["block_col_idx"], 64)
    bm = H.split_long_block_rows(H.block_mask_from_csr(dev(rp), dev(ci), 1024), 2)
    assert bm.items is not None and int((bm.block_mask_index >= 0).sum()) == 0
    out = H.attn_blocksparse_split_bf16(q.cuda(), k.cuda(), v.cuda(), bm, -0.25).float().cpu().numpy()
    ref = oracle.attention_blocksparse_fp64(q.float().numpy(), k.float().numpy(), v.float().numpy(),
                                            w["block_row_ptr"], w["block_col_idx"], 64, -0.25)
    assert oracle.rel_fro(out, ref) <= TOL_BF16


def test_masks_with_rows_of_similar_length_are_not_shared_out():
    w = workloads.attention_blocksparse(S=1024, H=1, D=64)
    rp, ci = workloads.blocks_to_csr(w["block_row_ptr"], w["block_col_idx"], 64)
    bm = H.attention_block_mask(dev(rp), dev(ci), 1024)
    assert bm.items is None and bm.n_slots == 0
    rp, ci = workloads.longformer_mask(4096)
    bm = H.attention_block_mask(dev(rp), dev(ci), 4096)
    assert bm.items is not None and bm.split_rows.cpu().tolist()[:3] == [0, 0, 7]


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("kind", ["strided", "causal", "random_with_bit_masks", "odd_count"])
def test_workgroups_that_take_two_items_change_nothing(oracle, D, kind):
    """pair_items of the work-list entry: every workgroup takes the k-th longest and then the k-th
    shortest item.  Bit for bit the result of one item per workgroup, whole block rows and
    shared-out stretches alike, with and without per-block bit masks, and an odd number of items."""
    from scorch_amd import native
    rng = np.random.default_rng(D + len(kind))
    heads = 3
    if kind == "random_with_bit_masks":
        S = 512
        mask = rng.random((S, S)) < 0.3
        mask[64:128] = False
        rp = np.concatenate([[0], np.cumsum(mask.sum(1))]).astype(np.int32)
        bm = H.block_mask_from_csr(dev(rp), dev(np.nonzero(mask)[1].astype(np.int32)), S)
    else:
        nb = {"strided": 24, "causal": 16, "odd_count": 7}[kind]
        S = 64 * nb
        brp, bci = workloads.blocksparse_pattern(nb, window=3 if kind == "strided" else nb, stride=4)
        bm = H.BlockMask(S, 64, dev(brp), dev(bci), None, None, int(bci.size) * 4096)
    q, k, v = (torch.randn(heads, S, D, device="cuda").to(torch.bfloat16) for _ in range(3))
    for longest in (None, 2):                                     # whole rows; rows shared out in stretches of two
        if longest is None:
            items, split_rows, n_slots = H._stretches(bm.row_lens(), max(int(bm.row_lens().max()), 1), True)
        else:
            items, split_rows, n_slots = H._stretches(bm.row_lens(), longest, True)
        t_items = torch.from_numpy(items).cuda().reshape(-1)
        t_rows = torch.from_numpy(split_rows).cuda().reshape(-1) if n_slots else None
        single = H._attn_bf16_items(q, k, v, bm, t_items, t_rows, n_slots, D ** -0.5, False)
        paired = H._attn_bf16_items(q, k, v, bm, t_items, t_rows, n_slots, D ** -0.5, True)
        assert torch.equal(single, paired)
        # wavefront priorities by the work a workgroup has left: they order the work, not the sums
        for step in (1, 3, 1000):
            assert torch.equal(single, H._attn_bf16_items(q, k, v, bm, t_items, t_rows, n_slots, D ** -0.5, False, step))
            assert torch.equal(single, H._attn_bf16_items(q, k, v, bm, t_items, t_rows, n_slots, D ** -0.5, True, step))
        if longest is None:
            whole = single
    plain = H.attn_blocksparse_bf16(q, k, v, bm.block_row_ptr, bm.block_col_idx, D ** -0.5,
                                    block_mask_index=bm.block_mask_index, block_masks=bm.block_masks)
    assert torch.equal(plain, whole)
    if kind != "random_with_bit_masks":
        ref = oracle.attention_blocksparse_fp64(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(),
                                                bm.block_row_ptr.cpu().numpy(), bm.block_col_idx.cpu().numpy(), 64, D ** -0.5)
        assert oracle.rel_fro(whole.float().cpu().numpy(), ref) <= TOL_BF16


def test_the_dispatch_pairs_items_where_it_was_measured_to_pay():
    """A causal mask at S = 4096 with 16 heads fills the chip once with uneven workgroups: the
    wrapper hands the block rows over as a paired work list; with 4 heads it does not.  Same bits."""
    nb = 64
    brp, bci = workloads.blocksparse_pattern(nb, window=nb, stride=1)
    t_brp, t_bci = dev(brp), dev(bci)
    for heads, expect in ((16, True), (4, False)):
        q, k, v = (torch.randn(heads, 64 * nb, 64, device="cuda").to(torch.bfloat16) for _ in range(3))
        out = H.attn_blocksparse_bf16(q, k, v, t_brp, t_bci, 0.125)
        assert t_brp._scorch_rows[3][(heads, 64)][0] is expect
        assert (t_brp._scorch_rows[3][(heads, 64)][1] > 0) is expect     # 8 pairs per CU / one workgroup per CU
        rc_out = torch.empty_like(q)
        from scorch_amd import native
        native.check(native.lib().scorch_hip_attn_blocksparse_bf16(
            heads, 64 * nb, 64, 64, t_bci.numel(), t_brp.data_ptr(), t_bci.data_ptr(), q.data_ptr(), k.data_ptr(),
            v.data_ptr(), 0.125, rc_out.data_ptr(), torch.cuda.current_stream().cuda_stream))
        assert torch.equal(out, rc_out)
