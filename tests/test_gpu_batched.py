"""One sparsity pattern, one launch for all heads: the batched SDDMM, row softmax and SpMM
entry points against per-head calls (bit for bit), and the three of them composed into the
reference's sparse attention (bench/bench_sparse_transformer.py:354-372) against an fp64 dense
masked softmax at the benchmark's own shape: S = 4096, head dimension 32, 8 heads, Longformer
mask (window 64 on either side, one global token)."""
import numpy as np
import pytest
import torch

from gpu_util import dev, spmm_path
from scorch_amd import scorch_ops_hip as H
from scorch_amd import workloads

pytestmark = pytest.mark.gpu


def _patterns():
    rng = np.random.default_rng(4)
    out = {"longformer_640": workloads.longformer_mask(640, window=64, n_global=1)}   # one long row, else 129
    rp, ci = workloads.blocks_to_csr(*workloads.blocksparse_pattern(12), block=64)    # rows of 64 .. 320 entries
    out["blocks_768"] = (rp, ci)
    lens = rng.integers(0, 30, 500); lens[[3, 250]] = [5000, 9000]                    # giant rows for the softmax
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(9500, int(n), replace=False)) for n in lens]).astype(np.int32)
    out["giant_rows"] = (rp, ci)
    return out


PATTERNS = _patterns()


@pytest.mark.parametrize("name", sorted(PATTERNS))
@pytest.mark.parametrize("D", [32, 64, 100])
def test_batched_steps_equal_per_head_calls(name, D):
    rp_np, ci_np = PATTERNS[name]
    M = rp_np.size - 1
    n_cols = int(ci_np.max()) + 1 if name == "giant_rows" else M
    heads = 3
    g = torch.Generator(device="cuda").manual_seed(D)
    q = torch.randn(heads, M, D, device="cuda", generator=g)
    k = torch.randn(heads, n_cols, D, device="cuda", generator=g)
    v = torch.randn(heads, n_cols, D, device="cuda", generator=g)
    rp, ci = dev(rp_np), dev(ci_np)
    mask_vals = torch.rand(ci.numel(), device="cuda", generator=g) + 0.5
    csr = [[], [rp, ci]]

    # which kernels serve a pattern is decided when it comes back for its second product (a mask
    # made of 64 x 64 blocks goes to the block kernels): decided first, compared afterwards
    for _ in range(2):
        H.sddmm_csr_float_batched([M, n_cols], csr, mask_vals, q, k)
    scores, rows = H.sddmm_csr_float_batched([M, n_cols], csr, mask_vals, q, k)
    assert scores.shape == (heads, ci.numel())
    assert torch.equal(rows, torch.repeat_interleave(torch.arange(M, device="cuda", dtype=torch.int32),
                                                     (rp[1:] - rp[:-1]).long()))
    probs = H.softmax_csr_float_batched(rp, scores, 0.2)
    for path in ("auto", "merge", "rows"):
        with spmm_path(path):
            out = H.spmm_csr_float_batched([M, n_cols], csr, probs, v)
        assert out.shape == (heads, M, D)
        for h in range(heads):
            one = H.sddmm_csr_float([M, n_cols], [M, n_cols], csr, mask_vals, [M, D], [[], []], q[h].reshape(-1),
                                    [n_cols, D], [[], []], k[h].reshape(-1))
            assert torch.equal(one.storage.value, scores[h])
            assert torch.equal(H.softmax_csr_float(rp, scores[h], 0.2), probs[h])
            with spmm_path(path):
                single = H.spmm_csr_float_v2([M, D], [M, n_cols], csr, probs[h], [n_cols, D], [[], []],
                                             v[h].reshape(-1)).storage.value
            assert torch.equal(single.view(M, D), out[h]), (path, h)


def test_sparse_attention_at_the_reference_benchmarks_shape():
    S, heads, D = 4096, 8, 32
    rp_np, ci_np = workloads.longformer_mask(S)
    rp, ci = dev(rp_np), dev(ci_np)
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k, v = (torch.randn(heads, S, D, device="cuda", generator=g) for _ in range(3))
    scale = D ** -0.5
    out = H.sparse_attention_csr(rp, ci, q, k, v, scale)
    assert out.shape == (heads, S, D) and out.dtype == torch.float32
    rows = torch.repeat_interleave(torch.arange(S, device="cuda"), (rp[1:] - rp[:-1]).long())
    live = torch.zeros(S, S, dtype=torch.bool, device="cuda")
    live[rows, ci.long()] = True
    worst = 0.0
    for h in range(heads):
        s = (q[h].double() @ k[h].double().T) * scale
        p = torch.softmax(s.masked_fill(~live, float("-inf")), dim=1)
        ref = p @ v[h].double()
        worst = max(worst, (torch.linalg.norm(out[h].double() - ref) / torch.linalg.norm(ref)).item())
    assert worst <= 1e-5, worst          # fp32 throughout (the bf16 bar of the fused kernel is 1e-2)
    # the mask has come back: its two products now run by blocks (same bar), and from here on the
    # result is the same bits from call to call
    again = H.sparse_attention_csr(rp, ci, q, k, v, scale)
    assert isinstance(rp._scorch_plan.blocked, H.BlockedCsr)
    worst = max((torch.linalg.norm(again[h].double() - out[h].double()) / torch.linalg.norm(out[h].double())).item()
                for h in range(heads))
    assert worst <= 2e-6, worst
    assert torch.equal(again, H.sparse_attention_csr(rp, ci, q, k, v, scale))


def test_softmax_with_a_known_longest_row_skips_the_giant_row_pass():
    """Once a product has inspected the pattern (so that its longest row is known and at most
    4096), the row softmax runs as one launch; same bits as without that knowledge, and a pattern
    with a longer row keeps the general form."""
    rng = np.random.default_rng(9)
    for longest in (4096, 4097):
        lens = rng.integers(0, 40, 300)
        lens[17] = longest
        rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        ci = np.concatenate([np.sort(rng.choice(8192, n, replace=False)) for n in lens]).astype(np.int32)
        vals = torch.from_numpy(rng.standard_normal((3, ci.size)).astype(np.float32)).cuda()
        drp, dci = dev(rp), dev(ci)
        before = H.softmax_csr_float_batched(drp, vals, 0.3)
        assert H._known_longest_row(drp, 300, ci.size) is None
        plan = H.csr_plan(drp, dci, 300, 8192)
        assert plan.max_row == longest and H._known_longest_row(drp, 300, ci.size) == longest
        after = H.softmax_csr_float_batched(drp, vals, 0.3)
        assert torch.equal(before, after)
        assert torch.equal(H.softmax_csr_float(drp, vals[1], 0.3), after[1])
        sums = torch.zeros(3, 300, device="cuda").index_add_(
            1, torch.repeat_interleave(torch.arange(300, device="cuda"), torch.from_numpy(lens).cuda()), after)
        assert torch.allclose(sums[:, lens > 0], torch.ones_like(sums[:, lens > 0]), atol=1e-5)
