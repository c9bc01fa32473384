"""SDDMM and SpMM on the matrix cores for CSR operands made of 64 x 64 blocks, through the C ABI
(scorch_hip_sddmm_csr_blocked_f32, scorch_hip_spmm_csr_blocked_f32) and through the dispatch
that chooses them.

Values: relative Frobenius error <= 1e-5 against an fp64 recomputation, and agreement with the
oracle's fp32 restatement of the reference's loops (csrc/kernels.h:508-570, csrc/spmm.h:2007-2089)
at the tolerance the reference's own tests use.  Structure: the result's coordinates are bit-exact,
one entry per mask entry in mask order.
"""
import numpy as np
import pytest
import torch

from gpu_util import dev, host
from scorch_amd import graphs, native
from scorch_amd import scorch_ops_hip as H

pytestmark = pytest.mark.gpu

TOL = 1e-5


class blocked_path:
    def __init__(self, mode):
        self.mode = mode

    def __enter__(self):
        self.previous, H.BLOCKED_PATH = H.BLOCKED_PATH, self.mode

    def __exit__(self, *exc):
        H.BLOCKED_PATH = self.previous
        return False


def pattern(kind, M, n_cols, rng):
    i, j = np.arange(M)[:, None], np.arange(n_cols)[None, :]
    if kind == "blocks":
        active = rng.random((M // 64, n_cols // 64)) < 0.35
        active[0, 0] = True
        if M > 64:
            active[1, :] = False                       # a block row without blocks
        return np.kron(active, np.ones((64, 64), dtype=bool))
    if kind == "window":
        return np.abs(i - j) <= 90
    if kind == "causal":
        return j <= i
    if kind == "window_global":                        # one row and one column that hold everything
        m = np.abs(i - j) <= 40
        m[0, :] = True
        m[:, 0] = True
        return m
    if kind == "random30":
        return rng.random((M, n_cols)) < 0.3
    if kind == "random2":
        return rng.random((M, n_cols)) < 0.02
    raise ValueError(kind)


def csr_of(mask):
    row_ptr = np.zeros(mask.shape[0] + 1, dtype=np.int32)
    row_ptr[1:] = np.cumsum(mask.sum(axis=1))
    return row_ptr, np.nonzero(mask)[1].astype(np.int32)


def products(rp, ci, mask_vals, A, B, P, V):
    """(SDDMM values (H, nnz), row coordinates, SpMM result (H, M, N), plan) through the batched wrappers."""
    M, n_cols = len(rp) - 1, B.shape[1]
    pos, crd = dev(rp), dev(ci)
    idx = [[], [pos, crd]]
    first, _ = H.sddmm_csr_float_batched([M, n_cols], idx, dev(mask_vals), dev(A), dev(B))
    # (the pattern's first product: general kernel; what serves it from now on is decided when it comes back)
    out, rows = H.sddmm_csr_float_batched([M, n_cols], idx, dev(mask_vals), dev(A), dev(B))
    c = H.spmm_csr_float_batched([M, n_cols], idx, dev(P), dev(V))
    np.testing.assert_allclose(host(first), host(out), rtol=1e-4, atol=1e-4)
    return host(out), host(rows), host(c), pos._scorch_plan


def check_values(oracle, rp, ci, mask_vals, A, B, P, V, out, rows, c):
    ref_rows = oracle.rows_of(rp)
    assert rows.dtype == np.int32 and np.array_equal(rows, ref_rows)
    for h in range(A.shape[0]):
        ref64 = oracle.sddmm_fp64(ref_rows, ci, mask_vals, A[h], B[h])
        assert oracle.rel_fro(out[h], ref64) <= TOL
        np.testing.assert_allclose(out[h], oracle.sddmm_coo_f32(ref_rows, ci, mask_vals, A[h], B[h]), rtol=1e-3,
                                   atol=1e-3)
        assert oracle.rel_fro(c[h], oracle.spmm_fp64(rp, ci, P[h], V[h])) <= TOL
        np.testing.assert_allclose(c[h], oracle.spmm_csr_f32_v2(rp, ci, P[h], V[h]), rtol=1e-3, atol=1e-3)


def operands(rng, heads, M, n_cols, D, nnz):
    f = lambda *shape: rng.standard_normal(shape).astype(np.float32)
    return f(nnz), f(heads, M, D), f(heads, n_cols, D), f(heads, nnz), f(heads, n_cols, D)


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("kind", ["blocks", "window", "causal", "random30"])
def test_block_kernels_against_fp64(oracle, kind, D):
    rng = np.random.default_rng(D + len(kind))
    M = n_cols = 384
    rp, ci = csr_of(pattern(kind, M, n_cols, rng))
    mv, A, B, P, V = operands(rng, 3, M, n_cols, D, ci.size)
    out, rows, c, plan = products(rp, ci, mv, A, B, P, V)
    assert isinstance(plan.blocked, H.BlockedCsr)               # these masks go to the block kernels
    check_values(oracle, rp, ci, mv, A, B, P, V, out, rows, c)
    if kind == "blocks":
        assert not c[:, 64:128].any()                           # the block row without blocks: zero rows


@pytest.mark.parametrize("shape,heads", [((64, 64), 1), ((128, 640), 8), ((640, 128), 16), ((256, 192), 5)])
def test_rectangular_masks_and_head_counts(oracle, shape, heads):
    rng = np.random.default_rng(shape[0] + heads)
    M, n_cols = shape
    rp, ci = csr_of(pattern("random30", M, n_cols, rng))
    mv, A, B, P, V = operands(rng, heads, M, n_cols, 64, ci.size)
    out, rows, c, plan = products(rp, ci, mv, A, B, P, V)
    assert isinstance(plan.blocked, H.BlockedCsr)
    check_values(oracle, rp, ci, mv, A, B, P, V, out, rows, c)


@pytest.mark.parametrize("D", [32, 128])
def test_thinly_filled_blocks_when_forced(oracle, D):
    """Two stored entries in a hundred: every row of every block is partly stored, most words
    have one or two bits set, some rows of a block none."""
    rng = np.random.default_rng(D)
    M, n_cols = 320, 448
    rp, ci = csr_of(pattern("random2", M, n_cols, rng))
    mv, A, B, P, V = operands(rng, 2, M, n_cols, D, ci.size)
    with blocked_path("always"):
        out, rows, c, plan = products(rp, ci, mv, A, B, P, V)
    assert isinstance(plan.blocked, H.BlockedCsr) and plan.blocked.fill < 0.05
    check_values(oracle, rp, ci, mv, A, B, P, V, out, rows, c)
    out2, rows2, c2, plan2 = products(rp, ci, mv, A, B, P, V)   # left to itself: the general kernels
    assert plan2.blocked is False
    check_values(oracle, rp, ci, mv, A, B, P, V, out2, rows2, c2)


def test_what_goes_to_the_block_kernels():
    rng = np.random.default_rng(3)
    def second_use(pos, crd, M, n, D):
        plan = H.csr_plan(pos, crd, M, n)
        assert H._blocked(plan, pos, crd, M, n, D) is None or H.BLOCKED_PATH == "always"   # first product: not yet
        return H._blocked(plan, pos, crd, M, n, D)

    f = lambda kind, M, n, D=64: second_use(*[dev(x) for x in csr_of(pattern(kind, M, n, rng))], M, n, D)
    assert f("causal", 256, 256) is not None
    assert f("causal", 256, 256, D=48) is None                  # dense width without a kernel
    assert f("causal", 250, 256) is None                        # rows not a multiple of 64
    assert f("random2", 256, 256) is None                       # a graph, not a mask
    # between the thresholds of the widths: 0.13 of the positions stored
    m = rng.random((256, 256)) < 0.135
    pos, crd = (dev(x) for x in csr_of(m))
    plan = H.csr_plan(pos, crd, 256, 256)
    assert second_use(pos, crd, 256, 256, 128) is not None
    assert H._blocked(plan, pos, crd, 256, 256, 32) is None
    with blocked_path("off"):
        assert f("causal", 256, 256) is None
    # a row that holds everything among rows that hold a window: its block row goes out in stretches
    pos, crd = (dev(x) for x in csr_of(pattern("window_global", 1024, 1024, rng)))
    bl = second_use(pos, crd, 1024, 1024, 64)
    assert bl is not None and bl.longest_block_row == 16
    assert bl.spmm_split_rows.tolist() == [0, 0, 3, 0] and bl.n_spmm_slots == 3 and bl.n_spmm_items == 18
    # rows of similar length stay whole
    pos, crd = (dev(x) for x in csr_of(pattern("window", 1024, 1024, rng)))
    bl = second_use(pos, crd, 1024, 1024, 64)
    assert bl.n_spmm_slots == 0 and bl.n_spmm_items == 16


def test_unbalanced_mask_values(oracle):
    rng = np.random.default_rng(8)
    M = n_cols = 1024
    rp, ci = csr_of(pattern("window_global", M, n_cols, rng))
    mv, A, B, P, V = operands(rng, 2, M, n_cols, 32, ci.size)
    out, rows, c, plan = products(rp, ci, mv, A, B, P, V)
    assert isinstance(plan.blocked, H.BlockedCsr)
    check_values(oracle, rp, ci, mv, A, B, P, V, out, rows, c)


def test_rows_with_unordered_columns_keep_the_general_kernels(oracle):
    rng = np.random.default_rng(9)
    M = n_cols = 128
    rp, ci = csr_of(pattern("random30", M, n_cols, rng))
    ci = ci.copy()
    lo, hi = rp[5], rp[6]
    ci[lo:hi] = ci[lo:hi][::-1]                                 # one row stored backwards
    mv, A, B, P, V = operands(rng, 2, M, n_cols, 64, ci.size)
    out, rows, c, plan = products(rp, ci, mv, A, B, P, V)
    assert plan.blocked is False
    ref_rows = oracle.rows_of(rp)
    for h in range(2):
        assert oracle.rel_fro(out[h], oracle.sddmm_fp64(ref_rows, ci, mv, A[h], B[h])) <= TOL
        assert oracle.rel_fro(c[h], oracle.spmm_fp64(rp, ci, P[h], V[h])) <= TOL


def test_batched_equals_per_head_and_repeats_bit_for_bit():
    rng = np.random.default_rng(10)
    M = n_cols = 256
    rp, ci = csr_of(pattern("causal", M, n_cols, rng))
    mv, A, B, P, V = operands(rng, 4, M, n_cols, 64, ci.size)
    pos, crd = dev(rp), dev(ci)
    idx = [[], [pos, crd]]
    H.sddmm_csr_float_batched([M, n_cols], idx, dev(mv), dev(A), dev(B))       # (first product: general kernel)
    out, rows = H.sddmm_csr_float_batched([M, n_cols], idx, dev(mv), dev(A), dev(B))
    c = H.spmm_csr_float_batched([M, n_cols], idx, dev(P), dev(V))
    assert isinstance(pos._scorch_plan.blocked, H.BlockedCsr)
    out_again, rows_again = H.sddmm_csr_float_batched([M, n_cols], idx, dev(mv), dev(A), dev(B))
    assert torch.equal(out, out_again) and rows_again is rows    # (the coordinates are written once)
    assert torch.equal(c, H.spmm_csr_float_batched([M, n_cols], idx, dev(P), dev(V)))
    for h in range(4):
        one = H.sddmm_csr_float([M, n_cols], [M, n_cols], idx, dev(mv), [M, 64], [[], []], dev(A[h]).reshape(-1),
                                [n_cols, 64], [[], []], dev(B[h]).reshape(-1))
        assert torch.equal(one.storage.value, out[h])
        assert one.storage.index.mode_indices[1][0] is crd
        prod = H.spmm_csr_float_v2([M, 64], [M, n_cols], idx, dev(P[h]), [n_cols, 64], [[], []], dev(V[h]).reshape(-1))
        assert torch.equal(prod.storage.value.view(M, 64), c[h])


def test_sparse_attention_through_the_block_kernels(oracle):
    rng = np.random.default_rng(11)
    S, heads, D = 512, 4, 64
    mask = pattern("window", S, S, rng)
    rp, ci = csr_of(mask)
    q, k, v = (rng.standard_normal((heads, S, D)).astype(np.float32) for _ in range(3))
    pos, crd = dev(rp), dev(ci)
    H.sparse_attention_csr(pos, crd, dev(q), dev(k), dev(v), D ** -0.5)
    got = host(H.sparse_attention_csr(pos, crd, dev(q), dev(k), dev(v), D ** -0.5))
    assert isinstance(pos._scorch_plan.blocked, H.BlockedCsr)
    for h in range(heads):
        assert oracle.rel_fro(got[h], oracle.attention_dense_fp64(q[h], k[h], v[h], mask, D ** -0.5)) <= TOL


def test_recorded_step_replays_the_block_kernels(oracle):
    rng = np.random.default_rng(12)
    S, heads, D = 256, 2, 32
    mask = pattern("causal", S, S, rng)
    rp, ci = csr_of(mask)
    pos, crd = dev(rp), dev(ci)
    q, k, v = (torch.zeros(heads, S, D, device="cuda") for _ in range(3))
    step = graphs.capture(lambda: H.sparse_attention_csr(pos, crd, q, k, v, D ** -0.5))
    assert isinstance(pos._scorch_plan.blocked, H.BlockedCsr)
    for seed in range(3):
        qh, kh, vh = (np.random.default_rng(100 + seed).standard_normal((3, heads, S, D)).astype(np.float32))
        q.copy_(dev(qh)), k.copy_(dev(kh)), v.copy_(dev(vh))
        got = host(step.replay())
        torch.cuda.synchronize()
        assert np.array_equal(got, host(H.sparse_attention_csr(pos, crd, q, k, v, D ** -0.5)))
        assert oracle.rel_fro(got[1], oracle.attention_dense_fp64(qh[1], kh[1], vh[1], mask, D ** -0.5)) <= TOL


def test_entry_points_refuse_what_they_do_not_serve():
    L = native.lib()
    z = torch.zeros(64 * 64, device="cuda")
    items = torch.tensor([0, 0, 1, 0], dtype=torch.int32, device="cuda")
    col = torch.zeros(1, dtype=torch.int32, device="cuda")
    words = torch.full((64,), -1, dtype=torch.int64, device="cuda")
    off = (torch.arange(64, dtype=torch.int32, device="cuda") * 64)
    args = lambda M, n, K: (1, M, n, K, 4096, 1, col.data_ptr(), words.data_ptr(), off.data_ptr(), 1, items.data_ptr(),
                            z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(), None, None)
    assert L.scorch_hip_sddmm_csr_blocked_f32(*args(64, 64, 48)) == native.EUNSUPPORTED
    assert "32, 64 or 128" in native.last_error()
    assert L.scorch_hip_sddmm_csr_blocked_f32(*args(60, 64, 64)) == native.EUNSUPPORTED
    assert L.scorch_hip_sddmm_csr_blocked_f32(*args(64, 64, 64)) == 0
    torch.cuda.synchronize()
    c = torch.zeros(128 * 64, device="cuda")
    spmm = lambda n_items, n_split=0, n_slots=0, ws=None, ws_bytes=0: L.scorch_hip_spmm_csr_blocked_f32(
        1, 128, 64, 64, 4096, 1, col.data_ptr(), words.data_ptr(), off.data_ptr(), None, n_items, items.data_ptr(),
        n_split, items.data_ptr() if n_split else None, n_slots, z.data_ptr(), z.data_ptr(), c.data_ptr(), ws,
        ws_bytes, None)
    assert spmm(1) == native.EINVAL and "every block row" in native.last_error()
    assert spmm(2, 1, 0) == native.EINVAL                        # split rows without slots
    assert spmm(2, 1, 2) == native.EWORKSPACE and "workspace" in native.last_error()
    assert L.scorch_hip_spmm_csr_blocked_workspace_bytes(3, 2, 64) == 3 * 2 * 64 * 64 * 4


def test_a_mask_of_ones_is_not_read(oracle):
    rng = np.random.default_rng(13)
    M = n_cols = 256
    rp, ci = csr_of(pattern("causal", M, n_cols, rng))
    _, A, B, _, _ = operands(rng, 2, M, n_cols, 64, ci.size)
    pos, crd, a, b = dev(rp), dev(ci), dev(A), dev(B)
    idx = [[], [pos, crd]]
    ones = torch.ones(ci.size, device="cuda")
    general, _ = H.sddmm_csr_float_batched([M, n_cols], idx, ones, a, b)    # the pattern's first product,
    assert ones._scorch_ones[1] is None                                     # first sight of the values: read
    first, _ = H.sddmm_csr_float_batched([M, n_cols], idx, ones, a, b)      # back unchanged: looked at, all 1
    assert isinstance(pos._scorch_plan.blocked, H.BlockedCsr)
    np.testing.assert_allclose(host(general), host(first), rtol=1e-4, atol=1e-4)
    assert ones._scorch_ones[1] is True
    second, _ = H.sddmm_csr_float_batched([M, n_cols], idx, ones, a, b)
    third, _ = H.sddmm_csr_float_batched([M, n_cols], idx, None, a, b)
    assert torch.equal(first, second) and torch.equal(first, third)
    ref_rows = oracle.rows_of(rp)
    assert oracle.rel_fro(host(first[1]), oracle.sddmm_fp64(ref_rows, ci, np.ones(ci.size, np.float32), A[1], B[1])) <= TOL
    ones[7] = -2.0                                                           # written to: looked at again
    changed, _ = H.sddmm_csr_float_batched([M, n_cols], idx, ones, a, b)
    again, _ = H.sddmm_csr_float_batched([M, n_cols], idx, ones, a, b)
    assert ones._scorch_ones[1] is False and torch.equal(changed, again)
    expect = first.clone()
    expect[:, 7] *= -2.0
    assert torch.equal(changed, expect)


def test_rows_of_the_dense_operand_that_no_entry_refers_to_are_not_used(oracle):
    """Columns the mask leaves out altogether (the padding of a batch): whatever the dense operands
    hold there -- NaN here -- stays out of both products, as with the general kernels."""
    rng = np.random.default_rng(14)
    M = n_cols = 256
    mask = pattern("causal", M, n_cols, rng)
    padded = np.r_[40:64, 130:131, 200:256]
    mask[:, padded] = False
    rp, ci = csr_of(mask)
    mv, A, B, P, V = operands(rng, 2, M, n_cols, 64, ci.size)
    B_bad, V_bad = B.copy(), V.copy()
    B_bad[:, padded] = np.nan
    V_bad[:, padded] = np.nan
    out, rows, c, plan = products(rp, ci, mv, A, B_bad, P, V_bad)
    assert isinstance(plan.blocked, H.BlockedCsr)
    assert np.isfinite(out).all() and np.isfinite(c).all()
    check_values(oracle, rp, ci, mv, A, B, P, V, out, rows, c)


def test_coordinate_mask_made_of_blocks(oracle):
    """The reference's prebuilt SDDMM takes a coordinate mask (csrc/kernels.h:508-570): one made
    of blocks, in row-major order, goes to the block kernel once it has come back; the result
    carries the mask's own index tensors either way."""
    rng = np.random.default_rng(15)
    M, n_cols, K = 256, 320, 64
    mask = pattern("random30", M, n_cols, rng)
    rp, ci = csr_of(mask)
    rows_np = oracle.rows_of(rp)
    mv = rng.standard_normal(ci.size).astype(np.float32)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((n_cols, K)).astype(np.float32)
    r, c, v, a, b = dev(rows_np), dev(ci), dev(mv), dev(A).reshape(-1), dev(B).reshape(-1)
    call = lambda: H.sddmm_coo_float_prebuilt([M, n_cols], [M, n_cols], [[r], [c]], v, [M, K], [[], []], a,
                                              [n_cols, K], [[], []], b)
    ref64 = oracle.sddmm_fp64(rows_np, ci, mv, A, B)
    first = call()                                       # general kernel
    assert r._scorch_coo_pos[1] is None
    second = call()                                      # the mask has come back: by blocks from here on
    assert isinstance(r._scorch_coo_pos[1], torch.Tensor) and np.array_equal(host(r._scorch_coo_pos[1]), rp)
    assert isinstance(r._scorch_coo_pos[1]._scorch_plan.blocked, H.BlockedCsr)
    third = call()
    for out in (first, second, third):
        assert out.storage.index.mode_indices[0][0] is r and out.storage.index.mode_indices[1][0] is c
        assert oracle.rel_fro(host(out.storage.value), ref64) <= TOL
    assert torch.equal(second.storage.value, third.storage.value)
    assert not torch.equal(first.storage.value, second.storage.value)      # (another order of the fp32 sums)
    # coordinates that are not in row order keep the general kernel
    perm = rng.permutation(ci.size)
    r2, c2, v2 = dev(rows_np[perm]), dev(ci[perm]), dev(mv[perm])
    for _ in range(3):
        out = H.sddmm_coo_float_prebuilt([M, n_cols], [M, n_cols], [[r2], [c2]], v2, [M, K], [[], []], a,
                                         [n_cols, K], [[], []], b)
    assert r2._scorch_coo_pos[1] is False
    assert oracle.rel_fro(host(out.storage.value), ref64[perm]) <= TOL


def test_through_matmul_and_einsum():
    """The reference's own calls (src/scorch/ops.py:248-372, 396-423) with a mask that is kept
    across calls, as its attention benchmark keeps it (bench/bench_sparse_transformer.py:236,357)."""
    import scorch_amd as scorch
    torch.manual_seed(16)
    S, D = 256, 32
    dense_mask = torch.tril(torch.ones(S, S))
    mask = scorch.STensor.from_csr(dense_mask.to_sparse_csr()).to("cuda")
    q, k, v = (torch.randn(S, D, device="cuda") for _ in range(3))
    live = dense_mask.bool().cuda()
    want_scores = (q.double() @ k.double().T)[live]
    probs = scorch.STensor.from_csr(torch.rand(S, S).tril().to_sparse_csr()).to("cuda")
    want_out = probs.to_torch(in_place=False).to_dense().double() @ v.double()
    for call in range(3):
        scores = scorch.einsum("ij,ik,jk->ij", mask, q, k)
        assert ((scores.values.double() - want_scores).norm() / want_scores.norm()).item() <= TOL
        out = scorch.matmul(probs, v)
        assert ((out.double() - want_out).norm() / want_out.norm()).item() <= TOL
    for operand in (mask, probs):
        assert isinstance(operand.index.mode_indices[1][0]._scorch_plan.blocked, H.BlockedCsr)
