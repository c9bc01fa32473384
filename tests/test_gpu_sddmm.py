"""SDDMM on the MI355X through the C ABI: coordinate and CSR masks.

Values: relative Frobenius error <= 1e-5 against an fp64 recomputation.
Structure: the output coordinates are bit-exact -- for a coordinate mask the
mask's own index tensors come back; for a CSR mask the result is the
coordinate list (row of each entry, col_idx) in mask order, one entry per mask
entry, explicit zeros kept.
"""
import numpy as np
import pytest
import torch

from conftest import random_csr
from gpu_util import dev, hip_sddmm_coo, hip_sddmm_csr, host
from scorch_amd import native
from scorch_amd import scorch_ops_hip as H
from scorch_amd import workloads

pytestmark = pytest.mark.gpu

TOL = 1e-5
SDDMM_CASES = ["sddmm_16_8", "sddmm_64_32", "sddmm_128_16", "sddmm_256_64", "sddmm_40_16", "sddmm_rect_k13"]


@pytest.mark.parametrize("name", SDDMM_CASES)
def test_golden_coo(golden, oracle, name):
    c = golden.case(name)
    shape = (c["A"].shape[0], c["B"].shape[0])
    got = hip_sddmm_coo(c["row_idx"], c["col_idx"], c["vals"], c["A"], c["B"], shape)
    ref64 = oracle.sddmm_fp64(c["row_idx"], c["col_idx"], c["vals"], c["A"], c["B"])
    assert oracle.rel_fro(got, ref64) <= TOL
    np.testing.assert_allclose(got, c["out_val"], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("name", SDDMM_CASES)
def test_golden_csr(golden, oracle, name):
    c = golden.case(name)
    shape = (c["A"].shape[0], c["B"].shape[0])
    row, col, val = hip_sddmm_csr(c["row_ptr"], c["col_idx"], c["vals"], c["A"], c["B"], shape)
    assert row.dtype == np.int32 and np.array_equal(row, c["out_row"]) and np.array_equal(col, c["out_col"])
    assert val.size == c["vals"].size
    np.testing.assert_allclose(val, c["out_val"], rtol=1e-4, atol=1e-5)
    assert (val[c["vals"] == 0] == 0).all()


# K chosen to hit every group width (4..64 lanes per entry), the scalar path (K % 4 != 0) and K > 256
@pytest.mark.parametrize("K", [1, 2, 5, 8, 13, 16, 32, 64, 65, 96, 128, 200, 256, 257, 260, 512, 1024, 1100, 1101])
def test_inner_dimensions(oracle, K):
    rng = np.random.default_rng(K)
    rp, ci, s = random_csr(rng, 211, 157, 0.07, empty_rows=(0, 7, 210))
    rows = oracle.rows_of(rp)
    A = rng.standard_normal((211, K)).astype(np.float32)
    B = rng.standard_normal((157, K)).astype(np.float32)
    ref64 = oracle.sddmm_fp64(rows, ci, s, A, B)
    coo = hip_sddmm_coo(rows, ci, s, A, B, (211, 157))
    r, c, csr = hip_sddmm_csr(rp, ci, s, A, B, (211, 157))
    assert oracle.rel_fro(coo, ref64) <= TOL and oracle.rel_fro(csr, ref64) <= TOL
    assert np.array_equal(coo, csr)                      # same arithmetic, same order
    assert np.array_equal(r, rows) and np.array_equal(c, ci)
    np.testing.assert_allclose(coo, oracle.sddmm_coo_f32(rows, ci, s, A, B), rtol=1e-4, atol=1e-5)


def test_coo_entries_in_any_order(oracle):
    rng = np.random.default_rng(5)
    rp, ci, s = random_csr(rng, 300, 300, 0.05)
    rows = oracle.rows_of(rp)
    A = rng.standard_normal((300, 64)).astype(np.float32)
    B = rng.standard_normal((300, 64)).astype(np.float32)
    perm = rng.permutation(s.size)
    got = hip_sddmm_coo(rows[perm], ci[perm], s[perm], A, B, (300, 300))
    assert oracle.rel_fro(got, oracle.sddmm_fp64(rows[perm], ci[perm], s[perm], A, B)) <= TOL


def test_csr_rows_with_long_empty_stretches(oracle):
    lens = np.zeros(70000, np.int64)
    lens[[5, 30000, 30001, 69999]] = [700, 3, 1, 900]
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    rng = np.random.default_rng(6)
    ci = rng.integers(0, 1000, int(rp[-1])).astype(np.int32)
    s = rng.uniform(-1, 1, ci.size).astype(np.float32)
    A = rng.standard_normal((70000, 16)).astype(np.float32)
    B = rng.standard_normal((1000, 16)).astype(np.float32)
    r, c, val = hip_sddmm_csr(rp, ci, s, A, B, (70000, 1000))
    rows = oracle.rows_of(rp)
    assert np.array_equal(r, rows)
    assert oracle.rel_fro(val, oracle.sddmm_fp64(rows, ci, s, A, B)) <= TOL


@pytest.mark.parametrize("K", [8, 64])
def test_dense_operands_at_odd_element_offsets(oracle, K):
    """A and B only 4-byte aligned (views one element into their buffers): K is a
    multiple of four, but the 16-byte loads are not allowed."""
    rng = np.random.default_rng(60 + K)
    rp, ci, s = random_csr(rng, 150, 120, 0.1, dtype=np.float32)
    A = rng.standard_normal((150, K)).astype(np.float32)
    B = rng.standard_normal((120, K)).astype(np.float32)
    big_a, big_b = torch.empty(150 * K + 1, device="cuda"), torch.empty(120 * K + 1, device="cuda")
    big_a[1:].copy_(dev(A).reshape(-1))
    big_b[1:].copy_(dev(B).reshape(-1))
    assert big_a[1:].data_ptr() % 16 == 4
    out = H.sddmm_csr_float([150, 120], [150, 120], [[], [dev(rp), dev(ci)]], dev(s), [150, K], [[], []],
                            big_a[1:], [120, K], [[], []], big_b[1:])
    rows = oracle.rows_of(rp)
    want = oracle.sddmm_fp64(rows, ci, s, A, B)
    assert oracle.rel_fro(host(out.storage.value), want) <= TOL


def test_closed_forms():
    n = 64
    eye = np.eye(n, dtype=np.float32)
    rows, cols = np.nonzero(np.ones((n, n)))
    out = hip_sddmm_coo(rows.astype(np.int32), cols.astype(np.int32), np.ones(n * n, np.float32), eye, eye, (n, n))
    assert np.array_equal(out.reshape(n, n), eye)
    empty = hip_sddmm_coo(np.zeros(0, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), eye, eye, (n, n))
    assert empty.size == 0


def test_row_indices_kernel_matches_sddmm_rows(oracle):
    w = workloads.gcn_powerlaw(M=30000, N=4, seed=8, max_degree=4000)
    rows = H.csr_row_indices(dev(w["row_ptr"]), int(w["col_idx"].size))
    assert np.array_equal(host(rows), oracle.rows_of(w["row_ptr"]))


def test_full_size_workload():
    """65,536 x 65,536 mask with 64 entries per row, K = 64: values against an
    fp64 gather-and-dot on the device, coordinates bit-exact."""
    w = workloads.sddmm_uniform(unit_mask=False)
    M, n_cols, K = w["M"], w["n_cols"], w["K"]
    rp, ci, s = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"])
    A, B = dev(w["A"]), dev(w["B"])
    out = H.sddmm_csr_float([M, n_cols], [M, n_cols], [[], [rp, ci]], s, [M, K], [[], []], A.reshape(-1),
                            [n_cols, K], [[], []], B.reshape(-1))
    rows_ref = dev(w["row_idx"])
    assert torch.equal(out.storage.index.mode_indices[0][0], rows_ref)
    assert out.storage.index.mode_indices[1][0] is ci
    ref64 = torch.empty(s.numel(), dtype=torch.float64, device="cuda")
    step = 1 << 20
    for p0 in range(0, s.numel(), step):
        sl = slice(p0, p0 + step)
        ref64[sl] = (A[rows_ref[sl].long()].double() * B[ci[sl].long()].double()).sum(1) * s[sl].double()
    err = (torch.linalg.norm(out.storage.value.double() - ref64) / torch.linalg.norm(ref64)).item()
    assert err <= TOL, err
    coo = H.sddmm_coo_float_prebuilt([M, n_cols], [M, n_cols], [[rows_ref], [ci]], s, [M, K], [[], []],
                                     A.reshape(-1), [n_cols, K], [[], []], B.reshape(-1))
    assert torch.equal(coo.storage.value, out.storage.value)


# ---- a reused mask: its entries listed per XCD ---------------------------------------------------
@pytest.mark.parametrize("K", [8, 32, 64, 100, 256])
def test_listed_path_equals_the_plain_one(K, monkeypatch):
    """The same products computed list by list (one list per XCD, by column range): bit for bit
    the plain kernel's values and row coordinates, for one product and for a batch over the mask."""
    from scorch_amd import scorch_ops_hip as H
    w = workloads.sddmm_uniform(M=3000, n_cols=2500, per_row=40, K=K, seed=K, unit_mask=False)
    rp, ci, sv = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"])
    A, B = dev(w["A"]), dev(w["B"])
    call = lambda: H.sddmm_csr_float([3000, 2500], [3000, 2500], [[], [rp, ci]], sv, [3000, K], [[], []],
                                     A.reshape(-1), [2500, K], [[], []], B.reshape(-1))
    monkeypatch.setattr(H, "SDDMM_PATH", "plain")
    plain = call()
    monkeypatch.setattr(H, "SDDMM_PATH", "listed")
    listed = call()
    assert rp._scorch_plan.sddmm_lists is not None
    assert torch.equal(plain.storage.value, listed.storage.value)
    assert torch.equal(plain.storage.index.mode_indices[0][0], listed.storage.index.mode_indices[0][0])
    A3 = torch.stack([A, A * 2, A - 1])
    B3 = torch.stack([B, B + 1, B * 0.5])
    got, rows = H.sddmm_csr_float_batched([3000, 2500], [[], [rp, ci]], sv, A3, B3)
    monkeypatch.setattr(H, "SDDMM_PATH", "plain")
    want, rows_plain = H.sddmm_csr_float_batched([3000, 2500], [[], [rp, ci]], sv, A3, B3)
    assert torch.equal(got, want) and torch.equal(rows, rows_plain)


def test_listed_path_with_ragged_rows_and_empty_column_ranges(oracle, monkeypatch):
    """Rows of very different lengths, empty rows, and all columns in the first eighth but one."""
    from scorch_amd import scorch_ops_hip as H
    rng = np.random.default_rng(31)
    lens = rng.integers(0, 50, 700); lens[[0, 350]] = [3000, 0]
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = rng.integers(0, 500, int(rp[-1])).astype(np.int32)
    ci[-1] = 3999
    sv = rng.uniform(-1, 1, ci.size).astype(np.float32)
    A = rng.standard_normal((700, 48)).astype(np.float32)
    B = rng.standard_normal((4000, 48)).astype(np.float32)
    monkeypatch.setattr(H, "SDDMM_PATH", "listed")
    rows, cols, vals = hip_sddmm_csr(rp, ci, sv, A, B, (700, 4000))
    want_rows = np.repeat(np.arange(700, dtype=np.int32), lens)
    assert np.array_equal(rows, want_rows) and np.array_equal(cols, ci)
    assert oracle.rel_fro(vals, oracle.sddmm_fp64(want_rows, ci, sv, A, B)) <= 1e-5


def test_auto_builds_the_lists_on_the_second_product_at_full_size(oracle):
    """65,536^2, 64 per row, K = 64: B is 16 MB, beyond one L2 and within the eight together."""
    from scorch_amd import scorch_ops_hip as H
    w = workloads.sddmm_uniform()
    M, n_cols, K = w["M"], w["n_cols"], w["K"]
    rp, ci, sv = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"])
    A, B = dev(w["A"]).reshape(-1), dev(w["B"]).reshape(-1)
    call = lambda: H.sddmm_csr_float([M, n_cols], [M, n_cols], [[], [rp, ci]], sv, [M, K], [[], []], A, [n_cols, K],
                                     [[], []], B).storage.value
    first = call()
    assert rp._scorch_plan.sddmm_lists is None
    second = call()
    assert rp._scorch_plan.sddmm_lists is not None
    assert torch.equal(first, second) and torch.equal(second, call())


@pytest.mark.parametrize("mask_format", ["ds", "oo"])
def test_einsum_with_dense_torch_operands_takes_the_direct_route(mask_format):
    """scorch.einsum("ij,ik,jk->ij", mask, Q, K) with torch tensors for Q and K: same entries,
    same order, same bits as with the operands wrapped in STensors first."""
    import scorch_amd as scorch
    from scorch_amd import STensor
    rng = np.random.default_rng(12)
    mask = ((rng.random((70, 90)) < 0.15) * rng.standard_normal((70, 90))).astype(np.float32)
    S = STensor.from_torch(torch.from_numpy(mask).to_sparse_csr()).to("cuda")
    if mask_format == "oo":
        S = S.to_sparse("oo")
    Q = torch.from_numpy(rng.standard_normal((70, 40)).astype(np.float32)).cuda()
    K = torch.from_numpy(rng.standard_normal((90, 40)).astype(np.float32)).cuda()
    direct = scorch.einsum("ij,ik,jk->ij", S, Q, K)
    general = scorch.einsum("ij,ik,jk->ij", S, STensor.from_torch(Q), STensor.from_torch(K))
    assert str(direct.format) == str(general.format) == "o,o"
    for a, b in zip(direct.index.mode_indices, general.index.mode_indices):
        assert torch.equal(a[0], b[0])
    assert torch.equal(direct.values, general.values)
    want = (Q.double() @ K.double().T).cpu().numpy() * mask
    np.testing.assert_allclose(host(direct.to_torch()), want, rtol=1e-4, atol=1e-5)
    times = {}
    again = scorch.einsum("ab,ac,bc->ab", S, Q, K, time_dict=times)      # other index names, same expression
    assert torch.equal(again.values, direct.values) and times["eval_time"] > 0


def test_row_coordinates_of_a_planned_mask_are_written_once(oracle):
    """The row coordinates of a CSR mask's SDDMM result depend on the pattern only: the first
    product writes them, later ones hand out the same tensor (as the reference hands out a
    coordinate mask's own index tensors), a changed pattern gets new ones."""
    rng = np.random.default_rng(61)
    M, C, K = 300, 200, 32
    rp, ci, s = random_csr(rng, M, C, 0.1)
    t_rp, t_ci, t_s = dev(rp), dev(ci), dev(s)
    call = lambda A, B: H.sddmm_csr_float([M, C], [M, C], [[], [t_rp, t_ci]], t_s, [M, K], [[], []], A.reshape(-1),
                                          [C, K], [[], []], B.reshape(-1))
    A1, B1 = (torch.randn(n, K, device="cuda") for n in (M, C))
    A2, B2 = (torch.randn(n, K, device="cuda") for n in (M, C))
    first, second = call(A1, B1), call(A2, B2)
    rows1, rows2 = first.storage.index.mode_indices[0][0], second.storage.index.mode_indices[0][0]
    assert rows2 is rows1 and np.array_equal(host(rows1), oracle.rows_of(rp))
    ref = oracle.sddmm_fp64(oracle.rows_of(rp), ci, s, host(A2), host(B2))
    assert oracle.rel_fro(host(second.storage.value), ref) <= 1e-5
    t_ci.copy_(torch.roll(t_ci, 1))                       # (any write: the plan no longer holds)
    t_ci.copy_(dev(ci))
    third = call(A1, B1)
    rows3 = third.storage.index.mode_indices[0][0]
    assert rows3 is not rows1 and torch.equal(rows3, rows1)
    assert torch.equal(third.storage.value, first.storage.value)


@pytest.mark.parametrize("path", ["plain", "listed", "coo"])
def test_a_mask_without_a_value_array_is_a_mask_of_ones(oracle, monkeypatch, path):
    """mask_vals = NULL through the C ABI (what the wrappers pass once a mask's values are known to
    be all 1): bit for bit the result with an array of ones, and the fp64 recomputation."""
    from scorch_amd import native
    from scorch_amd import scorch_ops_hip as H
    w = workloads.sddmm_uniform(M=1500, n_cols=2200, per_row=30, K=48, seed=9, unit_mask=True)
    M, n_cols, K, nnz = 1500, 2200, 48, int(w["col_idx"].size)
    rp, ci, rows = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["row_idx"])
    ones = torch.ones(nnz, device="cuda")
    A, B = dev(w["A"]).reshape(-1), dev(w["B"]).reshape(-1)
    L, stream = native.lib(), torch.cuda.current_stream().cuda_stream
    lists = None
    if path == "listed":
        lists = torch.empty(L.scorch_hip_sddmm_csr_lists_bytes(nnz), dtype=torch.uint8, device="cuda")
        native.check(L.scorch_hip_sddmm_csr_lists(M, n_cols, nnz, rp.data_ptr(), ci.data_ptr(), lists.data_ptr(),
                                                  lists.numel(), stream))

    def run(values):
        out = torch.full((nnz,), float("nan"), device="cuda")
        v = values.data_ptr() if values is not None else None
        if path == "plain":
            rc = L.scorch_hip_sddmm_csr_f32(M, n_cols, K, nnz, rp.data_ptr(), ci.data_ptr(), v, A.data_ptr(),
                                            B.data_ptr(), out.data_ptr(), None, stream)
        elif path == "listed":
            rc = L.scorch_hip_sddmm_csr_listed_f32(1, M, n_cols, K, nnz, lists.data_ptr(), lists.numel(), v, None,
                                                   A.data_ptr(), B.data_ptr(), out.data_ptr(), None, stream)
        else:
            rc = L.scorch_hip_sddmm_coo_f32(M, n_cols, K, nnz, rows.data_ptr(), ci.data_ptr(), v, A.data_ptr(),
                                            B.data_ptr(), out.data_ptr(), stream)
        native.check(rc)
        return out

    with_ones, without = run(ones), run(None)
    assert torch.equal(with_ones, without)
    assert oracle.rel_fro(host(without), oracle.sddmm_fp64(w["row_idx"], w["col_idx"], w["vals"], w["A"], w["B"])) <= 1e-5
    # through the wrappers: the verdict is reached when the same value tensor comes back unchanged
    monkeypatch.setattr(H, "SDDMM_PATH", "plain" if path == "coo" else path)
    if path == "coo":
        call = lambda: H.sddmm_coo_float_prebuilt([M, n_cols], [M, n_cols], [[rows], [ci]], ones, [M, K], [[], []], A,
                                                  [n_cols, K], [[], []], B).storage.value
    else:
        call = lambda: H.sddmm_csr_float([M, n_cols], [M, n_cols], [[], [rp, ci]], ones, [M, K], [[], []], A,
                                         [n_cols, K], [[], []], B).storage.value
    results = [call() for _ in range(3)]
    assert ones._scorch_ones[1] is True and all(torch.equal(r, with_ones) for r in results)
    ones[11] = 3.0                                            # no longer a mask of ones
    changed = call()
    expect = with_ones.clone()
    expect[11] *= 3.0
    assert torch.equal(changed, expect)


def test_values_differ_kernel():
    """What decides that a mask's values need not be read: 0 only when every value is the one asked about."""
    L = native.lib()
    flag = torch.full((2,), 7, dtype=torch.int32, device="cuda")

    def differ(vals, value=1.0):
        flag.fill_(7)
        native.check(L.scorch_hip_values_differ_f32(vals.numel(), vals.data_ptr(), value, flag.data_ptr(),
                                                    torch.cuda.current_stream().cuda_stream))
        got = flag.tolist()
        assert got[1] == 7
        return got[0]

    for n in (0, 1, 63, 64, 4097, 3_000_001):
        ones = torch.ones(n, device="cuda")
        assert differ(ones) == 0, n
        assert differ(ones, 2.0) == (1 if n else 0), n
        if n:
            for at in {0, n // 2, n - 1}:
                v = ones.clone()
                v[at] = 1.0000001
                assert differ(v) == 1, (n, at)
                v[at] = float("nan")
                assert differ(v) == 1, (n, at)


def test_mask_values_in_list_order(oracle, monkeypatch):
    """A mask whose values are not all ones: on its third product (seen, seen again unchanged,
    found not to be ones) the listed kernel reads a copy of the values in the order of its
    lists.  Same bits as the scattered reads; dropped when the values are written to; never made
    for a volatile tensor."""
    w = workloads.sddmm_uniform(M=4096, n_cols=65_536, per_row=80, K=32, seed=12, unit_mask=False)
    M, n_cols, K = w["M"], w["n_cols"], w["K"]
    rp, ci, vals, A, B = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"]), dev(w["A"]).reshape(-1), dev(w["B"]).reshape(-1)
    monkeypatch.setattr(H, "SDDMM_PATH", "listed")
    call = lambda v: H.sddmm_csr_float([M, n_cols], [M, n_cols], [[], [rp, ci]], v, [M, K], [[], []], A, [n_cols, K],
                                       [[], []], B).storage.value
    want = oracle.sddmm_fp64(w["row_idx"], w["col_idx"], w["vals"], w["A"], w["B"])
    first = call(vals)
    assert getattr(vals, "_scorch_listed", None) is None
    second = call(vals)                                   # the verdict: not all ones
    third = call(vals)                                    # ... and the copy
    assert vals._scorch_listed[2].numel() == vals.numel()
    fourth = call(vals)
    assert torch.equal(first, second) and torch.equal(first, third) and torch.equal(first, fourth)
    assert oracle.rel_fro(host(third), want) <= 1e-5
    # the copy holds what the lists say it holds
    L = native.lib()
    plan = rp._scorch_plan
    listed = torch.empty_like(vals)
    native.check(L.scorch_hip_sddmm_csr_list_values_f32(vals.numel(), plan.sddmm_lists.data_ptr(), plan.sddmm_lists.numel(),
                                                        vals.data_ptr(), listed.data_ptr(),
                                                        torch.cuda.current_stream().cuda_stream))
    assert torch.equal(listed, vals._scorch_listed[2])
    assert torch.equal(torch.sort(listed).values, torch.sort(vals).values)
    # new values: the copy is dropped with the version counter, and made again two products later
    vals.mul_(-2.0)
    assert torch.equal(call(vals), first * -2.0)
    assert torch.equal(call(vals), first * -2.0) and torch.equal(call(vals), first * -2.0)
    assert vals._scorch_listed[0] == H._stamp(vals)
    # a write PyTorch does not see: forget() drops the copy
    vals.data.mul_(0.5)
    H.forget(vals)
    assert getattr(vals, "_scorch_listed", None) is None
    assert torch.equal(call(vals), first * -1.0)
    # volatile values never get a copy
    other = vals.clone()
    H.mark_volatile(other)
    for _ in range(4):
        assert torch.equal(call(other), first * -1.0)
    assert getattr(other, "_scorch_listed", None) is None
