"""What is computed once per operand: the inspection of a CSR index (validation,
longest row), the chunk boundaries of the merge-path kernels, and the column-tile
copy of a wide dense operand -- and the dispatch that follows from them."""
import numpy as np
import pytest
import torch

from conftest import random_csr
from gpu_util import dev, hip_spmm, host, spmm_path
from scorch_amd import native, workloads
from scorch_amd import scorch_ops_hip as H

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _inspect(rp, ci, n_cols):
    report = torch.full((H.INSPECT_REPORT_INTS + 1,), -7, dtype=torch.int32, device="cuda")
    native.check(native.lib().scorch_hip_csr_inspect(rp.numel() - 1, n_cols, ci.numel(), rp.data_ptr(), ci.data_ptr(),
                                                     report.data_ptr(), torch.cuda.current_stream().cuda_stream))
    report = report.tolist()
    assert report[6:] == [0, 0, -7]              # reserved fields cleared, nothing written past the report
    return report[:4]


def test_inspection_report():
    w = workloads.gcn_powerlaw(M=30_000, N=1, seed=5, max_degree=7000)
    rp, ci = dev(w["row_ptr"]), dev(w["col_idx"])
    lens = np.diff(w["row_ptr"])
    assert _inspect(rp, ci, 30_000) == [0, 0, int(lens.max()), int((lens == 0).sum())]
    lens = np.array([0, 3, 0, 0, 5, 0], np.int64)
    rp = dev(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32))
    ci = dev(np.array([0, 1, 2, 0, 1, 2, 3, 9], np.int32))
    assert _inspect(rp, ci, 10) == [0, 0, 5, 4]
    assert _inspect(rp, ci, 9) == [0, 1, 5, 4]                       # column 9 of 9
    assert _inspect(rp, dev(np.array([0, 1, 2, 0, -1, 2, 3, 8], np.int32)), 9)[1] == 1
    assert _inspect(dev(np.array([1, 3, 3, 3, 8, 8, 8], np.int32)), ci, 10)[0] == 1       # starts at 1
    assert _inspect(dev(np.array([0, 3, 3, 3, 8, 8, 7], np.int32)), ci, 10)[0] == 1       # ends at 7, decreases
    assert _inspect(dev(np.array([0, 3, 2, 3, 8, 8, 8], np.int32)), ci, 10)[0] == 1       # decreases inside
    assert _inspect(dev(np.zeros(1, np.int32)), dev(np.zeros(0, np.int32)), 4) == [0, 0, 0, 0]   # no rows


@pytest.mark.parametrize("symbol", ["spmm_csr_float_v2", "prebuilt_spmv_csr_f32", "prebuilt_spmspm_csr_f32",
                                    "sddmm_csr_float"])
def test_malformed_operands_are_refused_before_any_kernel_reads_them(symbol):
    """A column index beyond K, a row pointer that decreases or does not end at nnz: ValueError
    from the inspection, not a memory fault from the kernel."""
    good_rp = np.array([0, 2, 2, 5], np.int32)
    good_ci = np.array([0, 3, 1, 2, 3], np.int32)
    vals = dev(np.ones(5, np.float32))

    def call(rp, ci):
        csr = [[], [dev(rp), dev(ci)]]
        if symbol == "spmm_csr_float_v2":
            return H.spmm_csr_float_v2([3, 8], [3, 4], csr, vals, [4, 8], [[], []], dev(np.ones(32, np.float32)))
        if symbol == "prebuilt_spmv_csr_f32":
            return H.prebuilt_spmv_csr_f32([3], [3, 4], csr, vals, [4], [[]], dev(np.ones(4, np.float32)))
        if symbol == "prebuilt_spmspm_csr_f32":
            eye = [[], [dev(np.arange(5, dtype=np.int32)), dev(np.arange(4, dtype=np.int32))]]
            return H.prebuilt_spmspm_csr_f32([3, 4], [3, 4], csr, vals, [4, 4], eye, dev(np.ones(4, np.float32)))
        return H.sddmm_csr_float([3, 4], [3, 4], csr, vals, [3, 2], [[], []], dev(np.ones(6, np.float32)), [4, 2],
                                 [[], []], dev(np.ones(8, np.float32)))

    call(good_rp, good_ci)
    with pytest.raises(ValueError, match="column index"):
        call(good_rp, np.array([0, 4, 1, 2, 3], np.int32))
    with pytest.raises(ValueError, match="column index"):
        call(good_rp, np.array([0, 3, -1, 2, 3], np.int32))
    for bad in ([0, 3, 2, 5], [1, 2, 2, 5], [0, 2, 2, 4]):
        with pytest.raises(ValueError, match="row_ptr"):
            call(np.array(bad, np.int32), good_ci)
    torch.cuda.synchronize()


def test_plan_is_kept_on_the_operand_and_rebuilt_when_it_changes():
    w = workloads.gcn_powerlaw(M=5000, N=32, seed=6, max_degree=2000)
    rp, ci, v, B = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"]), dev(w["B"]).reshape(-1)
    args = ([5000, 32], [5000, 5000], [[], [rp, ci]], v, [5000, 32], [[], []], B)
    first = H.spmm_csr_float_v2(*args).storage.value
    plan = rp._scorch_plan
    assert plan.max_row == int(np.diff(w["row_ptr"]).max()) > H.ROWS_KERNEL_MAX_ROW
    assert list(plan.bounds) == [(32, 4)]
    again = H.spmm_csr_float_v2(*args).storage.value
    assert rp._scorch_plan is plan and torch.equal(first, again)
    ci[0] = ci[0]                                   # written to: the plan no longer vouches for it
    H.spmm_csr_float_v2(*args)
    assert rp._scorch_plan is not plan
    ci[1] = 5000                                    # and a bad index is caught on the next call
    with pytest.raises(ValueError, match="column index"):
        H.spmm_csr_float_v2(*args)


def test_auto_dispatch_follows_the_longest_row(oracle, monkeypatch):
    calls = []
    lib = native.lib()

    class Spy:
        def __getattr__(self, name):
            fn = getattr(lib, name)
            if not name.startswith("scorch_hip_spmm_csr_"):
                return fn

            def wrapped(*a):
                calls.append(name)
                return fn(*a)
            return wrapped

    monkeypatch.setattr(native, "lib", lambda: Spy())
    rng = np.random.default_rng(3)
    rp, ci, v = random_csr(rng, 400, 300, 0.05)
    B = rng.standard_normal((300, 64)).astype(np.float32)
    got = hip_spmm(rp, ci, v, B, path="auto")
    assert "scorch_hip_spmm_csr_rows_f32" in calls and "scorch_hip_spmm_csr_planned_f32" not in calls
    assert oracle.rel_fro(got, oracle.spmm_fp64(rp, ci, v, B)) <= TOL
    calls.clear()
    lens = np.full(400, 3, np.int64); lens[7] = 900
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = rng.integers(0, 300, int(rp[-1])).astype(np.int32)
    v = rng.uniform(-1, 1, ci.size).astype(np.float32)
    got = hip_spmm(rp, ci, v, B, path="auto")
    assert "scorch_hip_spmm_csr_planned_f32" in calls and "scorch_hip_spmm_csr_rows_f32" not in calls
    assert oracle.rel_fro(got, oracle.spmm_fp64(rp, ci, v, B)) <= TOL


@pytest.mark.parametrize("N", [32, 128, 1024])
def test_precomputed_boundaries_change_nothing(N):
    """The merge-path kernels with their chunk boundaries read from the plan against the same
    kernels searching row_ptr: bit for bit."""
    w = workloads.gcn_powerlaw(M=40_000, N=N, seed=8, max_degree=9000)
    with spmm_path("merge"):
        planned = hip_spmm(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    with spmm_path("merge_unplanned"):
        searched = hip_spmm(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    assert np.array_equal(planned, searched)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32])
@pytest.mark.parametrize("N", [128, 520])
def test_mostly_empty_rows_one_fill_then_only_the_rows_with_entries(oracle, dtype, N):
    """SCORCH_HIP_HINT_MOSTLY_EMPTY_ROWS through the C ABI: the same result bit for bit as
    without the hint, rows cut by chunk boundaries and a row of thousands of entries included;
    and the Python layer takes that route by itself for a large result with mostly empty rows."""
    rng = np.random.default_rng(31)
    M, K = 70_000, 9_000
    lens = np.where(rng.random(M) < 0.08, rng.integers(1, 40, M), 0).astype(np.int64)
    lens[123] = 7000
    lens[M - 1] = 300
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens if n]).astype(np.int32)
    v = (rng.integers(-9, 9, ci.size) if np.issubdtype(dtype, np.integer) else rng.uniform(-1, 1, ci.size)).astype(dtype)
    B = (rng.integers(-9, 9, (K, N)) if np.issubdtype(dtype, np.integer) else rng.standard_normal((K, N))).astype(dtype)
    t_rp, t_ci, t_v, t_B = dev(rp), dev(ci), dev(v), dev(B).reshape(-1)
    L = native.lib()
    suffix = {np.float32: "f32", np.float64: "f64", np.int32: "i32"}[dtype]
    elem = np.dtype(dtype).itemsize
    ws = torch.empty(L.scorch_hip_spmm_csr_workspace_bytes(M, ci.size, N, elem), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for act in (0, H.HINT_MOSTLY_EMPTY_ROWS):
        out = torch.full((M * N,), 77, dtype=t_v.dtype, device="cuda")
        native.check(getattr(L, "scorch_hip_spmm_csr_planned_" + suffix)(
            M, K, N, ci.size, t_rp.data_ptr(), t_ci.data_ptr(), t_v.data_ptr(), t_B.data_ptr(), None, act,
            out.data_ptr(), None, 0, ws.data_ptr(), ws.numel(), stream))
        outs.append(out)
    assert torch.equal(outs[0], outs[1])
    want = oracle.spmm_fp64(rp, ci, v, B)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(host(outs[1]).reshape(M, N), want.astype(dtype))
    else:
        assert oracle.rel_fro(host(outs[1]).reshape(M, N), want) <= TOL
    auto = hip_spmm(rp, ci, v, B, path="auto")          # 36 MB and more of result, 92 % of the rows empty
    assert np.array_equal(auto, host(outs[0]).reshape(M, N))


def test_row_split_kernel_is_bit_reproducible_and_matches_the_reference(oracle):
    w = workloads.spmm_uniform()
    with spmm_path("rows"):
        a = hip_spmm(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
        b = hip_spmm(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    assert np.array_equal(a, b)
    assert oracle.rel_fro(a, oracle.spmm_fp64(w["row_ptr"], w["col_idx"], w["vals"], w["B"])) <= TOL
    np.testing.assert_allclose(a, oracle.spmm_csr_f32_v2(w["row_ptr"], w["col_idx"], w["vals"], w["B"]), rtol=1e-4,
                               atol=1e-5)


def test_tiled_layout_round_trip():
    """Bt[tile][k][c] holds B[k][32 tile + c], zeros past N."""
    K, N = 37, 70
    B = torch.randn(K, N, device="cuda")
    L = native.lib()
    nbytes = L.scorch_hip_dense_tiled_bytes(K, N, 4)
    assert nbytes == 3 * K * 128
    Bt = torch.full((nbytes // 4,), float("nan"), device="cuda")
    native.check(L.scorch_hip_dense_to_tiled_f32(K, N, B.data_ptr(), Bt.data_ptr(), nbytes,
                                                 torch.cuda.current_stream().cuda_stream))
    tiles = Bt.view(3, K, 32)
    padded = torch.zeros(K, 96, device="cuda")
    padded[:, :N] = B
    assert torch.equal(tiles.permute(1, 0, 2).reshape(K, 96), padded)
    assert L.scorch_hip_dense_tiled_recommended(16_384, 4096, 131_072, 4) == 1
    assert L.scorch_hip_dense_tiled_recommended(16_384, 128, 131_072, 4) == 0       # narrow rows
    assert L.scorch_hip_dense_tiled_recommended(1 << 20, 4096, 1 << 24, 4) == 0     # a slice would not fit an L2
    assert L.scorch_hip_dense_tiled_recommended(16_384, 4096, 16_384, 4) == 0       # rows of B used once


def test_a_dense_operand_seen_twice_is_tiled_and_tracks_changes(oracle):
    """Second product with the same unchanged wide operand: it is re-stored by column tiles and
    the tiled kernel takes over; writing to the operand drops the copy."""
    w = workloads.sae_decoder(M=512, K=2048, N=1024, k=16)          # 32 tiles, 256 KiB slices
    rp, ci, v = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"])
    B = dev(w["B"]).reshape(-1)
    args = ([512, 1024], [512, 2048], [[], [rp, ci]], v, [2048, 1024], [[], []], B)
    ref64 = oracle.spmm_fp64(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    with spmm_path("merge"):
        plain = host(H.spmm_csr_float_v2(*args).storage.value).reshape(512, 1024)
    assert not hasattr(B, "_scorch_tiled")
    first = H.spmm_csr_float_v2(*args).storage.value.clone()        # auto: seen once, plain kernel
    assert not hasattr(B, "_scorch_tiled")
    second = H.spmm_csr_float_v2(*args).storage.value.clone()       # seen twice: tiled from now on
    assert hasattr(B, "_scorch_tiled")
    third = H.spmm_csr_float_v2(*args).storage.value.clone()
    assert torch.equal(second, third)
    for got in (first, second):
        assert oracle.rel_fro(host(got).reshape(512, 1024), ref64) <= TOL
    np.testing.assert_allclose(host(second).reshape(512, 1024), plain, rtol=1e-5, atol=1e-6)
    B.mul_(2.0)                                                     # the copy is stale now
    fourth = H.spmm_csr_float_v2(*args).storage.value
    assert oracle.rel_fro(host(fourth).reshape(512, 1024), 2 * ref64) <= TOL
    fifth = H.spmm_csr_float_v2(*args).storage.value                # tiled again, from the new values
    assert B._scorch_tiled[0] == B._version
    assert oracle.rel_fro(host(fifth).reshape(512, 1024), 2 * ref64) <= TOL


def test_a_recorded_step_never_reads_a_tiled_copy(oracle):
    """A wide dense operand that has a column-tile copy (built by eager products) and is then
    handed to a captured step and rewritten in place between replays: every replay sees the new
    values, and the capture has made the operand volatile, so no copy of it is kept any more."""
    from scorch_amd import graphs
    rng = np.random.default_rng(41)
    M, K, N = 512, 2048, 2048
    rp, ci, v = random_csr(rng, M, K, 0.01)
    t_rp, t_ci, t_v = dev(rp), dev(ci), dev(v)
    B = torch.randn(K * N, device="cuda")
    product = lambda b: H.spmm_csr_float_v2([M, N], [M, K], [[], [t_rp, t_ci]], t_v, [K, N], [[], []], b).storage.value
    for _ in range(3):
        product(B)
    assert getattr(B, "_scorch_tiled", None) is not None        # eager products built the copy
    step = graphs.capture(product, B, warmup=3)
    assert H.is_volatile(B) and getattr(B, "_scorch_tiled", None) is None
    for _ in range(3):
        B.copy_(torch.randn(K * N, device="cuda"))
        got = step().clone()
        assert oracle.rel_fro(host(got).reshape(M, N), oracle.spmm_fp64(rp, ci, v, host(B).reshape(K, N))) <= TOL
        assert torch.equal(got, product(B))                     # the eager call runs from the operand itself too


def test_matmul_keeps_the_tiled_copy_on_the_callers_tensor(oracle):
    import scorch_amd as scorch
    w = workloads.sae_decoder(M=256, K=2048, N=1024, k=16)
    A = scorch.STensor.from_csr_arrays(dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"]), (256, 2048))
    W = dev(w["B"])
    outs = [scorch.matmul(A, W, format="dd") for _ in range(3)]
    assert hasattr(W, "_scorch_tiled") and hasattr(A.index.mode_indices[1][0], "_scorch_plan")
    ref64 = oracle.spmm_fp64(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    for out in outs:
        assert out.shape == (256, 1024) and oracle.rel_fro(host(out), ref64) <= TOL


@pytest.mark.parametrize("relu", [False, True])
def test_tiled_kernel_with_rows_cut_by_chunks_and_an_epilogue(oracle, relu):
    """Long rows (carries folded by the fix-up), N not a multiple of the tile width or of 4."""
    rng = np.random.default_rng(17)
    lens = rng.integers(0, 40, 600); lens[[0, 300, 599]] = [700, 1500, 420]
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = rng.integers(0, 900, int(rp[-1])).astype(np.int32)
    v = rng.uniform(-1, 1, ci.size).astype(np.float32)
    for N in (1000, 1027):
        B = rng.standard_normal((900, N)).astype(np.float32)
        bias = rng.standard_normal(N).astype(np.float32)
        got = hip_spmm(rp, ci, v, B, bias=bias, relu=relu, path="tiled")
        want = oracle.spmm_fp64(rp, ci, v, B) + bias
        want = np.maximum(want, 0) if relu else want
        assert oracle.rel_fro(got, want) <= TOL
        again = hip_spmm(rp, ci, v, B, bias=bias, relu=relu, path="tiled")
        assert np.array_equal(got, again)


def test_tiled_kernel_when_the_even_resplit_makes_chunks_longer_than_the_usual_ones(oracle):
    """4096 rows of 32 entries with a hundred rows of 330 to 600: the tiled kernel re-splits the work
    into a multiple of 128 chunks of more than 256 items, and a chunk that ends inside one of the
    long rows stages up to 64 items more.  Checked against fp64 and against the merge path."""
    rng = np.random.default_rng(3)
    M, K, N = 4096, 4096, 4096
    lens = np.full(M, 32, np.int64)
    lens[rng.choice(M, 100, replace=False)] = rng.integers(330, 601, 100)
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens]).astype(np.int32)
    v = rng.uniform(-1, 1, ci.size).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    want = oracle.spmm_fp64(rp, ci, v, B)
    got = hip_spmm(rp, ci, v, B, path="tiled")
    assert oracle.rel_fro(got, want) <= TOL
    merge = hip_spmm(rp, ci, v, B, path="merge")
    assert oracle.rel_fro(got, merge) <= 1e-6                # (long rows are summed in another grouping)
    np.testing.assert_allclose(got, merge, rtol=1e-2, atol=1e-4)
    assert np.array_equal(got, hip_spmm(rp, ci, v, B, path="tiled"))


@pytest.mark.parametrize("longest", [1, 7, 33, 64, 200])
@pytest.mark.parametrize("relu", [None, False, True])
def test_tiled_kernel_over_row_lengths_and_epilogues(oracle, longest, relu, monkeypatch):
    """The tiled kernel against fp64 and, bit for bit where no row is shared by all lane groups
    (at most 64 entries), against the merge path: empty rows, rows cut by chunk boundaries, an
    epilogue, N not a multiple of the tile width."""
    rng = np.random.default_rng(100 * longest + (0 if relu is None else 1 + relu))
    M, K = 3000, 1500
    lens = rng.integers(0, longest + 1, M)
    lens[rng.choice(M, 40, replace=False)] = longest
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(K, n, replace=False)) for n in lens] + [np.zeros(0, np.int64)]).astype(np.int32)
    v = rng.uniform(-1, 1, ci.size).astype(np.float32)
    for N in (1024, 1027):
        B = rng.standard_normal((K, N)).astype(np.float32)
        bias = None if relu is None else rng.standard_normal(N).astype(np.float32)
        want = oracle.spmm_fp64(rp, ci, v, B)
        if bias is not None:
            want = np.maximum(want + bias, 0) if relu else want + bias
        got = hip_spmm(rp, ci, v, B, bias=bias, relu=bool(relu), path="tiled")
        assert oracle.rel_fro(got, want) <= TOL
        assert np.array_equal(got, hip_spmm(rp, ci, v, B, bias=bias, relu=bool(relu), path="tiled"))
        # without a plan the longest row is unknown and the launch that folds shared rows' partial sums
        # always runs; with one it is left out when no row can be shared: the same bits either way
        monkeypatch.setenv("SCORCH_HIP_PLAN", "0")
        unplanned = hip_spmm(rp, ci, v, B, bias=bias, relu=bool(relu), path="tiled")
        monkeypatch.delenv("SCORCH_HIP_PLAN")
        assert np.array_equal(got, unplanned)
