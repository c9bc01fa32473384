"""SpMV, CSR row softmax and the Python-level matmul / einsum routing on the
MI355X.  SpMV and softmax tolerances: relative Frobenius error <= 1e-5 against
fp64; integer SpMV bit-exact."""
import numpy as np
import pytest
import torch

import scorch_amd as scorch
from conftest import random_csr
from gpu_util import dev, hip_spmv, host
from scorch_amd import STensor, ops
from scorch_amd import scorch_ops_hip as H
from scorch_amd import workloads

pytestmark = pytest.mark.gpu
TOL = 1e-5


def test_spmv_golden(golden):
    c = golden.case("spmv_i64_literal")
    assert hip_spmv(c["row_ptr"], c["col_idx"], c["vals"], c["x"]).tolist() == [7, 22, 0, 29]
    for name in ("spmv_f32", "spmv_f64", "spmv_i32"):
        c = golden.case(name)
        got = hip_spmv(c["row_ptr"], c["col_idx"], c["vals"], c["x"])
        if name == "spmv_i32":
            assert np.array_equal(got, c["y"])
        else:
            np.testing.assert_allclose(got, c["y"], rtol=1e-5 if name == "spmv_f32" else 1e-13, atol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
@pytest.mark.parametrize("density", [0.002, 0.05, 0.6])   # group widths 2 .. 64
def test_spmv_against_oracle(oracle, dtype, density):
    rng = np.random.default_rng(int(density * 1000))
    rp, ci, v = random_csr(rng, 1500, 400, density, dtype=dtype, empty_rows=(0, 1499))
    x = (rng.integers(-1000, 1000, 400) if np.issubdtype(dtype, np.integer)
         else rng.standard_normal(400)).astype(dtype)
    got = hip_spmv(rp, ci, v, x)
    want = oracle.spmv_csr_typed(rp, ci, v, x)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got, want)
    else:
        dense64 = oracle.spmm_fp64(rp, ci, v, x.reshape(-1, 1)).reshape(-1)
        assert oracle.rel_fro(got, dense64) <= (TOL if dtype == np.float32 else 1e-13)


def test_softmax_against_oracle(oracle):
    w = workloads.gcn_powerlaw(M=8000, N=4, seed=12, max_degree=3000)
    rng = np.random.default_rng(0)
    vals = rng.standard_normal(w["col_idx"].size).astype(np.float32) * 5
    got = host(H.softmax_csr_float(dev(w["row_ptr"]), dev(vals), 0.125))
    assert oracle.rel_fro(got, oracle.softmax_csr_fp64(w["row_ptr"], vals, 0.125)) <= TOL
    np.testing.assert_allclose(got, oracle.softmax_csr_f32(w["row_ptr"], vals, 0.125), rtol=1e-4, atol=1e-7)
    sums = np.add.reduceat(got, w["row_ptr"][:-1])
    np.testing.assert_allclose(sums, 1.0, rtol=1e-5)


def test_softmax_every_row_length_tier(oracle):
    """Row lengths chosen around each hand-over of the kernel: lane groups, quarter
    wavefronts, wavefronts, the workgroup (up to 4096 entries) and the giant-row
    kernel (first 8192 entries in registers, the rest re-read)."""
    lens = np.array([0, 1, 7, 8, 9, 16, 17, 63, 64, 65, 255, 256, 257, 0, 1023, 1024, 1025, 2047, 2048, 2049, 3,
                     4095, 4096, 4097, 8191, 8192, 8193, 20000, 5, 0], np.int64)
    rng = np.random.default_rng(3)
    for mean_pad in (0, 400):  # few short rows -> narrow groups; many -> group width follows the mean
        all_lens = np.concatenate([lens, np.full(mean_pad, 2, np.int64)])
        rp = np.concatenate([[0], np.cumsum(all_lens)]).astype(np.int32)
        vals = (rng.standard_normal(int(rp[-1])) * 4).astype(np.float32)
        got = host(H.softmax_csr_float(dev(rp), dev(vals), 0.5))
        want = oracle.softmax_csr_fp64(rp, vals, 0.5)
        assert oracle.rel_fro(got, want) <= TOL
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=1e-12)


def test_softmax_full_size(oracle):
    """The headline graph's pattern (1,048,576 rows, 17 M entries, rows up to 50,000 entries):
    against the restatement, and every non-empty row sums to one."""
    w = workloads.gcn_powerlaw(N=1)
    rng = np.random.default_rng(5)
    vals = (rng.standard_normal(w["col_idx"].size) * 6).astype(np.float32)
    rp = dev(w["row_ptr"])
    out = H.softmax_csr_float(rp, dev(vals), 0.5)
    assert torch.equal(out, H.softmax_csr_float(rp, dev(vals), 0.5))  # same bits on every run
    got = host(out)
    want = oracle.softmax_csr_f32(w["row_ptr"], vals, 0.5)
    assert oracle.rel_fro(got, want.astype(np.float64)) <= TOL
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-9)
    rows = torch.repeat_interleave(torch.arange(w["M"], device="cuda"), (rp[1:] - rp[:-1]).long())
    sums = torch.zeros(w["M"], dtype=torch.float64, device="cuda").index_add_(0, rows, out.double())
    nonempty = (rp[1:] > rp[:-1])
    assert torch.allclose(sums[nonempty], torch.ones_like(sums[nonempty]), rtol=1e-5)


@pytest.mark.parametrize("n_rows,length", [(300, 5000), (2100, 4097), (40, 9000)])
def test_softmax_many_long_rows(oracle, n_rows, length):
    """Every row beyond the workgroup tier: more listed rows than the giant-row kernel has
    workgroups (it walks the list), fewer, and rows longer than its registers hold."""
    rng = np.random.default_rng(n_rows)
    rp = (np.arange(n_rows + 1, dtype=np.int64) * length).astype(np.int32)
    vals = (rng.standard_normal(int(rp[-1])) * 3).astype(np.float32)
    got = host(H.softmax_csr_float(dev(rp), dev(vals), 0.7))
    want = oracle.softmax_csr_f32(rp, vals, 0.7)
    assert oracle.rel_fro(got, want.astype(np.float64)) <= TOL
    np.testing.assert_allclose(got.reshape(n_rows, length).sum(axis=1), 1.0, rtol=1e-5)


def test_softmax_long_rows_among_very_short_ones(oracle):
    """A mean row length of two (lane groups of two, 512 rows to a workgroup) with every row of
    one stretch far beyond the workgroup tier: more listed rows in one workgroup than it has threads."""
    rng = np.random.default_rng(12)
    lens = np.full(700_000, 1, np.int64)
    lens[1024:1024 + 300] = 4100 + rng.integers(0, 50, 300)
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    vals = (rng.standard_normal(int(rp[-1])) * 2).astype(np.float32)
    got = host(H.softmax_csr_float(dev(rp), dev(vals), 1.0))
    want = oracle.softmax_csr_f32(rp, vals, 1.0)
    assert oracle.rel_fro(got, want.astype(np.float64)) <= TOL
    assert np.all(got[:1024] == 1.0)


def test_softmax_in_place(oracle):
    """out may alias vals, also for rows that are re-read and for prefetched ones"""
    lens = np.array([3, 9000, 5000, 12, 20000, 300, 4500, 0, 70], np.int64)
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    vals = (np.random.default_rng(8).standard_normal(int(rp[-1])) * 3).astype(np.float32)
    v = dev(vals)
    pos = dev(rp)
    L = H.native.lib()
    need = L.scorch_hip_softmax_csr_workspace_bytes(len(lens), v.numel())
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    rc = L.scorch_hip_softmax_csr_f32(len(lens), v.numel(), pos.data_ptr(), v.data_ptr(), 0.5, v.data_ptr(),
                                      ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert oracle.rel_fro(host(v), oracle.softmax_csr_fp64(rp, vals, 0.5)) <= TOL


@pytest.mark.parametrize("lens", [[4_200_000], [3, 70_000, 0, 1_500_000, 12, 65_536, 65_537, 5000, 200_000],
                                  [17, 20_000_000],      # (more entries than 1024 stretches of 16,384 hold)
                                  # more than 512 rows beyond 4096 entries: those up to 65,536 stay one workgroup's
                                  [4100] * 600 + [20_000, 70_000, 30_000, 65_536],
                                  # rows beyond 65,536 entries none of which stands out: one workgroup's each
                                  [70_000] * 150 + [5, 600_000]])
def test_softmax_rows_shared_out_among_workgroups(oracle, lens):
    """Rows of more than 65,536 entries are served in stretches by many workgroups (a single row of
    millions would otherwise be one workgroup's): against the fp64 recomputation, the same bits on
    every run, in place, and for a batch of value arrays over the pattern."""
    lens = np.array(lens, np.int64)
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    rng = np.random.default_rng(int(lens.sum()) % 1000)
    vals = (rng.standard_normal(int(rp[-1])) * 4).astype(np.float32)
    vals[int(rp[-1]) // 2] = 40.0                          # one entry that towers over its row
    pos, v = dev(rp), dev(vals)
    out = H.softmax_csr_float(pos, v, 0.5)
    want = oracle.softmax_csr_fp64(rp, vals, 0.5)
    assert oracle.rel_fro(host(out), want) <= TOL
    np.testing.assert_allclose(host(out), want, rtol=5e-5, atol=1e-30)
    assert torch.equal(out, H.softmax_csr_float(pos, v, 0.5))
    sums = np.add.reduceat(host(out).astype(np.float64), rp[:-1][lens > 0])
    np.testing.assert_allclose(sums, 1.0, rtol=1e-5)
    # a batch: every problem's rows, also the ones served in stretches
    batch = torch.stack([v, v * 0.5 + 1.0, -v])
    got = H.softmax_csr_float_batched(pos, batch, 0.5)
    for h in range(3):
        assert torch.equal(got[h], H.softmax_csr_float(pos, batch[h].contiguous(), 0.5))
    # in place through the C ABI
    L = H.native.lib()
    need = L.scorch_hip_softmax_csr_workspace_bytes(len(lens), v.numel())
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    inplace = v.clone()
    rc = L.scorch_hip_softmax_csr_f32(len(lens), v.numel(), pos.data_ptr(), inplace.data_ptr(), 0.5, inplace.data_ptr(),
                                      ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and torch.equal(inplace, out)


@pytest.mark.parametrize("lens", [[3, 0, 4096, 17, 900], [3, 9000, 5000, 12, 65_536, 300, 0, 70],
                                  [5, 65_537, 100, 300_000, 4097]])
def test_softmax_with_the_longest_row_stated(oracle, lens):
    """scorch_hip_softmax_csr_known_rows_f32 leaves out the launches no row of the stated length
    needs (no list of giant rows up to 4096 entries, no stretches up to 16,384): the same bits as
    the entry point that is told nothing, for one value array and for a batch; a negative length
    is refused."""
    lens = np.array(lens, np.int64)
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    vals = (np.random.default_rng(int(lens.max())).standard_normal(int(rp[-1])) * 3).astype(np.float32)
    pos = dev(rp)
    batch = torch.stack([dev(vals), dev(vals) * -0.5 + 2.0])
    M, nnz, longest = len(lens), int(rp[-1]), int(lens.max())
    L = H.native.lib()
    stream = torch.cuda.current_stream().cuda_stream
    need = L.scorch_hip_softmax_csr_workspace_bytes(M, nnz)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    plain, told = torch.full_like(batch, -1.0), torch.full_like(batch, -1.0)
    assert L.scorch_hip_softmax_csr_batched_f32(2, M, nnz, pos.data_ptr(), batch.data_ptr(), 0.5, plain.data_ptr(),
                                                ws.data_ptr(), need, stream) == 0
    short = longest <= 4096
    assert L.scorch_hip_softmax_csr_known_rows_f32(2, M, nnz, longest, pos.data_ptr(), batch.data_ptr(), 0.5,
                                                   told.data_ptr(), None if short else ws.data_ptr(),
                                                   0 if short else need, stream) == 0
    assert torch.equal(plain, told)
    assert oracle.rel_fro(host(told[0]), oracle.softmax_csr_fp64(rp, vals, 0.5)) <= TOL
    if not short:      # the longer rows need the workspace
        assert L.scorch_hip_softmax_csr_known_rows_f32(2, M, nnz, longest, pos.data_ptr(), batch.data_ptr(), 0.5,
                                                       told.data_ptr(), None, 0, stream) == H.native.EWORKSPACE
    assert L.scorch_hip_softmax_csr_known_rows_f32(2, M, nnz, -1, pos.data_ptr(), batch.data_ptr(), 0.5,
                                                   told.data_ptr(), ws.data_ptr(), need, stream) == H.native.EINVAL
    if short:          # a longer row than stated is left unwritten, not a fault: nothing is listed without a workspace
        lie = torch.full_like(batch, -1.0)
        wide = dev(np.array([0, 5000, 5003], np.int32))
        assert L.scorch_hip_softmax_csr_known_rows_f32(1, 2, 5003, 100, wide.data_ptr(), batch.data_ptr(), 0.5,
                                                       lie.data_ptr(), None, 0, stream) == 0
        torch.cuda.synchronize()
        assert bool((lie[0, :5000] == -1.0).all()) and abs(float(lie[0, 5000:5003].sum()) - 1.0) < 1e-5
    # the Python layer: a product over the pattern has inspected it, the softmax then states the longest row
    ci = dev(np.concatenate([np.arange(n, dtype=np.int32) for n in lens]))
    H.spmm_csr_float_v2([M, 4], [M, longest], [[], [pos, ci]], batch[0].contiguous(), [longest, 4], [[], []],
                        torch.ones(longest, 4, device="cuda"))
    assert H._known_longest_row(pos, M, nnz) == longest
    assert torch.equal(H.softmax_csr_float(pos, batch[0].contiguous(), 0.5), plain[0])
    assert torch.equal(H.softmax_csr_float_batched(pos, batch, 0.5), plain)


def test_softmax_with_empty_rows_and_large_values(oracle):
    rp = np.array([0, 0, 4, 4, 5], np.int32)
    vals = np.array([1000.0, 1001.0, 999.0, 1000.5, -3.0], np.float32)
    got = host(H.softmax_csr_float(dev(rp), dev(vals), 1.0))
    assert np.isfinite(got).all() and got[4] == 1.0
    np.testing.assert_allclose(got, oracle.softmax_csr_fp64(rp, vals), rtol=1e-5)


# ---- the Python interface (reference: tests/test_scorch/test_matmul_dispatch.py) ----------------
@pytest.mark.parametrize("use_cache", [True, False])
def test_sparse_stensor_spmm_does_not_call_torch_matmul(use_cache, monkeypatch):
    torch.manual_seed(0)
    n = 32
    a_torch = torch.rand(n, n) * (torch.rand(n, n) < 0.1)
    b_torch = torch.rand(n, n)
    expected = torch.matmul(a_torch, b_torch)
    a = STensor.from_torch(a_torch, "A").to_sparse("ds").to("cuda")
    b = STensor.from_torch(b_torch, "B").to("cuda")

    def forbidden(*args, **kwargs):
        raise AssertionError("torch.matmul should not be used for sparse STensor matmul")

    monkeypatch.setattr(ops.torch, "matmul", forbidden)
    out = scorch.matmul(a, b, format="dd", use_cache=use_cache)
    assert isinstance(out, torch.Tensor) and out.is_cuda and out.shape == (n, n)
    assert torch.allclose(out.cpu(), expected, atol=1e-3, rtol=1e-3)


def test_matmul_accepts_torch_operands_and_fills_time_dict():
    torch.manual_seed(1)
    a = (torch.rand(300, 200) * (torch.rand(300, 200) < 0.05)).cuda()
    b = torch.rand(200, 128).cuda()
    td = {}
    out = scorch.matmul(scorch.from_csr(a.to_sparse_csr()), b, time_dict=td)
    assert td["eval_time"] > 0
    assert torch.allclose(out, a @ b, atol=1e-4, rtol=1e-4)
    out2 = scorch.einsum("ik,kj->ij", a.to_sparse_csr(), b, format="dd")
    assert torch.equal(out, out2)
    nc = b.t().contiguous().t()                      # non-contiguous dense operand is flattened first
    assert torch.equal(scorch.matmul(scorch.from_csr(a.to_sparse_csr()), nc), out)


def test_the_usual_spmm_calls_do_not_wrap_the_dense_operand(monkeypatch):
    """matmul(A, B), matmul(A, B, format="dd"), einsum("ij,jk->ik", A, B) and the matrix-vector forms
    reach the kernel without building STensors around the dense operand and the result (which
    costs more host time than the kernel of a small product takes); a request for a sparse result
    still goes the general way."""
    torch.manual_seed(5)
    a_t = torch.rand(96, 80) * (torch.rand(96, 80) < 0.1)
    A = scorch.from_csr(a_t.to_sparse_csr()).to("cuda")
    B, x = torch.rand(80, 24).cuda(), torch.rand(80).cuda()
    want, want_v = scorch.matmul(A, B), scorch.matmul(A, x)
    sparse_result = scorch.matmul(A, B, format="ds")
    wrapped = []
    real = STensor.from_torch
    monkeypatch.setattr(STensor, "from_torch", staticmethod(lambda *a, **k: (wrapped.append(1), real(*a, **k))[1]))
    for got in (scorch.matmul(A, B, format="dd"), scorch.matmul(A, B, output_format="dd"),
                scorch.einsum("ij,jk->ik", A, B), scorch.einsum("ab,bc->ac", A, B, format="dd")):
        assert isinstance(got, torch.Tensor) and torch.equal(got, want)
    for got in (scorch.matmul(A, x, format="d"), scorch.einsum("ij,j->i", A, x)):
        assert isinstance(got, torch.Tensor) and torch.equal(got, want_v)
    assert not wrapped
    again = scorch.matmul(A, B, format="ds")
    assert wrapped and isinstance(again, STensor)
    assert torch.equal(again.to_dense().to_torch(), sparse_result.to_dense().to_torch())
    assert torch.allclose(want.cpu(), a_t @ B.cpu(), atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float64, torch.int32, torch.int64])
def test_matmul_other_dtypes(dtype):
    torch.manual_seed(2)
    a = ((torch.rand(64, 64) * 20).round() * (torch.rand(64, 64) < 0.1)).to(dtype)
    b = (torch.rand(64, 16) * 20).round().to(dtype)
    out = scorch.matmul(STensor.from_torch(a).to_sparse("ds").to("cuda"), b.cuda())
    assert out.dtype == dtype and torch.equal(out.cpu(), a @ b)


def test_matmul_vector_operand():
    torch.manual_seed(3)
    a = torch.rand(100, 80) * (torch.rand(100, 80) < 0.1)
    x = torch.rand(80)
    out = scorch.matmul(STensor.from_torch(a).to_sparse("ds").to("cuda"), x.cuda())
    assert out.shape == (100,) and torch.allclose(out.cpu(), a @ x, atol=1e-5)


@pytest.mark.parametrize("n,d,sparsity", [(16, 8, 0.5), (64, 32, 0.9), (128, 16, 0.95), (256, 64, 0.99)])
@pytest.mark.parametrize("mask_format", ["ds", "oo"])
def test_einsum_sddmm(n, d, sparsity, mask_format):
    """reference: tests/test_scorch/test_kernels_comprehensive.py:376-411"""
    torch.manual_seed(n + d)
    mask = torch.rand(n, n) * (torch.rand(n, n) > sparsity)
    Q, K = torch.rand(n, d), torch.rand(n, d)
    mask_st = STensor.from_torch(mask).to_sparse(mask_format).to("cuda")
    result = scorch.einsum("ij,ik,jk->ij", mask_st, Q.cuda(), K.cuda())
    assert isinstance(result, STensor) and str(result.format) == "o,o"     # all-coordinate output
    assert result._nnz() == mask_st._nnz()
    assert torch.allclose(result.to_torch().cpu(), (Q @ K.T) * mask, atol=1e-3, rtol=1e-3)
    kj = scorch.einsum("ij,ik,kj->ij", mask_st, Q.cuda(), K.t().contiguous().cuda())
    assert torch.allclose(kj.values, result.values, atol=1e-6)


def test_spmm_bias_act_interface():
    torch.manual_seed(42)
    a = torch.randn(64, 64) * (torch.rand(64, 64) < 0.1)
    b, bias = torch.randn(64, 16), torch.randn(16)
    A = STensor.from_torch(a).to_sparse("ds").to("cuda")
    plain = scorch.spmm_bias_act(A, b.cuda(), bias.cuda())
    relu = scorch.spmm_bias_act(A, STensor.from_torch(b.cuda()), bias.cuda(), relu=True)
    assert torch.allclose(plain.cpu(), a @ b + bias, atol=1e-4)
    assert torch.allclose(relu.cpu(), torch.relu(a @ b + bias), atol=1e-4)


def test_unfused_attention_pipeline_matches_dense(oracle):
    """SDDMM -> row softmax -> SpMM over a CSR mask, the per-head composition of
    bench/bench_sparse_transformer.py:354-372, against masked dense attention in fp64."""
    S, D = 512, 64
    brp, bci = workloads.blocksparse_pattern(S // 64)
    rp, ci = workloads.blocks_to_csr(brp, bci, 64)
    rng = np.random.default_rng(4)
    q, k, v = (rng.standard_normal((S, D)).astype(np.float32) for _ in range(3))
    mask = STensor.from_csr_arrays(dev(rp), dev(ci), torch.ones(ci.size, device="cuda"), (S, S))
    scores = scorch.einsum("ij,ik,jk->ij", mask, dev(q), dev(k))
    probs = H.softmax_csr_float(dev(rp), scores.values, D ** -0.5)
    out = scorch.matmul(STensor.from_csr_arrays(dev(rp), dev(ci), probs, (S, S)), dev(v), format="dd")
    dense_mask = np.zeros((S, S), bool)
    dense_mask[oracle.rows_of(rp), ci] = True
    assert oracle.rel_fro(host(out), oracle.attention_dense_fp64(q, k, v, dense_mask, D ** -0.5)) <= TOL


# ---- @compile (reference: tests/test_scorch/test_compile.py:70-127) ----------------------------
def _csr_and_dense_cuda(n=64, k=16, density=0.1, seed=42):
    torch.manual_seed(seed)
    vals = torch.rand(n, n) * (torch.rand(n, n) < density).float()
    return vals, STensor.from_csr(vals.to_sparse_csr(), "A").to("cuda"), torch.rand(n, k)


def test_compile_spmm_bias_relu_csr():
    dense_a, adj, x = _csr_and_dense_cuda()
    bias = torch.rand(x.size(1))

    @scorch.compile
    def fused(adj, x, bias):
        h = scorch.matmul(adj, x, format="dd")
        h = h + bias
        return torch.relu(h)

    result = fused(adj, x.cuda(), bias.cuda())
    assert isinstance(result, torch.Tensor) and result.is_cuda
    assert torch.allclose(result.cpu(), torch.relu(dense_a @ x + bias), atol=1e-4)
    assert list(fused._cache.values())[0][0].fused_symbol == "spmm_csr_bias_relu_float"
    # second call reuses the trace and the runner
    again = fused(adj, x.cuda(), bias.cuda())
    assert torch.equal(result, again) and len(fused._cache) == 1


def test_compile_spmm_bias_csr_and_unfused_chain():
    dense_a, adj, x = _csr_and_dense_cuda(seed=7)
    bias = torch.rand(x.size(1))

    @scorch.compile
    def bias_only(adj, x, bias):
        return scorch.matmul(adj, x, format="dd") + bias

    @scorch.compile
    def tanh_chain(adj, x, bias):
        return torch.tanh(scorch.matmul(adj, x, format="dd") * bias)

    out = bias_only(adj, x.cuda(), bias.cuda())
    assert torch.allclose(out.cpu(), dense_a @ x + bias, atol=1e-4)
    chained = tanh_chain(adj, x.cuda(), bias.cuda())
    assert list(tanh_chain._cache.values())[0][0].fused_symbol is None      # runs matmul + torch ops
    assert torch.allclose(chained.cpu(), torch.tanh((dense_a @ x) * bias), atol=1e-4)


def test_compile_matches_unfused():
    _, adj, x = _csr_and_dense_cuda(n=300, k=128, seed=9)
    bias = torch.rand(128).cuda()

    @scorch.compile
    def fused(adj, x, bias):
        return torch.relu(scorch.matmul(adj, x, format="dd") + bias)

    unfused = torch.relu(scorch.matmul(adj, x.cuda(), format="dd") + bias)
    assert torch.allclose(fused(adj, x.cuda(), bias), unfused, atol=1e-5)


def test_matmul_normalises_a_transposed_csr_operand():
    """A CSR operand stored in mode order [1, 0] is re-stored before dispatch
    (reference: src/scorch/ops.py:333-346)."""
    torch.manual_seed(11)
    a = torch.rand(50, 70) * (torch.rand(50, 70) < 0.1)
    b = torch.rand(70, 32)
    A = STensor.from_torch(a).to_sparse("ds").to("cuda").change_mode_order([1, 0])
    assert A.shape == (70, 50) and A.index.mode_order == [1, 0]
    out = scorch.matmul(A, b.cuda())
    assert torch.allclose(out.cpu(), a @ b, atol=1e-5)
    assert A.index.mode_order == [1, 0]          # the caller's tensor is left as it was


def test_format_plumbing_stays_on_the_device():
    """The formats either side of the kernels, built and converted on the device:
    coordinate -> CSR (from_coo + to_sparse), CSR transpose, back to torch, and the
    unfused chain SDDMM -> softmax -> SpMM fed from them (reference:
    src/scorch/stensor.py:318-365, 785-896, 454-475)."""
    torch.manual_seed(5)
    n, d = 96, 32
    dense = (torch.rand(n, n) * (torch.rand(n, n) < 0.15)).cuda()
    coo = dense.to_sparse()
    A = scorch.from_coo(indices=coo.indices(), values=coo.values(), shape=(n, n))
    assert A.is_cuda and str(A.format) == "o,o"
    A_csr = A.to_sparse("ds")
    assert A_csr.is_cuda and all(t.is_cuda for lvl in A_csr.index.mode_indices for t in lvl)
    assert torch.equal(A_csr.to_torch(in_place=False), dense)
    At = A_csr.copy().change_mode_order([1, 0])
    assert At.is_cuda and At.shape == (n, n)
    q, k = torch.rand(n, d).cuda(), torch.rand(n, d).cuda()
    scores = scorch.einsum("ij,ik,jk->ij", A_csr, q, k)
    assert scores.is_cuda
    want = dense * (q @ k.t())
    assert torch.allclose(scores.to_torch(in_place=False), want, atol=1e-4)
    out = scorch.matmul(A_csr, q)
    assert out.is_cuda and torch.allclose(out, dense @ q, atol=1e-4)


def test_sparse_to_sparse_conversion_does_not_densify():
    """Coordinate <-> CSR for a matrix far too large to materialise (2^20 x 2^20),
    with a repeated coordinate (summed) and an explicit zero (kept)."""
    n = 1 << 20
    g = torch.Generator(device="cuda").manual_seed(9)
    rows = torch.randint(0, n, (200_000,), device="cuda", generator=g)
    cols = torch.randint(0, n, (200_000,), device="cuda", generator=g)
    vals = torch.rand(200_000, device="cuda", generator=g)
    rows[1], cols[1] = rows[0], cols[0]          # a repeated coordinate
    vals[2] = 0.0                                # an explicit zero
    A = scorch.from_coo(indices=torch.stack([rows, cols]), values=vals, shape=(n, n))
    C = A.to_sparse("ds")
    pos, crd = C.index.mode_indices[1]
    assert C.is_cuda and pos.dtype == torch.int32 and pos.numel() == n + 1
    keys = torch.unique(rows * n + cols)
    assert int(pos[-1]) == keys.numel() == C.values.numel()
    back = C.to_sparse("oo")
    r2, c2 = back.index.mode_indices[0][0].long(), back.index.mode_indices[1][0].long()
    assert torch.equal(r2 * n + c2, keys)        # sorted by (row, column), nothing dropped
    assert torch.isclose(back.values.sum(), vals.sum(), rtol=1e-4)
    x = torch.rand(n, 8, device="cuda", generator=g)
    want = torch.zeros(n, 8, device="cuda").index_add_(0, rows, vals[:, None] * x[cols])
    assert torch.allclose(scorch.matmul(C, x), want, atol=1e-4)


def test_index_check_stops_a_bad_operand_before_the_launch():
    """An out-of-range column raises ValueError from the inspection every operand gets when
    it is first seen; the product's kernel is not launched."""
    pos = torch.tensor([0, 1, 2], dtype=torch.int32, device="cuda")
    crd = torch.tensor([0, 7], dtype=torch.int32, device="cuda")      # 7 >= K = 4
    val = torch.ones(2, device="cuda")
    B = torch.ones(4 * 8, device="cuda")
    with pytest.raises(ValueError, match="column index lies outside"):
        H.spmm_csr_float_v2([2, 8], [2, 4], [[], [pos, crd]], val, [4, 8], [[], []], B)
    good = torch.tensor([0, 3], dtype=torch.int32, device="cuda")
    out = H.spmm_csr_float_v2([2, 8], [2, 4], [[], [pos, good]], val, [4, 8], [[], []], B)
    assert torch.equal(out.storage.value, torch.ones(16, device="cuda"))


# ---- HIP graphs -------------------------------------------------------------------------------------
def test_steps_replay_from_a_hip_graph():
    """The entry points only enqueue kernels on the caller's stream (no allocation,
    no synchronisation, no memset), so a step can be captured once and replayed.
    Each replay is checked against an eager call on fresh operand values, with
    eager work and synchronisations between the replays."""
    w = workloads.spmm_uniform()
    M, K, N = w["M"], w["K"], w["N"]
    rp, ci, v = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"])
    B = dev(w["B"]).reshape(-1)
    x = B[:K].clone()
    spmm = lambda: H.spmm_csr_float_v2([M, N], [M, K], [[], [rp, ci]], v, [K, N], [[], []], B).storage.value
    spmv = lambda: H.prebuilt_spmv_csr_f32([M], [M, K], [[], [rp, ci]], v, [K], [[]], x).storage.value
    sddmm = lambda: H.sddmm_csr_float([M, K], [M, K], [[], [rp, ci]], v, [M, N], [[], []], B[:M * N],
                                      [K, N], [[], []], B).storage.value
    # row softmax over a pattern with rows for every tier, the listed (giant) ones included:
    # their count in the workspace has to start from zero in every replay
    lens = np.concatenate([np.full(300, 5), [9000, 70, 5000, 300, 12000], np.full(50, 40)])
    s_rp = dev(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32))
    s_val = torch.empty(int(lens.sum()), device="cuda")
    softmax = lambda: H.softmax_csr_float(s_rp, s_val, 0.5)
    steps = (spmm, spmv, sddmm, softmax)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up off the default stream, as graph capture wants it
        for fn in steps:
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = tuple(fn() for fn in steps)
    gen = torch.Generator(device="cuda").manual_seed(17)
    for _ in range(4):
        B.copy_(torch.randn(B.shape, device="cuda", generator=gen))
        x.copy_(torch.randn(x.shape, device="cuda", generator=gen))
        s_val.copy_(torch.randn(s_val.shape, device="cuda", generator=gen) * 3)
        eager = [fn().clone() for fn in steps]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want)


def test_a_two_layer_gcn_forward_captured_once_and_replayed():
    """scorch_amd.graphs.capture: the layers of a small GCN (dense product, fused SpMM + bias +
    ReLU, dense product, fused SpMM + bias) as one graph; replays on new features equal the
    eager pass bit for bit, with eager work and synchronisations between the replays."""
    import scorch_amd as scorch
    from scorch_amd import STensor, graphs
    rng = np.random.default_rng(23)
    n, f_in, hidden, classes = 2708, 1433, 16, 7          # the shape of the Cora citation graph
    rp, ci, v = random_csr(rng, n, n, 0.002)
    A = STensor.from_csr_arrays(dev(rp), dev(ci), dev(v), (n, n))
    X = torch.randn(n, f_in, device="cuda")
    W1, b1 = torch.randn(f_in, hidden, device="cuda") * 0.05, torch.randn(hidden, device="cuda")
    W2, b2 = torch.randn(hidden, classes, device="cuda") * 0.2, torch.randn(classes, device="cuda")

    def forward(x):
        h = scorch.spmm_bias_act(A, x @ W1, b1, relu=True)
        return scorch.spmm_bias_act(A, h @ W2, b2)

    step = graphs.capture(forward, X)
    gen = torch.Generator(device="cuda").manual_seed(5)
    for _ in range(4):
        X.copy_(torch.randn(X.shape, device="cuda", generator=gen))
        want = forward(X).clone()
        torch.cuda.synchronize()
        got = step()
        torch.cuda.synchronize()
        assert got is step.result and torch.equal(got, want)
    dense = torch.sparse_csr_tensor(dev(rp).long(), dev(ci).long(), dev(v), size=(n, n)).to_dense().double()
    ref = dense @ (torch.relu(dense @ (X.double() @ W1.double()) + b1.double()) @ W2.double()) + b2.double()
    np.testing.assert_allclose(host(step()), host(ref), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("a_fmt,b_fmt", [("oo", "dd"), ("ds", "oo"), ("oo", "ds"), ("oo", "oo"), ("dd", "ds"),
                                         ("dd", "oo"), ("ds", "ds")])
@pytest.mark.parametrize("out_fmt", [None, "dd", "ds", "oo"])
def test_matmul_in_every_mix_of_matrix_formats(a_fmt, b_fmt, out_fmt, dtype):
    """What the reference's matmul accepts (ops.py:248-372: any format pair, an
    optional result format), served by re-storing operands and result around the
    prebuilt kernels."""
    torch.manual_seed(11)
    a_t = (torch.rand(37, 29) * (torch.rand(37, 29) < 0.15)).to(dtype)
    b_t = (torch.rand(29, 23) * (torch.rand(29, 23) < 0.2)).to(dtype)
    expect = a_t.double() @ b_t.double()

    def stored(t, fmt, name):
        s = STensor.from_torch(t, name)
        return (s if fmt == "dd" else s.to_sparse(fmt)).to("cuda")

    a, b = stored(a_t, a_fmt, "A"), stored(b_t, b_fmt, "B")
    kwargs = {} if out_fmt is None else {"format": out_fmt}
    out = scorch.matmul(a, b, **kwargs)
    if isinstance(out, STensor):
        assert out_fmt is None or str(out.format) == str(scorch.parse_format(out_fmt))
        assert out.values.is_cuda and out.shape == (37, 23)
        got = out.to_torch()
    else:
        assert out_fmt in (None, "dd") and out.is_cuda
        got = out
    assert torch.allclose(got.cpu().double(), expect, atol=1e-5)
    same = scorch.einsum("ik,kj->ij", a, b, **kwargs)
    same = same.to_torch() if isinstance(same, STensor) else same
    assert torch.equal(same.cpu(), got.cpu())


def test_spmv_matmul_wksp_and_precompile_follow_the_reference_signatures():
    """reference: src/scorch/ops.py:48-136 (spmv), :139-245 (matmul_wksp), :933-945"""
    torch.manual_seed(12)
    a_t = torch.rand(40, 31) * (torch.rand(40, 31) < 0.2)
    b_t = torch.rand(31, 18) * (torch.rand(31, 18) < 0.2)
    x_t = torch.rand(31)
    scorch.precompile_kernels()
    a = STensor.from_torch(a_t, "A").to_sparse("ds").to("cuda")
    y = scorch.spmv(a, STensor.from_torch(x_t, "x").to("cuda"))
    assert isinstance(y, STensor) and str(y.format) == "d" and y.shape == (40,)
    assert torch.allclose(y.to_torch().cpu(), a_t @ x_t, atol=1e-5)
    y_coo = scorch.spmv(a.to_sparse("oo"), STensor.from_torch(x_t, "x").to("cuda"))
    assert torch.allclose(y_coo.to_torch().cpu(), a_t @ x_t, atol=1e-5)
    times = {}
    c = scorch.matmul_wksp(a_t.cuda(), b_t.cuda(), time_dict=times)
    assert isinstance(c, STensor) and str(c.format) == "d,s" and times["eval_time"] > 0
    assert torch.allclose(c.to_torch().cpu(), a_t @ b_t, atol=1e-5)
    d = scorch.matmul_wksp(a, STensor.from_torch(b_t, "B").to_sparse("ds").to("cuda"), output_format="dd")
    assert isinstance(d, STensor) and d.format.is_dense()
    assert torch.allclose(d.to_torch().cpu(), a_t @ b_t, atol=1e-5)


def test_matmul_with_a_dense_torch_operand_takes_the_direct_route_and_agrees_with_the_general_one():
    """scorch.matmul(CSR STensor, torch.Tensor) calls the resolved kernel without wrapping the dense
    operand and the result; same bits as the general route, same keyword behaviour."""
    rng = np.random.default_rng(77)
    dense = (rng.random((96, 80)) < 0.1) * rng.standard_normal((96, 80))
    A = STensor.from_torch(torch.from_numpy(dense.astype(np.float32)).to_sparse_csr()).to("cuda")
    B = torch.from_numpy(rng.standard_normal((80, 24)).astype(np.float32)).cuda()
    direct = scorch.matmul(A, B)
    assert isinstance(direct, torch.Tensor) and direct.shape == (96, 24)
    general = scorch.matmul(A, STensor.from_torch(B))
    assert torch.equal(direct, general)
    np.testing.assert_allclose(host(direct), dense.astype(np.float32) @ host(B), rtol=1e-4, atol=1e-5)
    # a vector, a non-contiguous operand, the time dictionary, the other keyword routes
    x = B[:, 3].contiguous()
    assert torch.equal(scorch.matmul(A, x), scorch.matmul(A, STensor.from_torch(x)))
    Bt = torch.from_numpy(rng.standard_normal((24, 80)).astype(np.float32)).cuda().t()
    assert torch.equal(scorch.matmul(A, Bt), scorch.matmul(A, STensor.from_torch(Bt.contiguous())))
    times = {}
    assert torch.equal(scorch.matmul(A, B, time_dict=times), direct) and times["eval_time"] > 0
    assert torch.equal(scorch.matmul(A, B, use_cache=False), direct)
    as_csr = scorch.matmul(A, B, format="ds")
    assert isinstance(as_csr, STensor) and torch.equal(as_csr.to_torch(), direct)
    with pytest.raises(NotImplementedError):
        scorch.matmul(A, B.double())
