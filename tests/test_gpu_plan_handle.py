"""The plan handle of include/scorch_hip.h (scorch_hip_csr_plan_*): one object per CSR pattern,
one call per product, the library choosing the kernel.  Every product is checked against the
CPU oracle and, bit for bit, against the entry points it stands for."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import random_csr
from gpu_util import dev, hip_sddmm_csr, hip_spmm, host
from scorch_amd import native, workloads
from scorch_amd.csr_plan import (PLAN_SDDMM_F32, PLAN_SOFTMAX_F32, PLAN_SPMM_DENSE_F32, PLAN_SPMM_F32, CsrPlanHandle,
                                 DensePlanHandle)

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _direct_spmm(rp, ci, v, B, bias=None, relu=False):
    """scorch_hip_spmm_csr_f32 / _bias_act_f32 with a workspace of the caller's: no plan anywhere."""
    L = native.lib()
    M, (K, N) = rp.numel() - 1, B.shape
    ws = torch.empty(max(L.scorch_hip_spmm_csr_workspace_bytes(M, ci.numel(), N, 4), 1), dtype=torch.uint8,
                     device="cuda")
    out = torch.full((M, N), float("nan"), device="cuda")
    if bias is None:
        rc = L.scorch_hip_spmm_csr_f32(M, K, N, ci.numel(), rp.data_ptr(), ci.data_ptr(), v.data_ptr(), B.data_ptr(),
                                       out.data_ptr(), ws.data_ptr(), ws.numel(), _stream())
    else:
        rc = L.scorch_hip_spmm_csr_bias_act_f32(M, K, N, ci.numel(), rp.data_ptr(), ci.data_ptr(), v.data_ptr(),
                                                B.data_ptr(), bias.data_ptr(), int(relu), out.data_ptr(),
                                                ws.data_ptr(), ws.numel(), _stream())
    native.check(rc)
    return host(out)


def _operands(kind, rng):
    if kind == "short_rows":                      # all rows short: the row-split kernel
        rp, ci, v = random_csr(rng, 3000, 2500, 0.01)
        K, N = 2500, 48
    elif kind == "long_rows":                     # a power-law graph: the merge-path kernels
        w = workloads.gcn_powerlaw(M=20_000, N=1, seed=11, max_degree=6000)
        rp, ci, v = w["row_ptr"], w["col_idx"], w["vals"]
        K, N = 20_000, 64
    else:                                         # most rows empty and a 33 MB result: filled first
        M, K, N = 131_072, 4096, 64
        lens = np.where(rng.random(M) < 0.2, rng.integers(1, 40, M), 0)
        lens[7] = 700
        rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        ci = rng.integers(0, K, rp[-1]).astype(np.int32)
        v = rng.uniform(-1, 1, rp[-1]).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    return rp, ci, v, B


@pytest.mark.parametrize("kind", ["short_rows", "long_rows", "mostly_empty"])
def test_spmm_through_a_plan(kind, oracle):
    rng = np.random.default_rng(3)
    rp, ci, v, B = _operands(kind, rng)
    bias = rng.uniform(-1, 1, B.shape[1]).astype(np.float32)
    d_rp, d_ci, d_v, d_B, d_bias = dev(rp), dev(ci), dev(v), dev(B), dev(bias)
    with CsrPlanHandle(d_rp, d_ci, B.shape[0]) as plan:
        info = plan.info()
        lens = np.diff(rp)
        assert (info["M"], info["n_cols"], info["nnz"]) == (len(rp) - 1, B.shape[0], len(ci))
        assert info["longest_row"] == lens.max() and info["empty_rows"] == (lens == 0).sum()
        got = host(plan.spmm(d_v, d_B))
        again = host(plan.spmm(d_v, d_B))
        with_bias = host(plan.spmm(d_v, d_B, d_bias))
        with_relu = host(plan.spmm(d_v, d_B, d_bias, relu=True))
        held = plan.info()["device_bytes"]
    assert (held == 0) == (kind == "short_rows")         # the row-split kernel needs nothing kept
    assert np.array_equal(got, again)
    assert oracle.rel_fro(got, oracle.spmm_fp64(rp, ci, v, B)) <= TOL
    # the host layer plans the same operand the same way: same kernel, same bits
    assert np.array_equal(got, hip_spmm(rp, ci, v, B))
    assert np.array_equal(with_bias, hip_spmm(rp, ci, v, B, bias=bias))
    assert np.array_equal(with_relu, np.maximum(with_bias, 0))
    direct = _direct_spmm(d_rp, d_ci, d_v, d_B)
    if kind == "short_rows":
        np.testing.assert_allclose(got, direct, rtol=1e-4, atol=1e-5)
    else:
        assert np.array_equal(got, direct)
        assert np.array_equal(with_relu, _direct_spmm(d_rp, d_ci, d_v, d_B, d_bias, relu=True))


def test_a_plan_keeps_boundaries_for_eight_widths_and_replaces_the_oldest(oracle):
    w = workloads.gcn_powerlaw(M=6000, N=1, seed=4, max_degree=3000)
    rp, ci, v = w["row_ptr"], w["col_idx"], w["vals"]
    rng = np.random.default_rng(0)
    d_rp, d_ci, d_v = dev(rp), dev(ci), dev(v)
    L = native.lib()
    kept, workspace = [], 0                      # what the plan should hold: the widths, oldest use first
    with CsrPlanHandle(d_rp, d_ci, 6000) as plan:
        for N in (8, 16, 24, 32, 40, 48, 56, 64, 72, 8, 128, 16):
            B = rng.uniform(-1, 1, (6000, N)).astype(np.float32)
            got = host(plan.spmm(d_v, dev(B)))
            assert oracle.rel_fro(got, oracle.spmm_fp64(rp, ci, v, B)) <= TOL, N
            assert np.array_equal(got, _direct_spmm(d_rp, d_ci, d_v, dev(B))), N
            if N in kept:
                kept.remove(N)
            elif len(kept) == 8:
                kept.pop(0)                      # the ninth width takes the place of the oldest
            kept.append(N)
            workspace = max(workspace, L.scorch_hip_spmm_csr_workspace_bytes(6000, len(ci), N, 4))
            bounds = sum(L.scorch_hip_spmm_csr_bounds_bytes(6000, len(ci), n, 4) for n in kept)
            assert plan.info()["device_bytes"] == workspace + bounds, (N, kept)


def test_sddmm_through_a_plan(oracle):
    rng = np.random.default_rng(5)
    # (a) a small mask: the general kernel
    rp, ci, s = random_csr(rng, 700, 900, 0.03)
    A = rng.uniform(-1, 1, (700, 40)).astype(np.float32)
    B = rng.uniform(-1, 1, (900, 40)).astype(np.float32)
    with CsrPlanHandle(dev(rp), dev(ci), 900) as plan:
        rows = torch.full((len(ci),), -1, dtype=torch.int32, device="cuda")
        got = host(plan.sddmm(dev(s), dev(A), dev(B), rows))
        ones = host(plan.sddmm(None, dev(A), dev(B)))
        assert plan.info()["device_bytes"] == 0
    r_ref, c_ref, v_ref = hip_sddmm_csr(rp, ci, s, A, B, (700, 900))
    assert np.array_equal(host(rows), r_ref) and np.array_equal(got, v_ref)
    want = oracle.sddmm_fp64(oracle.rows_of(rp), ci, s, A, B)
    assert oracle.rel_fro(got, want) <= TOL
    assert oracle.rel_fro(ones, oracle.sddmm_fp64(oracle.rows_of(rp), ci, np.ones_like(s), A, B)) <= TOL
    # (b) a dense right operand of 8 MB and four entries per column or more: per-XCD entry lists
    M, n_cols, K = 4096, 65_536, 32
    lens = rng.integers(70, 100, M)
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(n_cols, n, replace=False)) for n in lens]).astype(np.int32)
    s = rng.uniform(-1, 1, len(ci)).astype(np.float32)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (n_cols, K)).astype(np.float32)
    d_rp, d_ci = dev(rp), dev(ci)
    with CsrPlanHandle(d_rp, d_ci, n_cols) as plan:
        plan.prepare(PLAN_SDDMM_F32, K)
        assert plan.info()["device_bytes"] >= 12 * len(ci)           # the lists exist
        rows = torch.full((len(ci),), -1, dtype=torch.int32, device="cuda")
        got = host(plan.sddmm(dev(s), dev(A), dev(B), rows))
        ones = host(plan.sddmm(None, dev(A), dev(B)))
    L = native.lib()
    plain = torch.empty(len(ci), device="cuda")
    d_s, d_A, d_B = dev(s), dev(A), dev(B)       # (named: a temporary's memory is handed out again at once)
    native.check(L.scorch_hip_sddmm_csr_f32(M, n_cols, K, len(ci), d_rp.data_ptr(), d_ci.data_ptr(), d_s.data_ptr(),
                                            d_A.data_ptr(), d_B.data_ptr(), plain.data_ptr(), None, _stream()))
    assert np.array_equal(got, host(plain))                          # the listed kernel gives the same bits
    assert np.array_equal(host(rows), oracle.rows_of(rp))
    assert oracle.rel_fro(got, oracle.sddmm_fp64(oracle.rows_of(rp), ci, s, A, B)) <= TOL
    assert oracle.rel_fro(ones, oracle.sddmm_fp64(oracle.rows_of(rp), ci, np.ones_like(s), A, B)) <= TOL


@pytest.mark.parametrize("longest", [300, 9000])
def test_softmax_through_a_plan(longest, oracle):
    rng = np.random.default_rng(longest)
    lens = rng.integers(0, 60, 500)
    lens[3] = longest
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(10_000, n, replace=False)) for n in lens]).astype(np.int32)
    v = rng.uniform(-6, 6, len(ci)).astype(np.float32)
    d_rp, d_v = dev(rp), dev(v)
    with CsrPlanHandle(d_rp, dev(ci), 10_000) as plan:
        plan.prepare(PLAN_SOFTMAX_F32)
        got = host(plan.softmax(d_v, 0.5))
    np.testing.assert_allclose(got, oracle.softmax_csr_fp64(rp, v, 0.5), rtol=2e-6, atol=1e-9)
    L = native.lib()
    ws = torch.empty(max(L.scorch_hip_softmax_csr_workspace_bytes(500, len(ci)), 1), dtype=torch.uint8, device="cuda")
    direct = torch.empty(len(ci), device="cuda")
    native.check(L.scorch_hip_softmax_csr_f32(500, len(ci), d_rp.data_ptr(), d_v.data_ptr(), 0.5, direct.data_ptr(),
                                              ws.data_ptr(), ws.numel(), _stream()))
    assert np.array_equal(got, host(direct))


def test_a_malformed_index_gets_no_plan():
    good_rp, good_ci = np.array([0, 2, 2, 5], np.int32), np.array([0, 3, 1, 2, 3], np.int32)
    CsrPlanHandle(dev(good_rp), dev(good_ci), 4).close()
    for rp, ci, what in ((good_rp, [0, 4, 1, 2, 3], "column index"), (good_rp, [0, 3, -1, 2, 3], "column index"),
                         ([0, 3, 2, 5], good_ci, "row_ptr"), ([1, 2, 2, 5], good_ci, "row_ptr"),
                         ([0, 2, 2, 4], good_ci, "row_ptr")):
        with pytest.raises(native.ScorchHipError, match=what) as err:
            CsrPlanHandle(dev(np.array(rp, np.int32)), dev(np.array(ci, np.int32)), 4)
        assert err.value.code == native.EINVAL
    # an empty matrix is a matrix
    with CsrPlanHandle(dev(np.zeros(1, np.int32)), dev(np.zeros(0, np.int32)), 4) as plan:
        out = plan.spmm(torch.empty(0, device="cuda"), torch.ones(4, 8, device="cuda"))
        assert out.shape == (0, 8)
    with CsrPlanHandle(dev(np.zeros(6, np.int32)), dev(np.zeros(0, np.int32)), 4) as plan:
        out = plan.spmm(torch.empty(0, device="cuda"), torch.ones(4, 8, device="cuda"))
        assert host(out).shape == (5, 8) and not host(out).any()
        assert plan.sddmm(None, torch.ones(5, 3, device="cuda"), torch.ones(4, 3, device="cuda")).numel() == 0
        assert plan.softmax(torch.empty(0, device="cuda")).numel() == 0
    torch.cuda.synchronize()


def test_a_closed_plan_and_bad_arguments_are_refused():
    L = native.lib()
    plan = CsrPlanHandle(dev(np.array([0, 1], np.int32)), dev(np.array([0], np.int32)), 1)
    assert L.scorch_hip_csr_plan_prepare(plan._handle, 17, 0, None) == native.EINVAL
    assert L.scorch_hip_csr_plan_prepare(plan._handle, PLAN_SPMM_F32, -1, None) == native.EINVAL
    one = torch.ones(1, device="cuda")
    assert L.scorch_hip_spmm_csr_plan_f32(plan._handle, 1, one.data_ptr(), one.data_ptr(), None, 5, one.data_ptr(),
                                          None) == native.EINVAL
    plan.close()
    plan.close()                                     # closing twice is closing once
    with pytest.raises(RuntimeError, match="closed"):
        plan.spmm(one, one.reshape(1, 1))
    info = (ctypes.c_int64 * 8)()
    assert L.scorch_hip_csr_plan_info(None, info) == native.EINVAL
    assert L.scorch_hip_csr_plan_destroy(None) == native.OK


def test_prepared_products_replay_from_a_graph(oracle):
    """After scorch_hip_csr_plan_prepare the product calls allocate nothing and wait for
    nothing: they can be recorded into a HIP graph, and every replay gives the eager bits."""
    w = workloads.gcn_powerlaw(M=8000, N=1, seed=2, max_degree=3000)
    rp, ci, v = w["row_ptr"], w["col_idx"], w["vals"]
    rng = np.random.default_rng(1)
    B = rng.uniform(-1, 1, (8000, 32)).astype(np.float32)
    d_v, d_B = dev(v), dev(B)
    with CsrPlanHandle(dev(rp), dev(ci), 8000) as plan:
        plan.prepare(PLAN_SPMM_F32, 32)
        eager = host(plan.spmm(d_v, d_B))
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = plan.spmm(d_v, d_B)
        for replay in range(3):
            d_B.mul_(2.0)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            want = oracle.spmm_fp64(rp, ci, v, B * 2.0 ** (replay + 1))
            assert oracle.rel_fro(host(out), want) <= TOL, replay
            assert np.array_equal(host(out), eager * np.float32(2.0 ** (replay + 1))), replay
        del graph


def test_a_reused_dense_operand_through_its_plan(oracle):
    """The decoder shape in small: B with rows of 2 KiB, gathered several times over.  Through the
    two plans the product takes the column-tile copy; it equals the Python layer's tiled path bit
    for bit, follows B's values only after update(), and replays from a graph."""
    rng = np.random.default_rng(8)
    M, K, N = 1500, 2048, 512
    rp, ci, v = random_csr(rng, M, K, 0.02)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    bias = rng.uniform(-1, 1, N).astype(np.float32)
    d_v, d_B, d_bias = dev(v), dev(B), dev(bias)
    with CsrPlanHandle(dev(rp), dev(ci), K) as plan, DensePlanHandle(d_B) as dense:
        plan.prepare(PLAN_SPMM_DENSE_F32, N)
        assert plan.info()["device_bytes"] > 0
        got = host(plan.spmm_dense(d_v, dense))
        assert oracle.rel_fro(got, oracle.spmm_fp64(rp, ci, v, B)) <= TOL
        assert np.array_equal(got, hip_spmm(rp, ci, v, B, path="tiled"))
        with_relu = host(plan.spmm_dense(d_v, dense, d_bias, relu=True))
        assert np.array_equal(with_relu, hip_spmm(rp, ci, v, B, bias=bias, relu=True, path="tiled"))
        np.testing.assert_allclose(got, host(plan.spmm(d_v, d_B)), rtol=1e-4, atol=1e-5)
        # new values in B: the plan's copy is the caller's to refresh
        d_B.mul_(2.0)
        assert np.array_equal(host(plan.spmm_dense(d_v, dense)), got)
        dense.update()
        assert np.array_equal(host(plan.spmm_dense(d_v, dense)), got * np.float32(2))
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = plan.spmm_dense(d_v, dense)
        for replay in range(3):
            d_v.mul_(0.5)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert np.array_equal(host(out), got * np.float32(2.0 * 0.5 ** (replay + 1))), replay
        del graph
    # a shape the tile layout does not pay for: the same call is the ordinary planned product
    B2 = rng.uniform(-1, 1, (K, 48)).astype(np.float32)
    with CsrPlanHandle(dev(rp), dev(ci), K) as plan, DensePlanHandle(dev(B2)) as dense:
        assert np.array_equal(host(plan.spmm_dense(d_v, dense)), host(plan.spmm(d_v, dense.B)))
    L = native.lib()
    assert L.scorch_hip_dense_plan_destroy(None) == native.OK
    assert L.scorch_hip_dense_plan_update(None, None) == native.EINVAL
    with CsrPlanHandle(dev(rp), dev(ci), K) as plan, DensePlanHandle(torch.ones(K + 1, 8, device="cuda")) as dense:
        with pytest.raises(native.ScorchHipError):
            plan.spmm_dense(d_v, dense)                      # K does not match


def test_a_c_host_of_the_library():
    """tests/host_c/plan_demo.c, built by scorch_amd.build.build_host_demo: a C99 program with the
    C ABI and the HIP runtime and nothing else does the stateless SpMM, the planned SpMM, SDDMM and
    softmax, checks them against its own loops in double, and sees a malformed index refused."""
    import os
    import subprocess
    from scorch_amd import build
    if not os.path.exists(build.HOST_DEMO_BIN):
        pytest.skip("tests/host_c/plan_demo is not built (python -m scorch_amd.build)")
    proc = subprocess.run([build.HOST_DEMO_BIN], capture_output=True, text=True, timeout=100)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.strip().endswith("ok"), proc.stdout
    assert "bit-identical: 1" in proc.stdout
