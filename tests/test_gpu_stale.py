"""What the device module keeps beside tensors must never serve old values.

The reference's call is stateless (src/scorch/prebuilt_kernels.py:198-224) and its one cache is
keyed on expression and formats, never on values (src/scorch/ops.py:425-488).  Here plans and
copies are stamped with a tensor's address, version counter and epoch; these tests write to
operands in the ways the version counter does not see -- replays of a recorded graph, ``.data``
-- and check every product against an fp64 recomputation of the values actually in memory.
"""
import numpy as np
import pytest
import torch

import scorch_amd as scorch
from conftest import random_csr
from gpu_util import dev, host
from scorch_amd import graphs
from scorch_amd import scorch_ops_hip as H

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _wide_case(rng, M=384, K=1024, N=512):
    """A product the column-tile copy applies to: rows of B of 2 KiB, every row of B used twice or more."""
    rp, ci, v = random_csr(rng, M, K, 0.02)
    assert ci.size >= 2 * K
    return rp, ci, v


def test_the_result_of_a_replayed_step_as_an_eager_operand(oracle):
    """R = A1 @ X is recorded; between replays R is multiplied eagerly by A2 (wide enough for the
    column-tile copy).  Every product must see the R of the latest replay."""
    rng = np.random.default_rng(50)
    K1, K2, N = 256, 1024, 512
    rp1, ci1, v1 = random_csr(rng, K2, K1, 0.05)
    rp2, ci2, v2 = _wide_case(rng, 384, K2, N)
    A1 = scorch.STensor.from_csr_arrays(dev(rp1), dev(ci1), dev(v1), (K2, K1))
    A2 = scorch.STensor.from_csr_arrays(dev(rp2), dev(ci2), dev(v2), (384, K2))
    X = torch.randn(K1, N, device="cuda")
    step = graphs.capture(lambda x: scorch.matmul(A1, x, format="dd"), X)
    R = step.result
    assert H.is_volatile(R) and H.is_volatile(X)
    for volatile in (True, False):
        H.mark_volatile(R, volatile=volatile)
        for replay in range(3):
            X.copy_(torch.randn(K1, N, device="cuda"))
            version = R._version
            assert step() is R
            assert R._version > version                      # a replay is a write
            want_r = oracle.spmm_fp64(rp1, ci1, v1, host(X))
            assert oracle.rel_fro(host(R), want_r) <= TOL
            want = oracle.spmm_fp64(rp2, ci2, v2, host(R).astype(np.float64))
            for _ in range(3):                               # the second product is the one that may build a copy
                got = scorch.matmul(A2, R, format="dd")
                assert oracle.rel_fro(host(got), want) <= TOL
        assert hasattr(R, "_scorch_tiled") == (not volatile)


def test_a_tiled_operand_written_through_data(oracle):
    """B.data.copy_() leaves B's version counter alone: forget(B) drops the column-tile copy, and a
    tensor marked volatile never gets one."""
    rng = np.random.default_rng(51)
    M, K, N = 384, 1024, 512
    rp, ci, v = _wide_case(rng, M, K, N)
    t_rp, t_ci, t_v = dev(rp), dev(ci), dev(v)
    B = torch.randn(K, N, device="cuda")
    product = lambda: H.spmm_csr_float_v2([M, N], [M, K], [[], [t_rp, t_ci]], t_v, [K, N], [[], []],
                                          B.reshape(-1)).storage.value.reshape(M, N)
    matches = lambda got: oracle.rel_fro(host(got), oracle.spmm_fp64(rp, ci, v, host(B).astype(np.float64))) <= TOL
    flat = B.reshape(-1)
    product_flat = lambda: H.spmm_csr_float_v2([M, N], [M, K], [[], [t_rp, t_ci]], t_v, [K, N], [[], []],
                                               flat).storage.value.reshape(M, N)
    for _ in range(3):
        assert matches(product_flat())
    assert hasattr(flat, "_scorch_tiled")
    version = flat._version
    B.data.copy_(torch.randn(K, N, device="cuda"))
    assert flat._version == version                          # the write the stamp cannot see
    H.forget(flat)
    assert not hasattr(flat, "_scorch_tiled")
    for _ in range(3):
        assert matches(product_flat())
    assert hasattr(flat, "_scorch_tiled")                    # built again, from the new values
    H.mark_volatile(flat)
    assert not hasattr(flat, "_scorch_tiled")
    for _ in range(2):
        B.data.copy_(torch.randn(K, N, device="cuda"))
        for _ in range(3):
            assert matches(product_flat())
    assert not hasattr(flat, "_scorch_tiled")
    # through matmul the copy lives on the caller's own tensor
    A = scorch.STensor.from_csr_arrays(t_rp, t_ci, t_v, (M, K))
    for _ in range(3):
        assert matches(scorch.matmul(A, B, format="dd"))
    assert hasattr(B, "_scorch_tiled")
    B.data.mul_(-3.0)
    H.forget(B)
    assert matches(scorch.matmul(A, B, format="dd"))


def _block_mask(rng, M=256):
    i, j = np.arange(M)[:, None], np.arange(M)[None, :]
    mask = j <= i
    rp = np.zeros(M + 1, np.int32)
    rp[1:] = np.cumsum(mask.sum(axis=1))
    return rp, np.nonzero(mask)[1].astype(np.int32)


def test_a_recorded_sddmm_reads_the_mask_values_of_every_replay(oracle):
    """An SDDMM over a mask of ones is recorded after a warm-up long enough for "all ones" to be
    known; the mask's values are then rewritten in place: the replay must use them."""
    rng = np.random.default_rng(52)
    M, K = 256, 64
    rp, ci = _block_mask(rng, M)
    rows = oracle.rows_of(rp)
    pos, crd = dev(rp), dev(ci)
    vals = torch.ones(ci.size, device="cuda")
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((M, K)).astype(np.float32)
    a, b = dev(A).reshape(-1), dev(B).reshape(-1)
    call = lambda values: H.sddmm_csr_float([M, M], [M, M], [[], [pos, crd]], values, [M, K], [[], []], a, [M, K],
                                            [[], []], b).storage.value
    for _ in range(4):
        eager = call(vals)
    assert isinstance(pos._scorch_plan.blocked, H.BlockedCsr) and vals._scorch_ones[1] is True
    assert oracle.rel_fro(host(eager), oracle.sddmm_fp64(rows, ci, host(vals), A, B)) <= TOL
    step = graphs.capture(call, vals, warmup=3)
    for _ in range(3):
        new = torch.from_numpy(rng.uniform(-2, 2, ci.size).astype(np.float32)).cuda()
        vals.copy_(new)
        got = step()
        assert oracle.rel_fro(host(got), oracle.sddmm_fp64(rows, ci, host(new), A, B)) <= TOL
    # eagerly, with the verdict known: a write through .data needs forget()
    H.mark_volatile(vals, volatile=False)
    vals.fill_(1.0)
    for _ in range(3):
        call(vals)
    assert vals._scorch_ones[1] is True
    vals.data.mul_(2.5)
    H.forget(vals)
    assert oracle.rel_fro(host(call(vals)), oracle.sddmm_fp64(rows, ci, host(vals), A, B)) <= TOL


def test_an_index_rewritten_through_data_is_inspected_again_after_forget():
    """A column index made out of range through .data: after forget() the next product inspects the
    index again and raises ValueError instead of launching a gather that reads out of bounds."""
    rng = np.random.default_rng(53)
    M, K, N = 200, 300, 64
    rp, ci, v = random_csr(rng, M, K, 0.05)
    pos, crd, vals = dev(rp), dev(ci), dev(v)
    B = torch.randn(K * N, device="cuda")
    product = lambda: H.spmm_csr_float_v2([M, N], [M, K], [[], [pos, crd]], vals, [K, N], [[], []], B)
    product()
    plan = pos._scorch_plan
    version = crd._version
    crd.data[5] = K + 7
    assert crd._version == version and pos._scorch_plan is plan
    H.forget(crd)                                            # the plan lives on pos; forgetting either index drops it
    with pytest.raises(ValueError, match="column index"):
        product()
    crd.data[5] = int(ci[5])
    H.forget(crd)
    product()
    assert pos._scorch_plan is not plan
    # and a write PyTorch does version needs no forget()
    crd[5] = K + 7
    with pytest.raises(ValueError, match="column index"):
        product()
    # forgetting the whole operand at once
    crd[5] = int(ci[5])
    A = scorch.STensor.from_csr_arrays(pos, crd, vals, (M, K))
    scorch.matmul(A, B.reshape(K, N), format="dd")
    pos.data[3] = -1                                         # a row pointer that decreases
    H.forget(A)
    with pytest.raises(ValueError, match="row_ptr"):
        scorch.matmul(A, B.reshape(K, N), format="dd")


def test_a_new_index_tensor_at_a_freed_tensors_address_is_not_taken_for_it():
    """The plan lives on the row pointer and names the column indices by address, version and
    length -- and by identity: the allocator hands a freed tensor's address to the next tensor of
    its size, which must be inspected as the new operand it is."""
    pos = dev(np.array([0, 2, 4], np.int32))
    B = torch.ones(8 * 16, device="cuda")
    vals = torch.ones(4, device="cuda")
    product = lambda crd: H.spmm_csr_float_v2([2, 16], [2, 8], [[], [pos, crd]], vals, [8, 16], [[], []], B)
    crd = dev(np.array([0, 3, 1, 7], np.int32))
    address = crd.data_ptr()
    product(crd)
    assert pos._scorch_plan.partner() is crd
    del crd
    for _ in range(4):                                       # the caching allocator reuses the block
        crd = dev(np.array([0, 3, 1, 8], np.int32))          # column 8 of 8
        if crd.data_ptr() == address:
            break
    with pytest.raises(ValueError, match="column index"):
        product(crd)
