"""scorch_hip_spmm_csr_f32_static: the SpMM entry point that allocates nothing
(its carry records live in a static device array inside the library) against
scorch_hip_spmm_csr_f32 on the same operands, through the C ABI, bit for bit.
Two calls in a row, the second on a smaller input, so that whatever the first
left in the shared array must not leak into the second."""
import numpy as np
import pytest
import torch

from scorch_amd import native, workloads

pytestmark = pytest.mark.gpu


def _operands(w):
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t(w["row_ptr"]), t(w["col_idx"]), t(w["vals"]), t(w["B"]).reshape(-1)


def _with_workspace(L, w, pos, crd, val, B):
    M, K, N, nnz = w["M"], w["K"], w["N"], int(w["col_idx"].size)
    C = torch.full((M * N,), float("nan"), device="cuda")
    ws = torch.empty(L.scorch_hip_spmm_csr_workspace_bytes(M, nnz, N, 4), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    native.check(L.scorch_hip_spmm_csr_f32(M, K, N, nnz, pos.data_ptr(), crd.data_ptr(), val.data_ptr(),
                                           B.data_ptr(), C.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    return C


def _static(L, w, pos, crd, val, B):
    M, K, N, nnz = w["M"], w["K"], w["N"], int(w["col_idx"].size)
    C = torch.full((M * N,), float("nan"), device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    native.check(L.scorch_hip_spmm_csr_f32_static(M, K, N, nnz, pos.data_ptr(), crd.data_ptr(), val.data_ptr(),
                                                  B.data_ptr(), C.data_ptr(), stream))
    return C


def test_static_scratch_entry_matches_the_workspace_entry_twice_in_a_row():
    L = native.lib()
    # rows of up to 20,000 entries: hundreds of chunks leave carries, so the scratch is really used
    big = workloads.gcn_powerlaw(M=60_000, N=128, seed=21, max_degree=20_000)
    small = workloads.gcn_powerlaw(M=3_000, N=96, seed=22, max_degree=1_500)
    for w in (big, small):
        ops = _operands(w)
        want = _with_workspace(L, w, *ops)
        got = _static(L, w, *ops)
        torch.cuda.synchronize()
        assert torch.isfinite(got).all()
        assert torch.equal(got, want), (w["M"], w["N"])


def test_static_scratch_entry_refuses_what_does_not_fit():
    L = native.lib()
    M, nnz, N = 1 << 20, 60_000_000, 512
    assert L.scorch_hip_spmm_csr_workspace_bytes(M, nnz, N, 4) > (48 << 20)
    one = torch.zeros(1, device="cuda")
    rc = L.scorch_hip_spmm_csr_f32_static(M, M, N, nnz, one.data_ptr(), one.data_ptr(), one.data_ptr(),
                                          one.data_ptr(), one.data_ptr(), None)
    assert rc == native.EWORKSPACE and "static buffer" in native.last_error()
