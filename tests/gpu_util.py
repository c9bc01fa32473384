"""Helpers for the GPU parity tests: move numpy inputs to the device and call
the kernels through scorch_ops_hip, i.e. through the C ABI of libscorch_hip.so."""
import numpy as np
import torch

from scorch_amd import scorch_ops_hip as H

SPMM_SYMBOL = {np.dtype(np.float32): "spmm_csr_float_v2", np.dtype(np.float64): "prebuilt_spmm_csr_f64",
               np.dtype(np.int32): "prebuilt_spmm_csr_i32", np.dtype(np.int64): "prebuilt_spmm_csr_i64"}
SPMV_SYMBOL = {np.dtype(np.float32): "prebuilt_spmv_csr_f32", np.dtype(np.float64): "prebuilt_spmv_csr_f64",
               np.dtype(np.int32): "prebuilt_spmv_csr_i32", np.dtype(np.int64): "prebuilt_spmv_csr_i64"}


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


class spmm_path:
    """``with spmm_path("rows"):`` pins the SpMM kernel the wrappers choose."""

    def __init__(self, path):
        self.path = path

    def __enter__(self):
        self.previous, H.SPMM_PATH = H.SPMM_PATH, self.path or H.SPMM_PATH

    def __exit__(self, *exc):
        H.SPMM_PATH = self.previous
        return False


def hip_spmm(row_ptr, col_idx, vals, B, bias=None, relu=False, K=None, path=None):
    with spmm_path(path):
        return _hip_spmm(row_ptr, col_idx, vals, B, bias, relu, K)


def _hip_spmm(row_ptr, col_idx, vals, B, bias, relu, K):
    M, N = len(row_ptr) - 1, B.shape[1]
    K = B.shape[0] if K is None else K
    args = ([M, N], [M, K], [[], [dev(row_ptr), dev(col_idx)]], dev(vals), [K, N], [[], []],
            dev(B).reshape(-1))
    if bias is None:
        out = getattr(H, SPMM_SYMBOL[np.dtype(vals.dtype)])(*args)
    elif relu:
        out = H.spmm_csr_bias_relu_float(*args, dev(bias))
    else:
        out = H.spmm_csr_bias_float(*args, dev(bias))
    assert out.storage.index.mode_indices == [[], []]
    return host(out.storage.value).reshape(M, N)


def hip_spmv(row_ptr, col_idx, vals, x):
    M, K = len(row_ptr) - 1, x.shape[0]
    out = getattr(H, SPMV_SYMBOL[np.dtype(vals.dtype)])(
        [M], [M, K], [[], [dev(row_ptr), dev(col_idx)]], dev(vals), [K], [[]], dev(x))
    return host(out.storage.value)


def hip_sddmm_coo(row_idx, col_idx, svals, A, B, shape):
    r, c = dev(row_idx), dev(col_idx)
    out = H.sddmm_coo_float_prebuilt(list(shape), list(shape), [[r], [c]], dev(svals), list(A.shape),
                                     [[], []], dev(A).reshape(-1), list(B.shape), [[], []],
                                     dev(B).reshape(-1))
    idx = out.storage.index.mode_indices
    assert idx[0][0] is r and idx[1][0] is c  # the mask's own index tensors come back
    return host(out.storage.value)


def hip_sddmm_csr(row_ptr, col_idx, svals, A, B, shape):
    out = H.sddmm_csr_float(list(shape), list(shape), [[], [dev(row_ptr), dev(col_idx)]], dev(svals),
                            list(A.shape), [[], []], dev(A).reshape(-1), list(B.shape), [[], []],
                            dev(B).reshape(-1))
    idx = out.storage.index.mode_indices
    return host(idx[0][0]), host(idx[1][0]), host(out.storage.value)
