"""Python face of the CPU checker.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the shipped package never does.

Three layers, from most to least trusted as ground truth:

* ``*_fp64``     -- float64 recomputation with numpy/scipy: what the
                    mathematics fixes.  The tolerance checks (relative
                    Frobenius error) are taken against these.
* ``ref_*``      -- the reference's own native module, compiled from its
                    sources into ``oracle/_ref/scorch_ops.so`` by
                    ``oracle/Makefile``; present only where that was built.
* the C restatement in ``scorch_oracle.c`` (``liboracle.so``), wrapped by the
  plain functions below.  It follows the reference loop by loop and is what
  gets timed as the CPU baseline when ``_ref`` is absent.

What pins each restatement (tests/test_oracle_golden.py, test_oracle_math.py,
test_oracle_ref.py):

* spmm_csr_f32_v2, spmm_csr_typed, spmm_csr_bias_act_f32, sddmm_coo_f32,
  sddmm_csr_f32, spmv_csr_typed, spgemm_csr_typed, spmm_coo_f32,
  spgemm_coo_f32: the reference's own outputs (golden fixtures written by its
  compiled native module, and that module live where it is built), plus closed
  forms and brute force.
* softmax_csr_f32 / softmax_csr_fp64 and attention_dense_fp64 /
  attention_blocksparse_fp64: PARITY UNPINNED against the reference -- it has
  no native kernel, test or stored vector for the row softmax or for fused
  attention (it composes them from torch operations in a benchmark script).
  They are pinned by mathematics only: scipy.special.softmax, shift
  invariance, rows summing to one, and the SDDMM -> softmax -> SpMM pipeline
  equalling masked dense attention.
"""
from __future__ import annotations

import ctypes
import importlib.util
import os
import subprocess
import sys
from typing import Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "scorch_ops.so")

_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")


def build(force: bool = False) -> None:
    """Compile liboracle.so (and _ref/scorch_ops.so where the reference
    sources are present) with oracle/Makefile."""
    targets = ["liboracle.so", "ref"]
    cmd = ["make", "-C", _HERE] + (["-B"] if force else []) + targets
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)


_lib = None
_NATIVE_LIB_PATH = os.path.join(_HERE, "liboracle_native.so")


def host_has_avx512() -> bool:
    """The prebuilt binaries here are compiled for x86-64-v4 (oracle/Makefile): on a host without
    AVX-512 their first vector instruction would kill the process with SIGILL, which no
    ``try`` can catch -- so the flags are read before anything is loaded."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("flags"):
                    flags = set(line.split(":", 1)[1].split())
                    return {"avx512f", "avx512bw", "avx512cd", "avx512dq", "avx512vl"} <= flags
    except OSError:
        pass
    return False


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = _LIB_PATH
        if not host_has_avx512():
            # this host cannot run the prebuilt library: compile the restatement for it
            path = _NATIVE_LIB_PATH
            if not os.path.exists(path):
                subprocess.run(["make", "-C", _HERE, "-B", "MARCH=native", "LIB=liboracle_native.so",
                                "liboracle_native.so"], check=True, stdout=subprocess.DEVNULL)
        elif not os.path.exists(path):
            build()
        _lib = ctypes.CDLL(path)
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


_NP_SUFFIX = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64",
              np.dtype(np.int32): "i32", np.dtype(np.int64): "i64"}


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


# --------------------------------------------------------------------------
# C restatement
# --------------------------------------------------------------------------
def spmm_csr_f32_v2(row_ptr, col_idx, vals, B, tile: int = 256, out: Optional[np.ndarray] = None,
                    zero_fill: bool = True) -> np.ndarray:
    """C = A @ B, the loop of spmm_csr_float_v2 (csrc/spmm.h:2007-2089)."""
    row_ptr, col_idx = _c(row_ptr, np.int32), _c(col_idx, np.int32)
    vals, B = _c(vals, np.float32), _c(B, np.float32)
    M, N = row_ptr.size - 1, B.shape[1]
    if out is None:
        out = np.empty((M, N), dtype=np.float32)
    lib().oracle_spmm_csr_f32_v2(ctypes.c_int(M), ctypes.c_int(N), _ptr(row_ptr), _ptr(col_idx),
                                 _ptr(vals), _ptr(B), _ptr(out), ctypes.c_int(tile),
                                 ctypes.c_int(1 if zero_fill else 0))
    return out


def spmm_csr_typed(row_ptr, col_idx, vals, B) -> np.ndarray:
    """C = A @ B for f32/f64/i32/i64, the loop of spmm_csr_typed<T>
    (csrc/spmm.h:91-150)."""
    vals = np.ascontiguousarray(vals)
    suffix = _NP_SUFFIX[vals.dtype]
    row_ptr, col_idx = _c(row_ptr, np.int32), _c(col_idx, np.int32)
    B = _c(B, vals.dtype)
    M, N = row_ptr.size - 1, B.shape[1]
    out = np.empty((M, N), dtype=vals.dtype)
    getattr(lib(), "oracle_spmm_csr_" + suffix)(ctypes.c_int(M), ctypes.c_int(N), _ptr(row_ptr),
                                                _ptr(col_idx), _ptr(vals), _ptr(B), _ptr(out))
    return out


def spmm_csr_bias_act_f32(row_ptr, col_idx, vals, B, bias, relu: bool) -> np.ndarray:
    """C = act(A @ B + bias), the loop of spmm_csr_bias_act (csrc/spmm.h:28-89)."""
    row_ptr, col_idx = _c(row_ptr, np.int32), _c(col_idx, np.int32)
    vals, B, bias = _c(vals, np.float32), _c(B, np.float32), _c(bias, np.float32)
    M, N = row_ptr.size - 1, B.shape[1]
    out = np.empty((M, N), dtype=np.float32)
    lib().oracle_spmm_csr_bias_act_f32(ctypes.c_int(M), ctypes.c_int(N), _ptr(row_ptr), _ptr(col_idx),
                                       _ptr(vals), _ptr(B), _ptr(bias), _ptr(out),
                                       ctypes.c_int(1 if relu else 0))
    return out


def sddmm_coo_f32(row_idx, col_idx, svals, A, B) -> np.ndarray:
    """out[p] = s[p] * <A[row[p]], B[col[p]]>, the loop of
    sddmm_coo_float_prebuilt (csrc/kernels.h:508-570)."""
    row_idx, col_idx = _c(row_idx, np.int32), _c(col_idx, np.int32)
    svals, A, B = _c(svals, np.float32), _c(A, np.float32), _c(B, np.float32)
    out = np.empty(svals.size, dtype=np.float32)
    lib().oracle_sddmm_coo_f32(ctypes.c_int64(svals.size), ctypes.c_int(A.shape[1]), _ptr(row_idx),
                               _ptr(col_idx), _ptr(svals), _ptr(A), _ptr(B), _ptr(out))
    return out


def sddmm_csr_f32(row_ptr, col_idx, svals, A, B) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """SDDMM with a CSR mask; returns the coordinate-format result
    (row, col, val) the reference's generated kernel produces for a "d,s"
    mask (src/scorch/ops.py:638-666, compiler/cin_lowerer.py:2286-2326)."""
    row_ptr, col_idx = _c(row_ptr, np.int32), _c(col_idx, np.int32)
    svals, A, B = _c(svals, np.float32), _c(A, np.float32), _c(B, np.float32)
    nnz = svals.size
    out_row = np.empty(nnz, dtype=np.int32)
    out_col = np.empty(nnz, dtype=np.int32)
    out_val = np.empty(nnz, dtype=np.float32)
    lib().oracle_sddmm_csr_f32(ctypes.c_int(row_ptr.size - 1), ctypes.c_int(A.shape[1]), _ptr(row_ptr),
                               _ptr(col_idx), _ptr(svals), _ptr(A), _ptr(B), _ptr(out_row),
                               _ptr(out_col), _ptr(out_val))
    return out_row, out_col, out_val


def spmv_csr_typed(row_ptr, col_idx, vals, x) -> np.ndarray:
    """y = A @ x for f32/f64/i32/i64, the loop of spmv_csr<T>
    (csrc/kernels.h:13-49)."""
    vals = np.ascontiguousarray(vals)
    suffix = _NP_SUFFIX[vals.dtype]
    row_ptr, col_idx = _c(row_ptr, np.int32), _c(col_idx, np.int32)
    x = _c(x, vals.dtype)
    M = row_ptr.size - 1
    out = np.empty(M, dtype=vals.dtype)
    getattr(lib(), "oracle_spmv_csr_" + suffix)(ctypes.c_int(M), _ptr(row_ptr), _ptr(col_idx),
                                                _ptr(vals), _ptr(x), _ptr(out))
    return out


def spgemm_csr_typed(a_row_ptr, a_col_idx, a_vals, b_row_ptr, b_col_idx, b_vals, n_cols: int):
    """C = A @ B with all three in CSR, f32/f64/i32/i64: the three phases of
    spmspm_csr<T> (csrc/kernels.h:52-202).  Returns (row_ptr, col_idx, vals);
    columns ascending within a row, structural zeros kept."""
    a_vals = np.ascontiguousarray(a_vals)
    suffix = _NP_SUFFIX[a_vals.dtype]
    a_pos, a_crd = _c(a_row_ptr, np.int32), _c(a_col_idx, np.int32)
    b_pos, b_crd, b_vals = _c(b_row_ptr, np.int32), _c(b_col_idx, np.int32), _c(b_vals, a_vals.dtype)
    M = a_pos.size - 1
    c_pos = np.zeros(M + 1, dtype=np.int32)
    lib().oracle_spgemm_csr_count(ctypes.c_int(M), ctypes.c_int(n_cols), _ptr(a_pos), _ptr(a_crd),
                                  _ptr(b_pos), _ptr(b_crd), _ptr(c_pos))
    nnz = int(c_pos[-1])
    c_crd = np.zeros(nnz, dtype=np.int32)
    c_val = np.zeros(nnz, dtype=a_vals.dtype)
    getattr(lib(), "oracle_spgemm_csr_" + suffix)(ctypes.c_int(M), ctypes.c_int(n_cols), _ptr(a_pos),
                                                  _ptr(a_crd), _ptr(a_vals), _ptr(b_pos), _ptr(b_crd),
                                                  _ptr(b_vals), _ptr(c_pos), _ptr(c_crd), _ptr(c_val))
    return c_pos, c_crd, c_val


def _runs(keys: np.ndarray):
    """(start, end) of every run of equal neighbouring values, in order."""
    if keys.size == 0:
        return []
    cuts = np.flatnonzero(keys[1:] != keys[:-1]) + 1
    starts = np.concatenate([[0], cuts])
    ends = np.concatenate([cuts, [keys.size]])
    return list(zip(starts.tolist(), ends.tolist()))


def spmm_coo_f32(row_idx, col_idx, vals, B, n_rows: int) -> np.ndarray:
    """C = A @ B for A as coordinates (csrc/spmm.h:247-372): each run of equal
    neighbouring rows is summed into a zeroed workspace, entry by entry, and the
    workspace added to that row of C; repeated coordinates therefore add up and
    the order of the runs does not matter beyond rounding.  fp32 throughout."""
    rows, cols, vals = _c(row_idx, np.int32), _c(col_idx, np.int32), _c(vals, np.float32)
    B = _c(B, np.float32)
    C = np.zeros((n_rows, B.shape[1]), dtype=np.float32)
    for lo, hi in _runs(rows):
        wksp = np.zeros(B.shape[1], dtype=np.float32)
        for p in range(lo, hi):
            wksp += vals[p] * B[cols[p]]
        C[rows[lo]] += wksp
    return C


def spgemm_coo_f32(a_row_idx, a_col_idx, a_vals, b_row_idx, b_col_idx, b_vals):
    """C = A @ B, all three as coordinates (spmspm_coo_float_opt, csrc/kernels.h:397-497).
    For each run of equal neighbouring rows of A, in A's order: every entry (i, j, v)
    of the run adds v * B[j, k] to sums[k] for the entries of B whose row is j, in
    B's storage order; the columns touched (cancelled sums included) are emitted in
    ascending order.  Returns (row, col, val).  Small inputs only (Python loops)."""
    a_rows, a_cols, a_vals = _c(a_row_idx, np.int32), _c(a_col_idx, np.int32), _c(a_vals, np.float32)
    b_rows, b_cols, b_vals = _c(b_row_idx, np.int32), _c(b_col_idx, np.int32), _c(b_vals, np.float32)
    by_row = {}
    for p in range(b_rows.size):  # B's entries of each row, in storage order
        by_row.setdefault(int(b_rows[p]), []).append(p)
    out_r, out_c, out_v = [], [], []
    for lo, hi in _runs(a_rows):
        sums = {}
        for p in range(lo, hi):
            v = a_vals[p]
            for q in by_row.get(int(a_cols[p]), ()):
                k = int(b_cols[q])
                sums[k] = np.float32(sums.get(k, np.float32(0)) + v * b_vals[q])
        for k in sorted(sums):
            out_r.append(int(a_rows[lo]))
            out_c.append(k)
            out_v.append(sums[k])
    return (np.asarray(out_r, dtype=np.int32), np.asarray(out_c, dtype=np.int32),
            np.asarray(out_v, dtype=np.float32))


def spgemm_fp64(a_row_ptr, a_col_idx, a_vals, b_row_ptr, b_col_idx, b_vals, shape_a, n_cols):
    """(A @ B) as a dense float64 array (small cases) via scipy."""
    A = _scipy_csr(a_row_ptr, a_col_idx, a_vals, shape_a)
    B = _scipy_csr(b_row_ptr, b_col_idx, b_vals, (shape_a[1], n_cols))
    return np.asarray((A @ B).todense())


def softmax_csr_f32(row_ptr, vals, scale: float = 1.0) -> np.ndarray:
    """Row softmax over stored values (bench/bench_sparse_transformer.py:277-297)."""
    row_ptr, vals = _c(row_ptr, np.int32), _c(vals, np.float32)
    out = np.zeros_like(vals)
    lib().oracle_softmax_csr_f32(ctypes.c_int(row_ptr.size - 1), _ptr(row_ptr), _ptr(vals),
                                 ctypes.c_float(scale), _ptr(out))
    return out


# --------------------------------------------------------------------------
# float64 recomputation (what the mathematics fixes)
# --------------------------------------------------------------------------
def _scipy_csr(row_ptr, col_idx, vals, shape):
    import scipy.sparse as sp
    return sp.csr_matrix((np.asarray(vals, np.float64), np.asarray(col_idx), np.asarray(row_ptr)),
                         shape=shape)


def spmm_fp64(row_ptr, col_idx, vals, B) -> np.ndarray:
    B64 = np.asarray(B, np.float64)
    A = _scipy_csr(row_ptr, col_idx, vals, (len(row_ptr) - 1, B64.shape[0]))
    return np.asarray(A @ B64)


def sddmm_fp64(row_idx, col_idx, svals, A, B, chunk: int = 1 << 20) -> np.ndarray:
    A64, B64 = np.asarray(A, np.float64), np.asarray(B, np.float64)
    s64 = np.asarray(svals, np.float64)
    out = np.empty(s64.size, np.float64)
    for p0 in range(0, s64.size, chunk):
        p1 = min(s64.size, p0 + chunk)
        out[p0:p1] = np.einsum("pk,pk->p", A64[row_idx[p0:p1]], B64[col_idx[p0:p1]]) * s64[p0:p1]
    return out


def rows_of(row_ptr) -> np.ndarray:
    row_ptr = np.asarray(row_ptr)
    return np.repeat(np.arange(row_ptr.size - 1, dtype=np.int32), np.diff(row_ptr))


def softmax_csr_fp64(row_ptr, vals, scale: float = 1.0) -> np.ndarray:
    row_ptr = np.asarray(row_ptr)
    v = np.asarray(vals, np.float64) * float(scale)
    out = np.zeros_like(v)
    rows = rows_of(row_ptr)
    if v.size == 0:
        return out
    mx = np.full(row_ptr.size - 1, -np.inf)
    np.maximum.at(mx, rows, v)
    e = np.exp(v - mx[rows])
    s = np.zeros(row_ptr.size - 1)
    np.add.at(s, rows, e)
    return e / s[rows]


def attention_dense_fp64(q, k, v, mask_bool, scale: float) -> np.ndarray:
    """softmax(q k^T * scale, -inf outside the mask) @ v in float64 for one head:
    the reference's own dense mode (bench/bench_sparse_transformer.py:330-335).
    Rows with no live entry give zeros."""
    q64, k64, v64 = (np.asarray(t, np.float64) for t in (q, k, v))
    s = (q64 @ k64.T) * float(scale)
    s = np.where(mask_bool, s, -np.inf)
    mx = s.max(axis=1, keepdims=True)
    mx = np.where(np.isfinite(mx), mx, 0.0)
    e = np.exp(s - mx)
    den = e.sum(axis=1, keepdims=True)
    p = np.divide(e, den, out=np.zeros_like(e), where=den > 0)
    return p @ v64


def rel_fro(x, ref64) -> float:
    """Relative Frobenius error ||x - ref|| / ||ref|| (0 when both are zero)."""
    x64 = np.asarray(x, np.float64).ravel()
    r64 = np.asarray(ref64, np.float64).ravel()
    den = np.linalg.norm(r64)
    num = np.linalg.norm(x64 - r64)
    return float(num / den) if den > 0 else float(num)


# --------------------------------------------------------------------------
# The reference's own native module, where it was built
# --------------------------------------------------------------------------
_ref_mod = None


def have_ref() -> bool:
    """The compiled reference module is there and this host can run it (it is built for
    x86-64-v4; see host_has_avx512)."""
    return os.path.exists(_REF_PATH) and host_has_avx512()


def ref_module():
    """Import oracle/_ref/scorch_ops.so (the reference's pybind module compiled
    from its own csrc/ops.cpp).  Raises FileNotFoundError when it was not built."""
    global _ref_mod
    if _ref_mod is None:
        if not have_ref():
            raise FileNotFoundError(_REF_PATH)
        import torch  # noqa: F401  (the module links against libtorch)
        spec = importlib.util.spec_from_file_location("scorch_ops", _REF_PATH)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _ref_mod = mod
    return _ref_mod


def _ref_binary(symbol: str, row_ptr, col_idx, vals, B, extra=()):
    import torch
    m = ref_module()
    vals_t = torch.from_numpy(np.ascontiguousarray(vals))
    B = np.ascontiguousarray(B)
    B_t = torch.from_numpy(B)
    M = len(row_ptr) - 1
    if B.ndim == 2:
        result_shape, b_shape, b_idx = [M, B.shape[1]], list(B.shape), [[], []]
    else:
        result_shape, b_shape, b_idx = [M], list(B.shape), [[]]
    a_idx = [[], [torch.from_numpy(_c(row_ptr, np.int32)), torch.from_numpy(_c(col_idx, np.int32))]]
    out = getattr(m, symbol)(result_shape, [M, int(B.shape[0])], a_idx, vals_t, b_shape, b_idx,
                             B_t.reshape(-1), *extra)
    return out.storage.value.numpy().reshape(result_shape).copy()


def ref_spmm(symbol: str, row_ptr, col_idx, vals, B) -> np.ndarray:
    """Call one of the reference's SpMM symbols (e.g. "spmm_csr_float_v2",
    "prebuilt_spmm_csr_f64") on numpy inputs."""
    return _ref_binary(symbol, row_ptr, col_idx, vals, B)


def ref_spmm_bias(row_ptr, col_idx, vals, B, bias, relu: bool) -> np.ndarray:
    import torch
    symbol = "spmm_csr_bias_relu_float" if relu else "spmm_csr_bias_float"
    return _ref_binary(symbol, row_ptr, col_idx, vals, B,
                       extra=(torch.from_numpy(_c(bias, np.float32)),))


def ref_spmv(symbol: str, row_ptr, col_idx, vals, x) -> np.ndarray:
    return _ref_binary(symbol, row_ptr, col_idx, vals, x)


def ref_spgemm(symbol: str, a_row_ptr, a_col_idx, a_vals, b_row_ptr, b_col_idx, b_vals, shape_a, n_cols):
    """Call one of the reference's CSR x CSR symbols (e.g. "prebuilt_spmspm_csr_f32");
    returns (row_ptr, col_idx, vals)."""
    import torch
    m = ref_module()
    M, K = shape_a
    t = lambda a, dt: torch.from_numpy(_c(a, dt))
    a_vals = np.ascontiguousarray(a_vals)
    out = getattr(m, symbol)([M, n_cols], [M, K], [[], [t(a_row_ptr, np.int32), t(a_col_idx, np.int32)]],
                             torch.from_numpy(a_vals), [K, n_cols],
                             [[], [t(b_row_ptr, np.int32), t(b_col_idx, np.int32)]],
                             torch.from_numpy(_c(b_vals, a_vals.dtype)))
    idx = out.storage.index.mode_indices[1]
    return idx[0].numpy().copy(), idx[1].numpy().copy(), out.storage.value.numpy().copy()


def ref_spmm_coo(row_idx, col_idx, vals, B, n_rows: int) -> np.ndarray:
    """Call the reference's spmm_coo_float on numpy inputs."""
    import torch
    m = ref_module()
    B = _c(B, np.float32)
    a_idx = [[torch.from_numpy(_c(row_idx, np.int32))], [torch.from_numpy(_c(col_idx, np.int32))]]
    out = m.spmm_coo_float([n_rows, B.shape[1]], [n_rows, B.shape[0]], a_idx,
                           torch.from_numpy(_c(vals, np.float32)), list(B.shape), [[], []],
                           torch.from_numpy(B).reshape(-1))
    return out.storage.value.numpy().reshape(n_rows, B.shape[1]).copy()


def ref_spgemm_coo(a_row_idx, a_col_idx, a_vals, b_row_idx, b_col_idx, b_vals, shape_a, n_cols):
    """Call the reference's spmspm_coo_float; returns (row, col, val)."""
    import torch
    m = ref_module()
    M, K = shape_a
    t = lambda a, dt: torch.from_numpy(_c(a, dt))
    out = m.spmspm_coo_float([M, n_cols], [M, K], [[t(a_row_idx, np.int32)], [t(a_col_idx, np.int32)]],
                             t(a_vals, np.float32), [K, n_cols],
                             [[t(b_row_idx, np.int32)], [t(b_col_idx, np.int32)]], t(b_vals, np.float32))
    idx = out.storage.index.mode_indices
    return idx[0][0].numpy().copy(), idx[1][0].numpy().copy(), out.storage.value.numpy().copy()


def ref_sddmm_coo(row_idx, col_idx, svals, A, B, shape):
    """Call the reference's sddmm_coo_float_prebuilt; returns (row, col, val)."""
    import torch
    m = ref_module()
    A, B = _c(A, np.float32), _c(B, np.float32)
    s_idx = [[torch.from_numpy(_c(row_idx, np.int32))], [torch.from_numpy(_c(col_idx, np.int32))]]
    out = m.sddmm_coo_float_prebuilt(list(shape), list(shape), s_idx,
                                     torch.from_numpy(_c(svals, np.float32)),
                                     list(A.shape), [[], []], torch.from_numpy(A).reshape(-1),
                                     list(B.shape), [[], []], torch.from_numpy(B).reshape(-1))
    idx = out.storage.index.mode_indices
    return idx[0][0].numpy().copy(), idx[1][0].numpy().copy(), out.storage.value.numpy().copy()


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    print("liboracle.so:", os.path.exists(_LIB_PATH), " _ref/scorch_ops.so:", have_ref(),
          " threads:", num_threads())


def attention_blocksparse_fp64(q, k, v, block_row_ptr, block_col_idx, block: int, scale: float) -> np.ndarray:
    """Block-sparse attention for (H, S, D) inputs in float64: per head, the
    masked dense softmax of attention_dense_fp64 with the mask expanded from its
    block pattern (every entry of an active block live).  Written for small S."""
    q, k, v = (np.asarray(t, np.float64) for t in (q, k, v))
    H, S, _ = q.shape
    nb = S // block
    blocks = np.zeros((nb, nb), dtype=bool)
    rows = rows_of(block_row_ptr)
    blocks[rows, np.asarray(block_col_idx)] = True
    mask = np.kron(blocks, np.ones((block, block), dtype=bool))
    return np.stack([attention_dense_fp64(q[h], k[h], v[h], mask, scale) for h in range(H)])
