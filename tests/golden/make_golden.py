"""Writes tests/golden/golden_ref.npz: inputs and outputs of the reference's
own native kernels on small cases.

Run once, in a container that holds the reference sources, after
``make -C oracle ref`` has compiled the reference's csrc/ops.cpp into
oracle/_ref/scorch_ops.so.  The outputs stored here come from that module
(symbols spmm_csr_float_v2, prebuilt_spmm_csr_{f32,f64,i32,i64},
spmm_csr_bias[_relu]_float, prebuilt_spmspm_csr_{f32,f64,i32,i64}, sddmm_coo_float_prebuilt,
prebuilt_spmv_csr_{f32,f64,i32,i64}, spmm_coo_float, spmspm_coo_float); the inputs come from this script's own
seeded numpy generators.  The file holds data only.

The cases re-express, with numpy's generator instead of torch's, the seeded and
literal cases of the reference's tests for this path:
tests/test_scorch/test_perf_large.py:15-23,52-73 (square, 95 % sparse),
test_matmul_dispatch.py:9-27 (n=32, 10 % dense), test_kernels.py:1310-1358
(literal diag(1..5)), test_kernels_comprehensive.py:260-271 (30x50 . 50x20),
:376-411 (SDDMM n/d/sparsity grid), test_compile.py:70-127 (n=64, k=16 fused
bias/ReLU), test_prebuilt_kernel_registry.py:21-38 (literal 4x4 int64 SpMV),
test_matmul_dispatch.py:30-48 (CSR x CSR),
plus the edge cases the kernels must survive (empty rows, no entries at all,
more than one 256-wide column tile, a row far longer than the rest).

    python tests/golden/make_golden.py
"""
from __future__ import annotations

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden_ref.npz")


def random_csr(rng, M, K, density, dtype=np.float32, lo=0.0, hi=1.0, empty_rows=()):
    keep = rng.random((M, K)) < density
    for r in empty_rows:
        keep[r, :] = False
    rows, cols = np.nonzero(keep)
    row_ptr = np.zeros(M + 1, dtype=np.int32)
    np.cumsum(np.bincount(rows, minlength=M), out=row_ptr[1:])
    if np.issubdtype(dtype, np.integer):
        vals = rng.integers(-50, 50, size=rows.size).astype(dtype)
    else:
        vals = rng.uniform(lo, hi, size=rows.size).astype(dtype)
    return row_ptr, cols.astype(np.int32), vals


def dense(rng, shape, dtype=np.float32):
    if np.issubdtype(dtype, np.integer):
        return rng.integers(-50, 50, size=shape).astype(dtype)
    return rng.random(shape).astype(dtype)


def main() -> None:
    if not O.have_ref():
        raise SystemExit("oracle/_ref/scorch_ops.so is missing: run `make -C oracle ref` first")
    data = {}

    def put(case, **arrays):
        for k, v in arrays.items():
            data[f"{case}/{k}"] = np.asarray(v)

    # ---- SpMM fp32: v2 (the dispatched symbol) and the typed kernel ----------
    spmm_cases = {
        "spmm_square95": dict(M=256, K=256, N=48, density=0.05, seed=7),
        "spmm_dispatch32": dict(M=32, K=32, N=32, density=0.10, seed=0),
        "spmm_rect": dict(M=30, K=50, N=20, density=0.20, seed=500),
        "spmm_wide300": dict(M=24, K=40, N=300, density=0.25, seed=11),
        "spmm_emptyrows": dict(M=40, K=33, N=17, density=0.15, seed=21, empty_rows=(0, 5, 6, 39)),
        "spmm_n1": dict(M=19, K=23, N=1, density=0.3, seed=22),
    }
    for name, c in spmm_cases.items():
        rng = np.random.default_rng(c["seed"])
        rp, ci, v = random_csr(rng, c["M"], c["K"], c["density"], empty_rows=c.get("empty_rows", ()))
        B = dense(rng, (c["K"], c["N"]))
        put(name, row_ptr=rp, col_idx=ci, vals=v, B=B,
            C_v2=O.ref_spmm("spmm_csr_float_v2", rp, ci, v, B),
            C_typed=O.ref_spmm("prebuilt_spmm_csr_f32", rp, ci, v, B))

    # one very long row among short ones (power-law shape in miniature)
    rng = np.random.default_rng(31)
    M, K, N = 64, 1024, 16
    rp, ci, v = random_csr(rng, M, K, 0.008)
    keep = rng.random(K) < 0.9
    long_cols = np.nonzero(keep)[0].astype(np.int32)
    r = 17
    ci = np.concatenate([ci[:rp[r]], long_cols, ci[rp[r + 1]:]])
    v = np.concatenate([v[:rp[r]], rng.uniform(-1, 1, long_cols.size).astype(np.float32), v[rp[r + 1]:]])
    lens = np.diff(rp)
    lens[r] = long_cols.size
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    B = dense(rng, (K, N))
    put("spmm_longrow", row_ptr=rp, col_idx=ci, vals=v, B=B,
        C_v2=O.ref_spmm("spmm_csr_float_v2", rp, ci, v, B),
        C_typed=O.ref_spmm("prebuilt_spmm_csr_f32", rp, ci, v, B))

    # no stored entries at all
    rp = np.zeros(11, dtype=np.int32)
    ci = np.zeros(0, dtype=np.int32)
    v = np.zeros(0, dtype=np.float32)
    B = dense(np.random.default_rng(1100), (10, 6))
    put("spmm_allzero", row_ptr=rp, col_idx=ci, vals=v, B=B,
        C_v2=O.ref_spmm("spmm_csr_float_v2", rp, ci, v, B),
        C_typed=O.ref_spmm("prebuilt_spmm_csr_f32", rp, ci, v, B))

    # literal diag(1..5) times a literal B
    rp = np.arange(6, dtype=np.int32)
    ci = np.arange(5, dtype=np.int32)
    v = np.arange(1, 6, dtype=np.float32)
    B = np.array([[1, 2, 3, 4, 5], [2, 2, 0, 0, 0], [3, 0, 3, 0, 0], [4, 0, 0, 4, 0], [5, 0, 0, 0, 5]],
                 dtype=np.float32)
    put("spmm_diag_literal", row_ptr=rp, col_idx=ci, vals=v, B=B,
        C_v2=O.ref_spmm("spmm_csr_float_v2", rp, ci, v, B),
        C_typed=O.ref_spmm("prebuilt_spmm_csr_f32", rp, ci, v, B))

    # ---- SpMM, the other three dtypes ----------------------------------------
    for suffix, dt in (("f64", np.float64), ("i32", np.int32), ("i64", np.int64)):
        rng = np.random.default_rng(100 + len(suffix) + ord(suffix[0]))
        rp, ci, v = random_csr(rng, 16, 16, 0.2, dtype=dt)
        B = dense(rng, (16, 16), dtype=dt)
        put(f"spmm_{suffix}", row_ptr=rp, col_idx=ci, vals=v, B=B,
            C_typed=O.ref_spmm(f"prebuilt_spmm_csr_{suffix}", rp, ci, v, B))
    # integer wrap-around: products overflow int32 and must wrap, not saturate
    rng = np.random.default_rng(77)
    rp, ci, _ = random_csr(rng, 12, 12, 0.4, dtype=np.int32)
    v = rng.integers(-2 ** 30, 2 ** 30, size=ci.size).astype(np.int32)
    B = rng.integers(-2 ** 30, 2 ** 30, size=(12, 9)).astype(np.int32)
    put("spmm_i32_wrap", row_ptr=rp, col_idx=ci, vals=v, B=B,
        C_typed=O.ref_spmm("prebuilt_spmm_csr_i32", rp, ci, v, B))

    # ---- fused bias / bias + ReLU ---------------------------------------------
    rng = np.random.default_rng(42)
    rp, ci, v = random_csr(rng, 64, 64, 0.1, lo=-1.0, hi=1.0)
    B = rng.standard_normal((64, 16)).astype(np.float32)
    bias = rng.standard_normal(16).astype(np.float32)
    put("spmm_bias", row_ptr=rp, col_idx=ci, vals=v, B=B, bias=bias,
        C_bias=O.ref_spmm_bias(rp, ci, v, B, bias, relu=False),
        C_bias_relu=O.ref_spmm_bias(rp, ci, v, B, bias, relu=True))

    # ---- SDDMM (coordinate mask) ------------------------------------------------
    for n, d, sparsity in ((16, 8, 0.5), (64, 32, 0.9), (128, 16, 0.95), (256, 64, 0.99), (40, 16, 0.9)):
        rng = np.random.default_rng(n + d)
        rp, ci, v = random_csr(rng, n, n, 1.0 - sparsity)
        rows = O.rows_of(rp)
        Q, Kt = dense(rng, (n, d)), dense(rng, (n, d))
        r_out, c_out, val = O.ref_sddmm_coo(rows, ci, v, Q, Kt, (n, n))
        put(f"sddmm_{n}_{d}", row_ptr=rp, row_idx=rows, col_idx=ci, vals=v, A=Q, B=Kt,
            out_row=r_out, out_col=c_out, out_val=val)
    # rectangular mask, K not a multiple of 4, explicit zero in the mask
    rng = np.random.default_rng(808)
    rp, ci, v = random_csr(rng, 37, 53, 0.15, lo=-1.0, hi=1.0)
    v[::7] = 0.0
    rows = O.rows_of(rp)
    Q, Kt = dense(rng, (37, 13)), dense(rng, (53, 13))
    r_out, c_out, val = O.ref_sddmm_coo(rows, ci, v, Q, Kt, (37, 53))
    put("sddmm_rect_k13", row_ptr=rp, row_idx=rows, col_idx=ci, vals=v, A=Q, B=Kt,
        out_row=r_out, out_col=c_out, out_val=val)

    # ---- SpMV -------------------------------------------------------------------
    A = np.array([[1, 0, 2, 0], [0, 3, 0, 4], [0, 0, 0, 0], [5, 0, 0, 6]], dtype=np.int64)
    rows, cols = np.nonzero(A)
    rp = np.concatenate([[0], np.cumsum(np.bincount(rows, minlength=4))]).astype(np.int32)
    x = np.array([1, 2, 3, 4], dtype=np.int64)
    put("spmv_i64_literal", row_ptr=rp, col_idx=cols.astype(np.int32), vals=A[rows, cols], x=x,
        y=O.ref_spmv("prebuilt_spmv_csr_i64", rp, cols.astype(np.int32), A[rows, cols], x))
    for suffix, dt in (("f32", np.float32), ("f64", np.float64), ("i32", np.int32)):
        rng = np.random.default_rng(900 + ord(suffix[1]))
        rp, ci, v = random_csr(rng, 50, 70, 0.2, dtype=dt, empty_rows=(3, 49))
        x = dense(rng, (70,), dtype=dt)
        put(f"spmv_{suffix}", row_ptr=rp, col_idx=ci, vals=v, x=x,
            y=O.ref_spmv(f"prebuilt_spmv_csr_{suffix}", rp, ci, v, x))

    # ---- SpGEMM (CSR x CSR -> CSR) --------------------------------------------------
    for suffix, dt in (("f32", np.float32), ("f64", np.float64), ("i32", np.int32), ("i64", np.int64)):
        rng = np.random.default_rng(1200 + ord(suffix[0]) + int(suffix[1:]))
        arp, aci, av = random_csr(rng, 48, 40, 0.12, dtype=dt, empty_rows=(5,))
        brp, bci, bv = random_csr(rng, 40, 56, 0.15, dtype=dt, empty_rows=(0, 17))
        crp, cci, cv = O.ref_spgemm(f"prebuilt_spmspm_csr_{suffix}", arp, aci, av, brp, bci, bv, (48, 40), 56)
        put(f"spgemm_{suffix}", a_row_ptr=arp, a_col_idx=aci, a_vals=av, b_row_ptr=brp, b_col_idx=bci,
            b_vals=bv, n_cols=np.int64(56), c_row_ptr=crp, c_col_idx=cci, c_vals=cv)
    # exact cancellation: the entry is stored although its value is zero
    arp = np.array([0, 2, 3], np.int32); aci = np.array([0, 1, 1], np.int32)
    av = np.array([1.0, -1.0, 2.0], np.float32)
    brp = np.array([0, 2, 4], np.int32); bci = np.array([0, 2, 0, 1], np.int32)
    bv = np.array([3.0, 5.0, 3.0, 7.0], np.float32)
    crp, cci, cv = O.ref_spgemm("spmspm_csr_float", arp, aci, av, brp, bci, bv, (2, 2), 3)
    put("spgemm_cancel", a_row_ptr=arp, a_col_idx=aci, a_vals=av, b_row_ptr=brp, b_col_idx=bci, b_vals=bv,
        n_cols=np.int64(3), c_row_ptr=crp, c_col_idx=cci, c_vals=cv)

    # ---- coordinate-form operands: spmm_coo_float, spmspm_coo_float ------------
    def coo_of(rp, ci):
        return np.repeat(np.arange(rp.size - 1, dtype=np.int32), np.diff(rp)), ci

    rng = np.random.default_rng(41)
    rp, ci, v = random_csr(rng, 37, 29, 0.15, empty_rows=(0, 11))
    r, c = coo_of(rp, ci)
    B = dense(rng, (29, 21))
    put("spmm_coo", row_idx=r, col_idx=c, vals=v, B=B, n_rows=np.int64(37), C=O.ref_spmm_coo(r, c, v, B, 37))
    # the same entries with runs of rows out of order and some coordinates repeated
    order = np.concatenate([np.flatnonzero(r >= 20), np.flatnonzero(r < 20), np.flatnonzero(r == 3)])
    r2, c2, v2 = r[order], c[order], v[order]
    put("spmm_coo_unsorted", row_idx=r2, col_idx=c2, vals=v2, B=B, n_rows=np.int64(37),
        C=O.ref_spmm_coo(r2, c2, v2, B, 37))

    rng = np.random.default_rng(42)
    arp, aci, av = random_csr(rng, 33, 27, 0.12, empty_rows=(4,))
    # (the reference sizes this kernel's per-column workspace by B's row count, so B must not be wider than tall)
    brp, bci, bv = random_csr(rng, 27, 25, 0.15, empty_rows=(0, 9))
    ar, ac = coo_of(arp, aci)
    br, bc = coo_of(brp, bci)
    shuffle = rng.permutation(br.size)  # the reference scans all of B for every entry of A: any order
    br, bc, bv = br[shuffle], bc[shuffle], bv[shuffle]
    cr, cc, cv = O.ref_spgemm_coo(ar, ac, av, br, bc, bv, (33, 27), 25)
    put("spgemm_coo", a_row_idx=ar, a_col_idx=ac, a_vals=av, b_row_idx=br, b_col_idx=bc, b_vals=bv,
        shape=np.array([33, 27, 25], np.int64), c_row_idx=cr, c_col_idx=cc, c_vals=cv)
    # cancellation (the entry stays) and a coordinate of B stored twice (the two add up)
    ar = np.array([0, 0, 1], np.int32); ac = np.array([0, 1, 1], np.int32)
    av = np.array([1.0, -1.0, 2.0], np.float32)
    br = np.array([0, 0, 1, 1, 1], np.int32); bc = np.array([0, 2, 0, 1, 1], np.int32)
    bv = np.array([3.0, 5.0, 3.0, 7.0, 0.5], np.float32)
    cr, cc, cv = O.ref_spgemm_coo(ar, ac, av, br, bc, bv, (2, 3), 3)
    put("spgemm_coo_cancel", a_row_idx=ar, a_col_idx=ac, a_vals=av, b_row_idx=br, b_col_idx=bc, b_vals=bv,
        shape=np.array([2, 3, 3], np.int64), c_row_idx=cr, c_col_idx=cc, c_vals=cv)

    np.savez_compressed(OUT, **data)
    print(f"wrote {OUT}: {len(data)} arrays, {os.path.getsize(OUT) / 1024:.1f} KiB")


if __name__ == "__main__":
    main()
