"""The C restatement against the reference's native module itself
(oracle/_ref/scorch_ops.so, compiled from the reference's csrc/ops.cpp by
oracle/Makefile) on fresh random inputs.  Skipped where that module was not
built (it needs the reference sources)."""
import numpy as np
import pytest

from conftest import random_csr
from scorch_amd import workloads


@pytest.fixture(scope="module")
def ref(oracle):
    if not oracle.have_ref():
        pytest.skip("oracle/_ref/scorch_ops.so not built")
    try:
        oracle.ref_module()
    except Exception as exc:  # e.g. built for another ISA
        pytest.skip(f"oracle/_ref/scorch_ops.so does not load here: {exc}")
    return oracle


@pytest.mark.parametrize("M,K,N,density,seed", [(200, 150, 33, 0.05, 0), (64, 64, 257, 0.2, 1),
                                                (500, 40, 128, 0.1, 2), (7, 900, 64, 0.3, 3)])
def test_spmm_f32_both_symbols(ref, M, K, N, density, seed):
    rng = np.random.default_rng(seed)
    rp, ci, v = random_csr(rng, M, K, density, empty_rows=(0,))
    B = rng.standard_normal((K, N)).astype(np.float32)
    np.testing.assert_allclose(ref.spmm_csr_f32_v2(rp, ci, v, B),
                               ref.ref_spmm("spmm_csr_float_v2", rp, ci, v, B), rtol=2e-6, atol=1e-6)
    np.testing.assert_allclose(ref.spmm_csr_typed(rp, ci, v, B),
                               ref.ref_spmm("prebuilt_spmm_csr_f32", rp, ci, v, B), rtol=2e-6, atol=1e-6)


def test_spmm_power_law_workload_small(ref):
    w = workloads.gcn_powerlaw(M=3000, N=64, seed=5, max_degree=800)
    got = ref.spmm_csr_f32_v2(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    expect = ref.ref_spmm("spmm_csr_float_v2", w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    np.testing.assert_allclose(got, expect, rtol=2e-6, atol=1e-6)
    assert ref.rel_fro(got, ref.spmm_fp64(w["row_ptr"], w["col_idx"], w["vals"], w["B"])) < 1e-6


@pytest.mark.parametrize("suffix,dtype", [("f64", np.float64), ("i32", np.int32), ("i64", np.int64)])
def test_spmm_other_dtypes(ref, suffix, dtype):
    rng = np.random.default_rng(20)
    rp, ci, v = random_csr(rng, 90, 70, 0.1, dtype=dtype)
    B = (rng.integers(-1000, 1000, size=(70, 19)) if np.issubdtype(dtype, np.integer)
         else rng.standard_normal((70, 19))).astype(dtype)
    got = ref.spmm_csr_typed(rp, ci, v, B)
    expect = ref.ref_spmm("prebuilt_spmm_csr_" + suffix, rp, ci, v, B)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got, expect)
    else:
        np.testing.assert_allclose(got, expect, rtol=1e-14)


@pytest.mark.parametrize("relu", [False, True])
def test_bias_act(ref, relu):
    rng = np.random.default_rng(21)
    rp, ci, v = random_csr(rng, 120, 80, 0.08, empty_rows=(3, 4))
    B = rng.standard_normal((80, 40)).astype(np.float32)
    bias = rng.standard_normal(40).astype(np.float32)
    np.testing.assert_allclose(ref.spmm_csr_bias_act_f32(rp, ci, v, B, bias, relu),
                               ref.ref_spmm_bias(rp, ci, v, B, bias, relu), rtol=2e-6, atol=1e-6)


@pytest.mark.parametrize("M,ncols,K,seed", [(100, 80, 64, 0), (33, 200, 7, 1), (300, 300, 128, 2)])
def test_sddmm_coo(ref, M, ncols, K, seed):
    rng = np.random.default_rng(seed)
    rp, ci, s = random_csr(rng, M, ncols, 0.1)
    rows = ref.rows_of(rp)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((ncols, K)).astype(np.float32)
    r_out, c_out, val = ref.ref_sddmm_coo(rows, ci, s, A, B, (M, ncols))
    np.testing.assert_allclose(ref.sddmm_coo_f32(rows, ci, s, A, B), val, rtol=1e-5, atol=1e-6)
    assert np.array_equal(r_out, rows) and np.array_equal(c_out, ci)


@pytest.mark.parametrize("suffix,dtype", [("f32", np.float32), ("f64", np.float64), ("i32", np.int32),
                                          ("i64", np.int64)])
def test_spmv(ref, suffix, dtype):
    rng = np.random.default_rng(30)
    rp, ci, v = random_csr(rng, 150, 110, 0.1, dtype=dtype, empty_rows=(149,))
    x = (rng.integers(-1000, 1000, size=110) if np.issubdtype(dtype, np.integer)
         else rng.standard_normal(110)).astype(dtype)
    got = ref.spmv_csr_typed(rp, ci, v, x)
    expect = ref.ref_spmv("prebuilt_spmv_csr_" + suffix, rp, ci, v, x)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got, expect)
    else:
        np.testing.assert_allclose(got, expect, rtol=1e-5 if dtype == np.float32 else 1e-13, atol=1e-6)


@pytest.mark.parametrize("suffix,dtype", [("f32", np.float32), ("f64", np.float64), ("i32", np.int32),
                                          ("i64", np.int64)])
def test_spgemm(ref, suffix, dtype):
    rng = np.random.default_rng(40)
    arp, aci, av = random_csr(rng, 130, 90, 0.08, dtype=dtype, empty_rows=(0, 129))
    brp, bci, bv = random_csr(rng, 90, 150, 0.1, dtype=dtype, empty_rows=(4,))
    got = ref.spgemm_csr_typed(arp, aci, av, brp, bci, bv, 150)
    want = ref.ref_spgemm("prebuilt_spmspm_csr_" + suffix, arp, aci, av, brp, bci, bv, (130, 90), 150)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got[2], want[2])
    else:
        np.testing.assert_allclose(got[2], want[2], rtol=1e-6 if dtype == np.float32 else 1e-14)


def _coo(rp, ci):
    return np.repeat(np.arange(rp.size - 1, dtype=np.int32), np.diff(rp)), ci


@pytest.mark.parametrize("seed,N", [(30, 17), (31, 64)])
def test_spmm_coo(ref, seed, N):
    rng = np.random.default_rng(seed)
    rp, ci, v = random_csr(rng, 80, 60, 0.1, empty_rows=(0, 41))
    r, c = _coo(rp, ci)
    B = rng.standard_normal((60, N)).astype(np.float32)
    np.testing.assert_allclose(ref.spmm_coo_f32(r, c, v, B, 80), ref.ref_spmm_coo(r, c, v, B, 80),
                               rtol=2e-6, atol=1e-6)
    runs = np.concatenate([np.flatnonzero(r >= 50), np.flatnonzero(r < 50), np.flatnonzero(r == 7)])
    np.testing.assert_allclose(ref.spmm_coo_f32(r[runs], c[runs], v[runs], B, 80),
                               ref.ref_spmm_coo(r[runs], c[runs], v[runs], B, 80), rtol=2e-6, atol=1e-5)


@pytest.mark.parametrize("seed", [32, 33])
def test_spgemm_coo(ref, seed):
    # B no wider than tall: the reference sizes this kernel's per-column arrays by B's row count
    rng = np.random.default_rng(seed)
    arp, aci, av = random_csr(rng, 50, 40, 0.1, empty_rows=(3,))
    brp, bci, bv = random_csr(rng, 40, 38, 0.12, empty_rows=(0, 20))
    ar, ac = _coo(arp, aci)
    br, bc = _coo(brp, bci)
    shuffle = rng.permutation(br.size)
    br, bc, bv = br[shuffle], bc[shuffle], bv[shuffle]
    r, k, v = ref.spgemm_coo_f32(ar, ac, av, br, bc, bv)
    wr, wk, wv = ref.ref_spgemm_coo(ar, ac, av, br, bc, bv, (50, 40), 38)
    assert np.array_equal(r, wr) and np.array_equal(k, wk)
    np.testing.assert_allclose(v, wv, rtol=2e-6, atol=1e-6)
