"""Pins the oracle to what the mathematics fixes, independently of the
reference's outputs: closed forms, special cases that reduce to a library
routine, and brute force on tiny inputs.  Each check is chosen so that a
plausible mistake (a transposed operand, a dropped term, a wrong index) fails.
"""
import numpy as np
import pytest
import scipy.sparse as sp
import scipy.special

from conftest import random_csr


def brute_spmm(row_ptr, col_idx, vals, B):
    M, N = len(row_ptr) - 1, B.shape[1]
    C = np.zeros((M, N), dtype=np.float64)
    for i in range(M):
        for p in range(row_ptr[i], row_ptr[i + 1]):
            for k in range(N):
                C[i, k] += float(vals[p]) * float(B[col_idx[p], k])
    return C


def spmm_variants(oracle):
    return [("v2", oracle.spmm_csr_f32_v2), ("typed", oracle.spmm_csr_typed)]


@pytest.mark.parametrize("which", ["v2", "typed"])
def test_spmm_identity_returns_B(oracle, which):
    fn = dict(spmm_variants(oracle))[which]
    rng = np.random.default_rng(1)
    B = rng.standard_normal((37, 21)).astype(np.float32)
    rp = np.arange(38, dtype=np.int32)
    out = fn(rp, np.arange(37, dtype=np.int32), np.ones(37, np.float32), B)
    assert np.array_equal(out, B)


@pytest.mark.parametrize("which", ["v2", "typed"])
def test_spmm_one_entry_per_row_is_a_row_gather(oracle, which):
    fn = dict(spmm_variants(oracle))[which]
    rng = np.random.default_rng(2)
    B = rng.standard_normal((50, 300)).astype(np.float32)   # 300 > one 256-wide tile
    perm = rng.integers(0, 50, size=64).astype(np.int32)
    out = fn(np.arange(65, dtype=np.int32), perm, np.ones(64, np.float32), B)
    assert np.array_equal(out, B[perm])


@pytest.mark.parametrize("which", ["v2", "typed"])
def test_spmm_rectangular_brute_force(oracle, which):
    # M != K != N so that any transposition of an operand or index breaks it
    fn = dict(spmm_variants(oracle))[which]
    rng = np.random.default_rng(3)
    rp, ci, v = random_csr(rng, 13, 29, 0.3, empty_rows=(4,))
    B = rng.standard_normal((29, 7)).astype(np.float32)
    np.testing.assert_allclose(fn(rp, ci, v, B), brute_spmm(rp, ci, v, B), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("which", ["v2", "typed"])
def test_spmm_matches_scipy_fp64(oracle, which):
    fn = dict(spmm_variants(oracle))[which]
    rng = np.random.default_rng(4)
    rp, ci, v = random_csr(rng, 300, 200, 0.05)
    B = rng.standard_normal((200, 130)).astype(np.float32)
    ref = sp.csr_matrix((v.astype(np.float64), ci, rp), shape=(300, 200)) @ B.astype(np.float64)
    assert oracle.rel_fro(fn(rp, ci, v, B), ref) < 1e-6
    assert oracle.rel_fro(oracle.spmm_fp64(rp, ci, v, B), ref) < 1e-15


def test_spmm_duplicate_columns_accumulate(oracle):
    rp = np.array([0, 3], dtype=np.int32)
    ci = np.array([1, 1, 0], dtype=np.int32)
    v = np.array([2.0, 3.0, 1.0], dtype=np.float32)
    B = np.array([[1.0, 10.0], [100.0, 1000.0]], dtype=np.float32)
    assert oracle.spmm_csr_f32_v2(rp, ci, v, B).tolist() == [[501.0, 5010.0]]


def test_spmm_regular_graph_preserves_constant_features(oracle):
    # ring with self-loops: every node has degree 3, so D^-1/2 (A+I) D^-1/2 has
    # rows summing to one and a constant feature column is a fixed point
    n = 40
    cols = np.stack([(np.arange(n) - 1) % n, np.arange(n), (np.arange(n) + 1) % n], axis=1)
    cols.sort(axis=1)
    rp = (np.arange(n + 1) * 3).astype(np.int32)
    v = np.full(3 * n, 1.0 / 3.0, dtype=np.float32)
    X = np.tile(np.array([[2.0, -5.0, 0.25]], dtype=np.float32), (n, 1))
    out = oracle.spmm_csr_f32_v2(rp, cols.reshape(-1).astype(np.int32), v, X)
    np.testing.assert_allclose(out, X, rtol=1e-6)


def test_spmm_empty_rows_and_empty_matrix_give_zeros(oracle):
    rng = np.random.default_rng(5)
    B = rng.standard_normal((6, 5)).astype(np.float32)
    rp = np.array([0, 0, 2, 2, 2], dtype=np.int32)
    out = oracle.spmm_csr_f32_v2(rp, np.array([1, 4], np.int32), np.array([1.0, 1.0], np.float32), B)
    assert not out[[0, 2, 3]].any() and np.array_equal(out[1], B[1] + B[4])
    zero = oracle.spmm_csr_typed(np.zeros(4, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), B)
    assert zero.shape == (3, 5) and not zero.any()


@pytest.mark.parametrize("dtype", [np.int32, np.int64])
def test_spmm_integer_matches_numpy_matmul(oracle, dtype):
    rng = np.random.default_rng(6)
    rp, ci, v = random_csr(rng, 20, 17, 0.3, dtype=dtype)
    B = rng.integers(-1000, 1000, size=(17, 9)).astype(dtype)
    dense = np.zeros((20, 17), dtype=dtype)
    dense[np.repeat(np.arange(20), np.diff(rp)), ci] = v
    assert np.array_equal(oracle.spmm_csr_typed(rp, ci, v, B), dense @ B)


@pytest.mark.parametrize("relu", [False, True])
def test_bias_act_is_act_of_product_plus_bias(oracle, relu):
    rng = np.random.default_rng(7)
    rp, ci, v = random_csr(rng, 31, 23, 0.2, empty_rows=(0, 30))
    B = rng.standard_normal((23, 11)).astype(np.float32)
    bias = rng.standard_normal(11).astype(np.float32)
    ref = oracle.spmm_fp64(rp, ci, v, B) + bias.astype(np.float64)
    if relu:
        ref = np.maximum(ref, 0.0)
    out = oracle.spmm_csr_bias_act_f32(rp, ci, v, B, bias, relu)
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-6)
    # empty rows are act(bias), not zero
    np.testing.assert_allclose(out[0], np.maximum(bias, 0) if relu else bias)


# ---- SDDMM -----------------------------------------------------------------------
def test_sddmm_uses_B_indexed_by_column_then_k(oracle):
    # rectangular mask and K so that reading B as [k, j] would index out of the intended values
    rng = np.random.default_rng(8)
    rp, ci, s = random_csr(rng, 9, 14, 0.4)
    rows = oracle.rows_of(rp)
    A = rng.standard_normal((9, 5)).astype(np.float32)
    B = rng.standard_normal((14, 5)).astype(np.float32)
    expect = (A.astype(np.float64) @ B.astype(np.float64).T)[rows, ci] * s
    np.testing.assert_allclose(oracle.sddmm_coo_f32(rows, ci, s, A, B), expect, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(oracle.sddmm_csr_f32(rp, ci, s, A, B)[2], expect, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(oracle.sddmm_fp64(rows, ci, s, A, B), expect, rtol=1e-12)


def test_sddmm_one_hot_operands_give_kronecker_delta(oracle):
    n, K = 12, 12
    A = np.eye(n, K, dtype=np.float32)
    B = np.eye(n, K, dtype=np.float32)
    rows, cols = np.nonzero(np.ones((n, n)))
    out = oracle.sddmm_coo_f32(rows.astype(np.int32), cols.astype(np.int32), np.ones(n * n, np.float32), A, B)
    assert np.array_equal(out.reshape(n, n), np.eye(n, dtype=np.float32))


def test_sddmm_k1_is_outer_product_sample_and_scales_with_mask(oracle):
    rng = np.random.default_rng(9)
    rp, ci, s = random_csr(rng, 15, 11, 0.5)
    rows = oracle.rows_of(rp)
    a = rng.standard_normal((15, 1)).astype(np.float32)
    b = rng.standard_normal((11, 1)).astype(np.float32)
    ones = oracle.sddmm_coo_f32(rows, ci, np.ones_like(s), a, b)
    np.testing.assert_allclose(ones, a[rows, 0] * b[ci, 0], rtol=1e-6)
    np.testing.assert_allclose(oracle.sddmm_coo_f32(rows, ci, s, a, b), s * ones, rtol=1e-6)


def test_sddmm_coo_accepts_any_entry_order(oracle):
    rng = np.random.default_rng(10)
    rp, ci, s = random_csr(rng, 20, 20, 0.3)
    rows = oracle.rows_of(rp)
    A = rng.standard_normal((20, 8)).astype(np.float32)
    B = rng.standard_normal((20, 8)).astype(np.float32)
    base = oracle.sddmm_coo_f32(rows, ci, s, A, B)
    perm = rng.permutation(s.size)
    shuffled = oracle.sddmm_coo_f32(rows[perm], ci[perm], s[perm], A, B)
    np.testing.assert_allclose(shuffled, base[perm], rtol=1e-6)


# ---- SpMV / softmax -----------------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
def test_spmv_matches_dense_product(oracle, dtype):
    rng = np.random.default_rng(11)
    rp, ci, v = random_csr(rng, 33, 27, 0.25, dtype=dtype, empty_rows=(5,))
    x = (rng.integers(-50, 50, size=27) if np.issubdtype(dtype, np.integer)
         else rng.standard_normal(27)).astype(dtype)
    dense = np.zeros((33, 27), dtype=np.float64 if not np.issubdtype(dtype, np.integer) else dtype)
    dense[np.repeat(np.arange(33), np.diff(rp)), ci] = v
    got = oracle.spmv_csr_typed(rp, ci, v, x)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got, dense @ x)
    else:
        np.testing.assert_allclose(got, dense @ x.astype(np.float64), rtol=1e-5, atol=1e-6)


def test_softmax_rows_match_scipy_and_sum_to_one(oracle):
    rng = np.random.default_rng(12)
    rp, _, v = random_csr(rng, 25, 40, 0.3, empty_rows=(3,), lo=-4.0, hi=4.0)
    out = oracle.softmax_csr_f32(rp, v, scale=0.5)
    out64 = oracle.softmax_csr_fp64(rp, v, scale=0.5)
    for i in range(25):
        seg = slice(rp[i], rp[i + 1])
        if rp[i] == rp[i + 1]:
            continue
        expect = scipy.special.softmax(v[seg].astype(np.float64) * 0.5)
        np.testing.assert_allclose(out[seg], expect, rtol=1e-5)
        np.testing.assert_allclose(out64[seg], expect, rtol=1e-12)
        assert abs(out[seg].sum() - 1.0) < 1e-5


def test_softmax_is_shift_invariant_and_survives_large_values(oracle):
    rp = np.array([0, 4], dtype=np.int32)
    v = np.array([1000.0, 1001.0, 999.0, 1000.5], dtype=np.float32)
    out = oracle.softmax_csr_f32(rp, v)
    assert np.isfinite(out).all()
    np.testing.assert_allclose(out, oracle.softmax_csr_f32(rp, v - 1000.0), rtol=1e-5)


def test_attention_dense_fp64_matches_csr_pipeline(oracle):
    # SDDMM -> row softmax -> SpMM over a CSR mask equals masked dense attention
    rng = np.random.default_rng(13)
    S, D = 24, 8
    rp, ci, _ = random_csr(rng, S, S, 0.4)
    rows = oracle.rows_of(rp)
    q, k, v = (rng.standard_normal((S, D)).astype(np.float32) for _ in range(3))
    scores = oracle.sddmm_fp64(rows, ci, np.ones(ci.size), q, k)
    probs = oracle.softmax_csr_fp64(rp, scores, scale=D ** -0.5)
    out = oracle.spmm_fp64(rp, ci, probs, v)
    mask = np.zeros((S, S), dtype=bool)
    mask[rows, ci] = True
    np.testing.assert_allclose(out, oracle.attention_dense_fp64(q, k, v, mask, D ** -0.5), rtol=1e-10,
                               atol=1e-12)


# ---- SpGEMM ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
def test_spgemm_matches_scipy_structure_and_values(oracle, dtype):
    rng = np.random.default_rng(14)
    arp, aci, av = random_csr(rng, 37, 29, 0.15, dtype=dtype, empty_rows=(2,), lo=0.5, hi=1.5)
    brp, bci, bv = random_csr(rng, 29, 41, 0.2, dtype=dtype, empty_rows=(7,), lo=0.5, hi=1.5)
    if np.issubdtype(dtype, np.integer):
        av, bv = np.abs(av) + 1, np.abs(bv) + 1            # no cancellation: scipy's pattern == structural
    rp, ci, v = oracle.spgemm_csr_typed(arp, aci, av, brp, bci, bv, 41)
    A = sp.csr_matrix((av.astype(np.float64), aci, arp), shape=(37, 29))
    B = sp.csr_matrix((bv.astype(np.float64), bci, brp), shape=(29, 41))
    C = (A @ B).tocsr()
    C.sort_indices()
    assert np.array_equal(rp, C.indptr) and np.array_equal(ci, C.indices)
    for i in range(37):
        assert (np.diff(ci[rp[i]:rp[i + 1]]) > 0).all()     # ascending, unique
    np.testing.assert_allclose(v.astype(np.float64), C.data, rtol=1e-5 if dtype == np.float32 else 1e-12)


def test_spgemm_identity_and_empty_operands(oracle):
    rng = np.random.default_rng(15)
    brp, bci, bv = random_csr(rng, 20, 33, 0.2)
    eye_rp, eye_ci, eye_v = np.arange(21, dtype=np.int32), np.arange(20, dtype=np.int32), np.ones(20, np.float32)
    rp, ci, v = oracle.spgemm_csr_typed(eye_rp, eye_ci, eye_v, brp, bci, bv, 33)
    assert np.array_equal(rp, brp) and np.array_equal(ci, bci) and np.array_equal(v, bv)
    rp, ci, v = oracle.spgemm_csr_typed(np.zeros(6, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32),
                                        brp, bci, bv, 33)
    assert rp.tolist() == [0] * 6 and ci.size == 0 and v.size == 0


def _coo(rp, ci):
    return np.repeat(np.arange(rp.size - 1, dtype=np.int32), np.diff(rp)), ci


def test_spmm_coo_is_the_csr_product_and_adds_repeated_coordinates(oracle):
    rng = np.random.default_rng(61)
    rp, ci, v = random_csr(rng, 40, 30, 0.2, empty_rows=(0, 7))
    B = rng.standard_normal((30, 13)).astype(np.float32)
    r, c = _coo(rp, ci)
    dense = np.zeros((40, 30))
    np.add.at(dense, (r, c), v.astype(np.float64))
    got = oracle.spmm_coo_f32(r, c, v, B, 40)
    assert oracle.rel_fro(got, dense @ B.astype(np.float64)) < 1e-6
    np.testing.assert_allclose(got, oracle.spmm_csr_typed(rp, ci, v, B), rtol=2e-6, atol=1e-6)
    # any order of the entries, every entry twice: twice the product
    order = rng.permutation(r.size)
    twice = oracle.spmm_coo_f32(np.tile(r[order], 2), np.tile(c[order], 2), np.tile(v[order], 2), B, 40)
    assert oracle.rel_fro(twice, 2 * (dense @ B.astype(np.float64))) < 1e-6


def test_spgemm_coo_is_the_csr_product_in_coordinates(oracle):
    rng = np.random.default_rng(62)
    arp, aci, av = random_csr(rng, 35, 28, 0.15, empty_rows=(2,))
    brp, bci, bv = random_csr(rng, 28, 50, 0.12, empty_rows=(0,))
    ar, ac = _coo(arp, aci)
    br, bc = _coo(brp, bci)
    shuffle = rng.permutation(br.size)  # B in any order
    r, k, v = oracle.spgemm_coo_f32(ar, ac, av, br[shuffle], bc[shuffle], bv[shuffle])
    crp, cci, cv = oracle.spgemm_csr_typed(arp, aci, av, brp, bci, bv, 50)
    assert np.array_equal(r, np.repeat(np.arange(35, dtype=np.int32), np.diff(crp)))
    assert np.array_equal(k, cci)
    np.testing.assert_allclose(v, cv, rtol=1e-5, atol=1e-6)
    full = oracle.spgemm_fp64(arp, aci, av, brp, bci, bv, (35, 28), 50)
    assert oracle.rel_fro(v, full[r, k]) < 1e-6
    assert np.count_nonzero(full) <= r.size  # nothing structural is missing


def test_spgemm_coo_emits_one_group_per_run_of_rows(oracle):
    # row 1 appears in two separate runs of A: two groups of output entries, as in the reference's loop
    ar = np.array([1, 0, 1], np.int32); ac = np.array([0, 0, 1], np.int32)
    av = np.array([2.0, 3.0, 5.0], np.float32)
    br = np.array([0, 1], np.int32); bc = np.array([1, 1], np.int32); bv = np.array([1.0, 10.0], np.float32)
    r, k, v = oracle.spgemm_coo_f32(ar, ac, av, br, bc, bv)
    assert list(r) == [1, 0, 1] and list(k) == [1, 1, 1] and list(v) == [2.0, 3.0, 50.0]
