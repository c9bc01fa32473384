"""The C restatement (oracle/scorch_oracle.c) against the reference's own
outputs stored in tests/golden/golden_ref.npz (made by tests/golden/make_golden.py
from the reference's compiled native module).

Integer results must be identical.  Floating-point results are compared at a
few ulps: both sides run the same loop order, but under -ffast-math the
compiler is free to contract and vectorise the two builds differently.
"""
import numpy as np
import pytest

FP_RTOL = 2e-6
FP_ATOL = 1e-6

SPMM_F32_CASES = ["spmm_square95", "spmm_dispatch32", "spmm_rect", "spmm_wide300", "spmm_emptyrows",
                  "spmm_n1", "spmm_longrow", "spmm_allzero", "spmm_diag_literal"]


def test_golden_file_lists_expected_cases(golden):
    for name in SPMM_F32_CASES + ["spmm_f64", "spmm_i32", "spmm_i64", "spmm_i32_wrap", "spmm_bias",
                                  "sddmm_16_8", "sddmm_256_64", "sddmm_rect_k13", "spmv_i64_literal"]:
        assert name in golden.names


@pytest.mark.parametrize("name", SPMM_F32_CASES)
def test_spmm_v2_matches_reference_output(golden, oracle, name):
    c = golden.case(name)
    got = oracle.spmm_csr_f32_v2(c["row_ptr"], c["col_idx"], c["vals"], c["B"])
    assert got.shape == c["C_v2"].shape
    np.testing.assert_allclose(got, c["C_v2"], rtol=FP_RTOL, atol=FP_ATOL)


@pytest.mark.parametrize("name", SPMM_F32_CASES)
def test_spmm_typed_f32_matches_reference_output(golden, oracle, name):
    c = golden.case(name)
    got = oracle.spmm_csr_typed(c["row_ptr"], c["col_idx"], c["vals"], c["B"])
    np.testing.assert_allclose(got, c["C_typed"], rtol=FP_RTOL, atol=FP_ATOL)


def test_spmm_diag_literal_is_exact(golden, oracle):
    c = golden.case("spmm_diag_literal")
    expect = np.diag(np.arange(1, 6, dtype=np.float32)) @ c["B"]
    assert np.array_equal(c["C_v2"], expect)  # the fixture itself
    assert np.array_equal(oracle.spmm_csr_f32_v2(c["row_ptr"], c["col_idx"], c["vals"], c["B"]), expect)


def test_spmm_f64_matches_reference_output(golden, oracle):
    c = golden.case("spmm_f64")
    got = oracle.spmm_csr_typed(c["row_ptr"], c["col_idx"], c["vals"], c["B"])
    assert got.dtype == np.float64
    np.testing.assert_allclose(got, c["C_typed"], rtol=1e-14, atol=1e-14)


@pytest.mark.parametrize("name", ["spmm_i32", "spmm_i64", "spmm_i32_wrap"])
def test_spmm_integer_is_bit_exact(golden, oracle, name):
    c = golden.case(name)
    got = oracle.spmm_csr_typed(c["row_ptr"], c["col_idx"], c["vals"], c["B"])
    assert got.dtype == c["C_typed"].dtype
    assert np.array_equal(got, c["C_typed"])


def test_spmm_i32_wrap_really_wraps(golden):
    c = golden.case("spmm_i32_wrap")
    rows = np.repeat(np.arange(len(c["row_ptr"]) - 1), np.diff(c["row_ptr"]))
    exact = np.zeros(c["C_typed"].shape, dtype=object)
    for r, j, v in zip(rows, c["col_idx"], c["vals"]):
        exact[r] += int(v) * c["B"][j].astype(object)
    wrapped = np.vectorize(lambda t: ((int(t) + 2 ** 31) % 2 ** 32) - 2 ** 31)(exact).astype(np.int64)
    assert np.abs(exact.astype(np.float64)).max() > 2 ** 31  # the case does overflow
    assert np.array_equal(wrapped, c["C_typed"].astype(np.int64))


@pytest.mark.parametrize("relu", [False, True])
def test_spmm_bias_act_matches_reference_output(golden, oracle, relu):
    c = golden.case("spmm_bias")
    got = oracle.spmm_csr_bias_act_f32(c["row_ptr"], c["col_idx"], c["vals"], c["B"], c["bias"], relu)
    np.testing.assert_allclose(got, c["C_bias_relu" if relu else "C_bias"], rtol=FP_RTOL, atol=FP_ATOL)
    if relu:
        assert (got >= 0).all() and (got == 0).any()


SDDMM_CASES = ["sddmm_16_8", "sddmm_64_32", "sddmm_128_16", "sddmm_256_64", "sddmm_40_16", "sddmm_rect_k13"]


@pytest.mark.parametrize("name", SDDMM_CASES)
def test_sddmm_coo_matches_reference_output(golden, oracle, name):
    c = golden.case(name)
    got = oracle.sddmm_coo_f32(c["row_idx"], c["col_idx"], c["vals"], c["A"], c["B"])
    np.testing.assert_allclose(got, c["out_val"], rtol=1e-5, atol=1e-6)
    # the reference returns the mask's own index arrays
    assert np.array_equal(c["out_row"], c["row_idx"]) and np.array_equal(c["out_col"], c["col_idx"])


@pytest.mark.parametrize("name", SDDMM_CASES)
def test_sddmm_csr_gives_coordinate_result_in_mask_order(golden, oracle, name):
    c = golden.case(name)
    row, col, val = oracle.sddmm_csr_f32(c["row_ptr"], c["col_idx"], c["vals"], c["A"], c["B"])
    assert np.array_equal(row, c["row_idx"]) and np.array_equal(col, c["col_idx"])
    assert val.size == c["vals"].size  # explicit zeros are kept
    np.testing.assert_allclose(val, c["out_val"], rtol=1e-5, atol=1e-6)


def test_sddmm_keeps_explicit_zero_entries(golden):
    c = golden.case("sddmm_rect_k13")
    assert (c["vals"] == 0).any()
    assert (c["out_val"][c["vals"] == 0] == 0).all()


def test_spmv_literal_int64(golden, oracle):
    c = golden.case("spmv_i64_literal")
    assert c["y"].tolist() == [7, 22, 0, 29]
    got = oracle.spmv_csr_typed(c["row_ptr"], c["col_idx"], c["vals"], c["x"])
    assert np.array_equal(got, c["y"])


@pytest.mark.parametrize("name,exact", [("spmv_f32", False), ("spmv_f64", False), ("spmv_i32", True)])
def test_spmv_matches_reference_output(golden, oracle, name, exact):
    c = golden.case(name)
    got = oracle.spmv_csr_typed(c["row_ptr"], c["col_idx"], c["vals"], c["x"])
    if exact:
        assert np.array_equal(got, c["y"])
    else:
        np.testing.assert_allclose(got, c["y"], rtol=1e-5 if name.endswith("f32") else 1e-13, atol=1e-6)


# ---- SpGEMM ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["spgemm_f32", "spgemm_f64", "spgemm_i32", "spgemm_i64", "spgemm_cancel"])
def test_spgemm_matches_reference_output(golden, oracle, name):
    c = golden.case(name)
    rp, ci, v = oracle.spgemm_csr_typed(c["a_row_ptr"], c["a_col_idx"], c["a_vals"], c["b_row_ptr"],
                                        c["b_col_idx"], c["b_vals"], int(c["n_cols"]))
    assert np.array_equal(rp, c["c_row_ptr"]) and np.array_equal(ci, c["c_col_idx"])   # structure: exact
    if np.issubdtype(v.dtype, np.integer):
        assert np.array_equal(v, c["c_vals"])
    else:
        np.testing.assert_allclose(v, c["c_vals"], rtol=1e-6, atol=1e-7)


def test_spgemm_keeps_entries_that_cancel_to_zero(golden):
    c = golden.case("spgemm_cancel")
    assert c["c_row_ptr"].tolist() == [0, 3, 5] and c["c_col_idx"].tolist() == [0, 1, 2, 0, 1]
    assert c["c_vals"][0] == 0.0                      # 1*3 + (-1)*3, stored all the same


@pytest.mark.parametrize("name", ["spmm_coo", "spmm_coo_unsorted"])
def test_spmm_coo_matches_reference_output(golden, oracle, name):
    c = golden.case(name)
    got = oracle.spmm_coo_f32(c["row_idx"], c["col_idx"], c["vals"], c["B"], int(c["n_rows"]))
    np.testing.assert_allclose(got, c["C"], rtol=FP_RTOL, atol=FP_ATOL)


def test_spmm_coo_fixture_does_not_depend_on_the_order_of_runs(golden):
    # the unsorted case repeats row 3's entries: that row doubles, the others agree with the sorted case
    a, b = golden.case("spmm_coo"), golden.case("spmm_coo_unsorted")
    expect = a["C"].copy()
    expect[3] *= 2
    np.testing.assert_allclose(b["C"], expect, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("name", ["spgemm_coo", "spgemm_coo_cancel"])
def test_spgemm_coo_matches_reference_output(golden, oracle, name):
    c = golden.case(name)
    r, k, v = oracle.spgemm_coo_f32(c["a_row_idx"], c["a_col_idx"], c["a_vals"], c["b_row_idx"],
                                    c["b_col_idx"], c["b_vals"])
    assert np.array_equal(r, c["c_row_idx"]) and np.array_equal(k, c["c_col_idx"])
    np.testing.assert_allclose(v, c["c_vals"], rtol=FP_RTOL, atol=FP_ATOL)


def test_spgemm_coo_keeps_cancelled_entries_and_adds_repeated_ones(golden):
    c = golden.case("spgemm_coo_cancel")
    assert list(c["c_row_idx"]) == [0, 0, 0, 1, 1] and list(c["c_col_idx"]) == [0, 1, 2, 0, 1]
    assert list(c["c_vals"]) == [0.0, -7.5, 5.0, 6.0, 15.0]  # 3 - 3; -(7 + 0.5); 5; 2 * 3; 2 * 7.5
