"""CSR x CSR -> CSR on the MI355X through the C ABI.

Structure (row_ptr, col_idx) is compared bit for bit with the oracle, which is
itself bit-identical to the reference's; values to 1e-5 relative Frobenius
error against fp64 (floating point) or bit for bit (integers).
"""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

import scorch_amd as scorch
from conftest import random_csr
from gpu_util import dev, host
from scorch_amd import STensor
from scorch_amd import scorch_ops_hip as H
from scorch_amd import workloads

pytestmark = pytest.mark.gpu
SYMBOL = {np.dtype(np.float32): "prebuilt_spmspm_csr_f32", np.dtype(np.float64): "prebuilt_spmspm_csr_f64",
          np.dtype(np.int32): "prebuilt_spmspm_csr_i32", np.dtype(np.int64): "prebuilt_spmspm_csr_i64"}


def hip_spgemm(arp, aci, av, brp, bci, bv, n_cols):
    M, K = len(arp) - 1, len(brp) - 1
    out = getattr(H, SYMBOL[np.dtype(av.dtype)])(
        [M, n_cols], [M, K], [[], [dev(arp), dev(aci)]], dev(av), [K, n_cols], [[], [dev(brp), dev(bci)]], dev(bv))
    idx = out.storage.index.mode_indices
    assert idx[0] == []
    return host(idx[1][0]), host(idx[1][1]), host(out.storage.value)


def check(oracle, arp, aci, av, brp, bci, bv, n_cols):
    rp, ci, v = hip_spgemm(arp, aci, av, brp, bci, bv, n_cols)
    wrp, wci, wv = oracle.spgemm_csr_typed(arp, aci, av, brp, bci, bv, n_cols)
    assert rp.dtype == np.int32 and ci.dtype == np.int32
    assert np.array_equal(rp, wrp), "row pointer differs"
    assert np.array_equal(ci, wci), "column indices differ"
    if np.issubdtype(av.dtype, np.integer):
        assert np.array_equal(v, wv)
    else:
        # fp64 values on the same structure (the oracle's structure is the reference's, checked above)
        _, _, ref64 = oracle.spgemm_csr_typed(arp, aci, av.astype(np.float64), brp, bci, bv.astype(np.float64),
                                              n_cols)
        assert oracle.rel_fro(v, ref64) <= (1e-5 if av.dtype == np.float32 else 1e-13)
    return rp, ci, v


@pytest.mark.parametrize("name", ["spgemm_f32", "spgemm_f64", "spgemm_i32", "spgemm_i64", "spgemm_cancel"])
def test_golden(golden, name):
    c = golden.case(name)
    rp, ci, v = hip_spgemm(c["a_row_ptr"], c["a_col_idx"], c["a_vals"], c["b_row_ptr"], c["b_col_idx"],
                           c["b_vals"], int(c["n_cols"]))
    assert np.array_equal(rp, c["c_row_ptr"]) and np.array_equal(ci, c["c_col_idx"])
    if np.issubdtype(v.dtype, np.integer):
        assert np.array_equal(v, c["c_vals"])
    else:
        np.testing.assert_allclose(v, c["c_vals"], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
def test_small_rows_one_wavefront_each(oracle, dtype):
    rng = np.random.default_rng(1)
    arp, aci, av = random_csr(rng, 700, 500, 0.01, dtype=dtype, empty_rows=(0, 699))
    brp, bci, bv = random_csr(rng, 500, 900, 0.012, dtype=dtype, empty_rows=(3,))
    check(oracle, arp, aci, av, brp, bci, bv, 900)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int64])
def test_medium_rows_one_workgroup_each(oracle, dtype):
    # ~60 entries per A row x ~40 per B row = ~2400 products: the LDS-hash workgroup path
    rng = np.random.default_rng(2)
    arp, aci, av = random_csr(rng, 150, 600, 0.1, dtype=dtype)
    brp, bci, bv = random_csr(rng, 600, 3000, 0.013, dtype=dtype)
    rp, _, _ = check(oracle, arp, aci, av, brp, bci, bv, 3000)
    assert np.diff(rp).max() > 256


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32])
def test_huge_rows_bitmap_path_and_all_three_mixed(oracle, dtype):
    # a few A rows select hundreds of B rows of ~100 entries (> 4096 products), the rest are small
    rng = np.random.default_rng(3)
    lens = rng.integers(0, 6, 400)
    lens[[7, 123, 399]] = [300, 650, 90]
    arp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    aci = np.concatenate([np.sort(rng.choice(800, int(n), replace=False)) for n in lens]).astype(np.int32)
    av = (rng.integers(-9, 9, aci.size) if np.issubdtype(dtype, np.integer)
          else rng.uniform(-1, 1, aci.size)).astype(dtype)
    brp, bci, bv = random_csr(rng, 800, 5000, 0.02, dtype=dtype)
    rp, _, _ = check(oracle, arp, aci, av, brp, bci, bv, 5000)
    assert np.diff(rp).max() > 4096


@pytest.mark.parametrize("n_cols,dtype", [(100_000, np.float32), (100_000, np.float64), (300_000, np.float32),
                                          (300_000, np.int64), (600_000, np.float32), (600_000, np.float64),
                                          (1_500_000, np.int32), (4_300_000, np.float32),
                                          (4_300_000, np.float64), (4_300_000, np.int32)])
def test_bitmap_tier_by_width(oracle, n_cols, dtype):
    """Rows beyond 4096 products at several widths of B: bitmap in LDS (4096 and
    16384 words, the wider ones in two and three ranges of columns) and in
    global memory.  One row has ~39,000 distinct columns, more than the LDS
    accumulators hold at the narrow widths; the others fit."""
    rng = np.random.default_rng(7)
    lens = rng.integers(0, 4, 60)
    lens[[5, 31, 59]] = [500, 120, 60]
    arp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    aci = np.concatenate([np.sort(rng.choice(900, int(n), replace=False)) for n in lens]).astype(np.int32)
    av = (rng.integers(-9, 9, aci.size) if np.issubdtype(dtype, np.integer)
          else rng.uniform(-1, 1, aci.size)).astype(dtype)
    b_lens = np.full(900, 100)
    brp = np.concatenate([[0], np.cumsum(b_lens)]).astype(np.int32)
    def distinct_sorted(count):
        cols = np.unique(rng.integers(0, n_cols, 2 * count))
        return np.sort(rng.choice(cols, count, replace=False))
    bci = np.concatenate([distinct_sorted(100) for _ in range(900)]).astype(np.int32)
    bv = (rng.integers(-9, 9, bci.size) if np.issubdtype(dtype, np.integer)
          else rng.uniform(-1, 1, bci.size)).astype(dtype)
    rp, _, _ = check(oracle, arp, aci, av, brp, bci, bv, n_cols)
    assert np.diff(rp).max() > 36_000


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int64])
def test_clustered_columns_fall_back_to_the_whole_row_sort(oracle, dtype):
    """Rows whose columns crowd a few sorting buckets: a dense run of columns plus
    one far outlier stretches the bucket width, so the run lands in a handful of
    buckets and the kernel has to sort the whole row instead.  One row for each
    workgroup tier (about 600 and about 2400 products), each column hit twice."""
    n_cols = 1 << 20
    rng = np.random.default_rng(21)
    b_rows, b_cols = [], []
    for r, (lo, hi) in enumerate([(5000, 5300), (5150, 5450), (70000, 71200), (70600, 71800)]):
        cols = np.arange(lo, hi)
        if r % 2:
            cols = np.append(cols, n_cols - 1 - r)  # the outlier
        b_rows.append(np.full(cols.size, r))
        b_cols.append(cols)
    b_rows, b_cols = np.concatenate(b_rows), np.concatenate(b_cols)
    B = sp.csr_matrix((rng.integers(1, 5, b_cols.size).astype(dtype), (b_rows, b_cols)), shape=(4, n_cols))
    A = sp.csr_matrix((np.array([2, 3, 1, 2, 1], dtype), (np.array([0, 0, 1, 1, 2]), np.array([0, 1, 2, 3, 0]))),
                      shape=(3, 4))
    A.sort_indices(), B.sort_indices()
    rp, ci, _ = check(oracle, A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data,
                      B.indptr.astype(np.int32), B.indices.astype(np.int32), B.data, n_cols)
    assert list(np.diff(rp)) == [451, 1801, 300]


@pytest.mark.parametrize("n,dtype", [(3000, np.float32), (3000, np.float64), (3000, np.int32),
                                     (140_000, np.float32)])
def test_many_products_on_few_distinct_columns(oracle, n, dtype):
    """A band of 69 entries per row, squared: 4761 products per row on 137 distinct
    columns.  The symbolic pass files such rows by their products; the numeric pass,
    which knows their length, gives them to the tier of at most 4096 output entries
    when B is no wider than that tier's bitmap (n = 3000; not at n = 140,000)."""
    half = 34
    rng = np.random.default_rng(23)
    rows = np.arange(n)[:, None]
    cols = rows + np.arange(-half, half + 1)[None, :]
    keep = (cols >= 0) & (cols < n)
    lens = keep.sum(axis=1)
    arp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    aci = cols[keep].astype(np.int32)
    av = (rng.integers(-9, 9, aci.size) if np.issubdtype(dtype, np.integer)
          else rng.uniform(-1, 1, aci.size)).astype(dtype)
    rp, _, _ = check(oracle, arp, aci, av, arp, aci, av, n)
    assert np.diff(rp).max() == 4 * half + 1 and lens.max() ** 2 > 4096


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
def test_wavefront_rows_sorted_by_buckets_and_by_rank(oracle, dtype):
    """Rows of 65 to 256 output entries (a wavefront each) are sorted by buckets over
    their column range, unless the columns crowd a few buckets: row 0 spreads 200
    columns evenly, row 1 has a run of 120 consecutive columns and two far outliers
    (one bucket would hold the whole run: the rank count takes over), row 2 puts
    exactly 17 columns into one bucket, one more than a bucket may hold, row 3 has
    64 entries (rank count by size) and row 4 has 256, each column hit twice."""
    n_cols = 1 << 20
    rng = np.random.default_rng(29)
    b_cols = [np.sort(rng.choice(n_cols, 200, replace=False)),
              np.concatenate([[5], np.arange(1000, 1120), [900_000]]),
              np.concatenate([np.arange(0, 17), np.arange(1, 100) * 8192]),
              np.sort(rng.choice(n_cols, 64, replace=False)),
              np.sort(rng.choice(n_cols, 128, replace=False)),
              np.sort(rng.choice(n_cols, 128, replace=False))]
    b_cols[5][:64] = b_cols[4][:64]          # half of row 4's columns come from both B rows
    b_cols[5] = np.unique(b_cols[5])
    brp = np.concatenate([[0], np.cumsum([c.size for c in b_cols])]).astype(np.int32)
    bci = np.concatenate(b_cols).astype(np.int32)
    draw = (lambda k: rng.integers(1, 9, k)) if np.issubdtype(dtype, np.integer) else (lambda k: rng.uniform(0.5, 1.5, k))
    bv = draw(bci.size).astype(dtype)
    arp = np.array([0, 1, 2, 3, 4, 6], np.int32)
    aci = np.array([0, 1, 2, 3, 4, 5], np.int32)
    av = draw(aci.size).astype(dtype)
    rp, ci, _ = check(oracle, arp, aci, av, brp, bci, bv, n_cols)
    assert list(np.diff(rp)[:4]) == [200, 122, 116, 64] and 128 < np.diff(rp)[4] <= 256


@pytest.mark.parametrize("n_cols", [3000, 15_000, 16_500, 31_000, 34_000])
@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int64])
def test_bitmap_tiers_around_the_widths_that_fit_sums_by_column(oracle, n_cols, dtype):
    """B no wider than the sums a workgroup keeps in LDS (about 32 K four-byte or
    16 K eight-byte values with 1024 threads, 4096 with 256) has its rows summed by
    column in one walk; wider, by rank in two.  Rows of about 2,000, 6,000 and
    40,000 products on either side of those widths, some columns hit many times."""
    rng = np.random.default_rng(31)
    lens = rng.integers(0, 3, 40)
    lens[[3, 17, 39]] = [20, 60, 400]
    arp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    aci = np.concatenate([np.sort(rng.choice(500, int(n), replace=False)) for n in lens]).astype(np.int32)
    b_cols = [np.sort(rng.choice(n_cols, 100, replace=False)) for _ in range(500)]
    brp = np.arange(501, dtype=np.int32) * 100
    bci = np.concatenate(b_cols).astype(np.int32)
    draw = (lambda k: rng.integers(-9, 9, k)) if np.issubdtype(dtype, np.integer) else (lambda k: rng.uniform(-1, 1, k))
    av, bv = draw(aci.size).astype(dtype), draw(bci.size).astype(dtype)
    rp, _, _ = check(oracle, arp, aci, av, brp, bci, bv, n_cols)
    assert np.diff(rp)[39] > 2000


def test_structure_is_the_same_on_every_run_and_inputs_untouched(oracle):
    rng = np.random.default_rng(4)
    arp, aci, av = random_csr(rng, 300, 300, 0.05)
    first = hip_spgemm(arp, aci, av, arp, aci, av, 300)
    for _ in range(3):
        again = hip_spgemm(arp, aci, av, arp, aci, av, 300)
        assert np.array_equal(first[0], again[0]) and np.array_equal(first[1], again[1])
        np.testing.assert_allclose(first[2], again[2], rtol=1e-5, atol=1e-6)   # atomics: summation order varies


def test_empty_operands():
    z = np.zeros(0, np.int32)
    rp, ci, v = hip_spgemm(np.zeros(6, np.int32), z, np.zeros(0, np.float32), np.zeros(4, np.int32), z,
                           np.zeros(0, np.float32), 9)
    assert rp.tolist() == [0] * 6 and ci.size == 0 and v.size == 0


@pytest.mark.parametrize("use_cache", [True, False])
def test_sparse_stensor_spgemm_does_not_call_torch_matmul(use_cache, monkeypatch):
    """reference: tests/test_scorch/test_matmul_dispatch.py:30-48 (with the CSR result kept sparse)"""
    from scorch_amd import ops
    torch.manual_seed(1)
    n = 32
    a_t = torch.rand(n, n) * (torch.rand(n, n) < 0.05)
    b_t = torch.rand(n, n) * (torch.rand(n, n) < 0.05)
    expected = torch.matmul(a_t, b_t)
    a = STensor.from_torch(a_t, "A").to_sparse("ds").to("cuda")
    b = STensor.from_torch(b_t, "B").to_sparse("ds").to("cuda")

    def forbidden(*args, **kwargs):
        raise AssertionError("torch.matmul should not be used for sparse STensor matmul")

    monkeypatch.setattr(ops.torch, "matmul", forbidden)
    out = scorch.matmul(a, b, use_cache=use_cache)
    assert isinstance(out, STensor) and str(out.format) == "d,s" and out.shape == (n, n)
    assert torch.allclose(out.to_torch().cpu(), expected, atol=1e-5)


@pytest.mark.parametrize("nodes", [131072, 524288])
def test_graph_squared_at_the_benchmark_sizes(oracle, nodes):
    """A @ A for the benchmark's graphs (bench.py --workload spgemm_powerlaw and four times as
    many nodes): 30 M and 120 M result entries, structure bit for bit, values against fp64."""
    from scorch_amd import workloads
    w = workloads.gcn_powerlaw(M=nodes, N=4, max_degree=5000)
    rp, _, _ = check(oracle, w["row_ptr"], w["col_idx"], w["vals"], w["row_ptr"], w["col_idx"], w["vals"], nodes)
    assert rp[-1] > 200 * nodes


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.int64])
def test_many_rows_of_few_products(oracle, dtype):
    """Enough rows (>= 32,768) for wavefronts to take four rows each: rows of 0 to 32 products go
    to quarter wavefronts, their neighbours of up to 256 to the whole wavefront in turn, a few
    beyond that to the workgroup kernels.  Tridiagonal-like with denser stretches."""
    M = 40_003
    rng = np.random.default_rng(31)
    lens = rng.integers(0, 4, M)
    lens[rng.integers(0, M, 3000)] = rng.integers(4, 17, 3000)   # up to 16 x 16 = 256 products
    lens[rng.integers(0, M, 40)] = rng.integers(300, 900, 40)    # beyond the wavefront tier
    lens[[0, M - 1]] = [0, 3]
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    cols = np.concatenate([np.sort(rng.choice(M, int(n), replace=False)) for n in lens]).astype(np.int32)
    vals = (rng.integers(-9, 9, cols.size) if np.issubdtype(dtype, np.integer)
            else rng.uniform(-1, 1, cols.size)).astype(dtype)
    products = np.zeros(M, np.int64)
    np.add.at(products, np.repeat(np.arange(M), lens), lens[cols])
    assert (products <= 32).sum() > 30_000 and ((products > 32) & (products <= 256)).sum() > 300
    assert (products > 256).sum() >= 30 and (products == 0).any()
    check(oracle, rp, cols, vals, rp, cols, vals, M)


def test_graph_squared_power_law(oracle):
    """A @ A for a power-law graph: rows from one entry to tens of thousands."""
    from scorch_amd import workloads
    w = workloads.gcn_powerlaw(M=20000, N=4, seed=21, max_degree=3000)
    check(oracle, w["row_ptr"], w["col_idx"], w["vals"], w["row_ptr"], w["col_idx"], w["vals"], 20000)


# ---- all three in coordinate form (the reference's spmspm_coo_float) -----------------------
def hip_spgemm_coo(ar, ac, av, br, bc, bv, shape):
    M, K, N = (int(x) for x in shape)
    out = H.spmspm_coo_float([M, N], [M, K], [[dev(ar)], [dev(ac)]], dev(av), [K, N], [[dev(br)], [dev(bc)]],
                             dev(bv))
    idx = out.storage.index.mode_indices
    return host(idx[0][0]), host(idx[1][0]), host(out.storage.value)


@pytest.mark.parametrize("name", ["spgemm_coo", "spgemm_coo_cancel"])
def test_golden_coordinate_operands(golden, name):
    c = golden.case(name)
    r, k, v = hip_spgemm_coo(c["a_row_idx"], c["a_col_idx"], c["a_vals"], c["b_row_idx"], c["b_col_idx"],
                             c["b_vals"], c["shape"])
    assert r.dtype == np.int32 and k.dtype == np.int32
    assert np.array_equal(r, c["c_row_idx"]) and np.array_equal(k, c["c_col_idx"])
    np.testing.assert_allclose(v, c["c_vals"], rtol=1e-5, atol=1e-6)


def test_coordinate_operands_give_the_csr_product(oracle):
    rng = np.random.default_rng(73)
    arp, aci, av = random_csr(rng, 900, 700, 0.01, empty_rows=(0,))
    brp, bci, bv = random_csr(rng, 700, 1500, 0.01, empty_rows=(5,))
    ar = np.repeat(np.arange(900, dtype=np.int32), np.diff(arp))
    br = np.repeat(np.arange(700, dtype=np.int32), np.diff(brp))
    shuffle = rng.permutation(br.size)  # B in any storage order
    r, k, v = hip_spgemm_coo(ar, aci, av, br[shuffle], bci[shuffle], bv[shuffle], (900, 700, 1500))
    wrp, wci, _ = oracle.spgemm_csr_typed(arp, aci, av, brp, bci, bv, 1500)
    assert np.array_equal(r, np.repeat(np.arange(900, dtype=np.int32), np.diff(wrp)))
    assert np.array_equal(k, wci)
    _, _, ref64 = oracle.spgemm_csr_typed(arp, aci, av.astype(np.float64), brp, bci, bv.astype(np.float64), 1500)
    assert oracle.rel_fro(v, ref64) <= 1e-5


def test_coordinate_stensors_multiply_on_the_device():
    torch.manual_seed(3)
    a_t = torch.rand(40, 30) * (torch.rand(40, 30) < 0.1)
    b_t = torch.rand(30, 20) * (torch.rand(30, 20) < 0.15)
    a = STensor.from_torch(a_t, "A").to_sparse("oo").to("cuda")
    b = STensor.from_torch(b_t, "B").to_sparse("oo").to("cuda")
    out = scorch.matmul(a, b)
    assert isinstance(out, STensor) and str(out.format) == "o,o" and out.shape == (40, 20)
    assert torch.allclose(out.to_torch().cpu(), a_t @ b_t, atol=1e-5)
    dense = scorch.matmul(a, STensor.from_torch(b_t, "B").to("cuda"))
    assert isinstance(dense, torch.Tensor) and torch.allclose(dense.cpu(), a_t @ b_t, atol=1e-5)


def test_result_beyond_the_int32_row_pointer_is_reported():
    """32,769 rows that each select one dense row of 65,536 entries: 2^31 + 65,536 result entries.
    The symbolic pass counts them in 64 bits and says so instead of wrapping the row pointer."""
    from scorch_amd import native
    M, N = (1 << 15) + 1, 1 << 16
    a_pos = torch.arange(M + 1, dtype=torch.int32, device="cuda")
    a_crd = torch.zeros(M, dtype=torch.int32, device="cuda")
    b_pos = torch.tensor([0, N], dtype=torch.int32, device="cuda")
    b_crd = torch.arange(N, dtype=torch.int32, device="cuda")
    with pytest.raises(native.ScorchHipError, match="2\\^31") as err:
        H.prebuilt_spmspm_csr_f32([M, N], [M, 1], [[], [a_pos, a_crd]], torch.ones(M, device="cuda"), [1, N],
                                  [[], [b_pos, b_crd]], torch.ones(N, device="cuda"))
    assert err.value.code == native.EUNSUPPORTED
    # one row fewer fits: the symbolic pass alone (the result itself would take 17 GB)
    M -= 2
    L = native.lib()
    c_pos = torch.empty(M + 1, dtype=torch.int32, device="cuda")
    ws = torch.empty(L.scorch_hip_spgemm_csr_workspace_bytes(M, N, 1), dtype=torch.uint8, device="cuda")
    native.check(L.scorch_hip_spgemm_csr_symbolic(M, 1, N, a_pos.data_ptr(), a_crd.data_ptr(), b_pos.data_ptr(),
                                                  b_crd.data_ptr(), c_pos.data_ptr(), ws.data_ptr(), ws.numel(),
                                                  torch.cuda.current_stream().cuda_stream))
    assert int(c_pos[-1]) == M * N and int(c_pos[1]) == N


def test_reproducible_mode_gives_the_same_bits_on_every_run(oracle, monkeypatch):
    """fp32 sums in 64-bit fixed point: identical values from run to run (the default mode's
    atomics only promise that to rounding), the same structure, and within the fp32 bar of fp64."""
    w = workloads.gcn_powerlaw(M=30_000, N=1, seed=13, max_degree=4000)
    rp, ci, v = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"])
    shape = [30_000, 30_000]
    call = lambda: H.prebuilt_spmspm_csr_f32(shape, shape, [[], [rp, ci]], v, shape, [[], [rp, ci]], v)
    plain = call()
    monkeypatch.setattr(H, "SPGEMM_REPRODUCIBLE", True)
    runs = [call() for _ in range(3)]
    for r in runs[1:]:
        assert torch.equal(r.storage.value, runs[0].storage.value)
    for mine, theirs in zip(runs[0].storage.index.mode_indices[1], plain.storage.index.mode_indices[1]):
        assert torch.equal(mine, theirs)
    A = sp.csr_matrix((w["vals"].astype(np.float64), w["col_idx"], w["row_ptr"]), shape=(30_000, 30_000))
    ref = (A @ A).tocsr()
    ref.sort_indices()
    assert np.array_equal(host(runs[0].storage.index.mode_indices[1][1]), ref.indices)
    assert oracle.rel_fro(host(runs[0].storage.value), ref.data) <= 1e-5
    assert oracle.rel_fro(host(plain.storage.value), ref.data) <= 1e-5
    # the COO x COO symbol and matmul go the same way
    small = H.spmspm_csr_float([3, 3], [3, 3], [[], [dev(np.array([0, 1, 2, 3], np.int32)),
                                                      dev(np.array([2, 0, 1], np.int32))]], dev(np.array([0.5, -2.0, 3.0], np.float32)),
                               [3, 3], [[], [dev(np.array([0, 1, 2, 3], np.int32)), dev(np.array([1, 2, 0], np.int32))]],
                               dev(np.array([4.0, 0.25, -1.0], np.float32)))
    assert host(small.storage.value).tolist() == [-0.5, -8.0, 0.75]
