"""Invariants of the seeded workload generators (small sizes)."""
import numpy as np

from scorch_amd import workloads


def rows_sorted_unique(row_ptr, col_idx):
    for i in range(len(row_ptr) - 1):
        seg = col_idx[row_ptr[i]:row_ptr[i + 1]]
        if seg.size > 1 and not (np.diff(seg) > 0).all():
            return False
    return True


def test_generators_are_deterministic():
    a = workloads.gcn_powerlaw(M=500, N=8, seed=9)
    b = workloads.gcn_powerlaw(M=500, N=8, seed=9)
    assert all(np.array_equal(a[k], b[k]) for k in ("row_ptr", "col_idx", "vals", "B"))
    c = workloads.gcn_powerlaw(M=500, N=8, seed=10)
    assert not np.array_equal(a["col_idx"], c["col_idx"])


def test_spmm_uniform_shape_and_density():
    w = workloads.spmm_uniform(M=512, K=400, N=16, density=0.02, seed=1)
    assert w["row_ptr"].dtype == np.int32 and w["col_idx"].dtype == np.int32
    assert w["row_ptr"][0] == 0 and w["row_ptr"][-1] == w["col_idx"].size == w["vals"].size
    assert rows_sorted_unique(w["row_ptr"], w["col_idx"])
    assert 0.015 < w["col_idx"].size / (512 * 400) < 0.025
    assert w["col_idx"].min() >= 0 and w["col_idx"].max() < 400 and np.abs(w["vals"]).max() <= 1
    assert w["B"].shape == (400, 16) and w["B"].dtype == np.float32


def test_gcn_powerlaw_structure_and_normalisation():
    w = workloads.gcn_powerlaw(M=4000, N=4, seed=2, max_degree=500)
    rp, ci, v = w["row_ptr"], w["col_idx"], w["vals"]
    assert rows_sorted_unique(rp, ci)
    deg = np.diff(rp)
    rows = np.repeat(np.arange(4000), deg)
    assert ((rows == ci).reshape(-1).sum()) == 4000           # exactly one self-loop per node
    assert deg.min() >= 1 and deg.max() <= 501 and deg.max() > 10 * np.median(deg)  # heavy tail
    assert 8 < deg.mean() < 24
    expect = 1.0 / np.sqrt(deg[rows].astype(np.float64) * deg[ci].astype(np.float64))
    np.testing.assert_allclose(v, expect, rtol=1e-6)


def test_sddmm_uniform_has_exact_row_length():
    w = workloads.sddmm_uniform(M=300, n_cols=200, per_row=16, K=8, seed=3)
    assert (np.diff(w["row_ptr"]) == 16).all() and rows_sorted_unique(w["row_ptr"], w["col_idx"])
    assert np.array_equal(w["row_idx"], np.repeat(np.arange(300), 16))
    assert (w["vals"] == 1).all() and w["A"].shape == (300, 8) and w["B"].shape == (200, 8)
    assert abs(w["A"].std() - np.sqrt(1 / 8)) < 0.02
    u = workloads.sddmm_uniform(M=30, n_cols=20, per_row=4, K=8, seed=3, unit_mask=False)
    assert u["vals"].min() < 0 < u["vals"].max()


def test_blocksparse_pattern_counts():
    brp, bci = workloads.blocksparse_pattern(128)
    assert bci.size == 1466                                  # S = 8192, 64-wide blocks
    for bi in range(128):
        cols = bci[brp[bi]:brp[bi + 1]]
        assert cols.max() == bi and (cols <= bi).all()
        assert all((bi - c < 4) or ((bi - c) % 8 == 0) for c in cols)
    rp, ci = workloads.blocks_to_csr(*workloads.blocksparse_pattern(4), block=8)
    assert rp[-1] == ci.size == 10 * 64 and rows_sorted_unique(rp, ci)


def test_sae_decoder_topk():
    w = workloads.sae_decoder(M=64, K=512, N=32, k=8, seed=4)
    assert (np.diff(w["row_ptr"]) == 8).all() and rows_sorted_unique(w["row_ptr"], w["col_idx"])
    assert (w["vals"] > 0).all() and w["B"].shape == (512, 32)
    assert abs(w["B"].std() - 0.125) < 0.01


def test_gcn_powerlaw_neighbour_window():
    """window > 0: every neighbour lies within window / 2 of its row (wrapping), the degrees keep their
    shape, and the normalisation is unchanged."""
    M, W = 5000, 64
    w = workloads.gcn_powerlaw(M=M, N=4, seed=3, max_degree=400, window=W)
    rows = np.repeat(np.arange(M), np.diff(w["row_ptr"]))
    gap = np.abs(w["col_idx"].astype(np.int64) - rows)
    gap = np.minimum(gap, M - gap)
    assert gap.max() <= W // 2 and (gap == 0).sum() == M          # self-loops included
    assert np.all(np.diff(w["row_ptr"]) >= 1) and np.diff(w["row_ptr"]).max() <= W
    d = np.diff(w["row_ptr"]).astype(np.float64)
    np.testing.assert_allclose(w["vals"], 1 / np.sqrt(d[rows] * d[w["col_idx"]]), rtol=1e-6)
    plain = workloads.gcn_powerlaw(M=M, N=4, seed=3, max_degree=400)
    assert np.abs(plain["col_idx"].astype(np.int64) - np.repeat(np.arange(M), np.diff(plain["row_ptr"]))).max() > M // 4


def test_longformer_mask_matches_the_reference_benchmarks_counts():
    """reference: bench/README_sparse_transformer.md:78-81 (window 64 on either side, one global
    token): 62,782 entries at S = 512, 532,286 at S = 4096; and the definition itself
    (bench/bench_sparse_transformer.py:194-209) on a small dense mask."""
    for S, nnz in ((512, 62_782), (4096, 532_286)):
        rp, ci = workloads.longformer_mask(S)
        assert rp[-1] == ci.size == nnz and rows_sorted_unique(rp, ci)
    S, w, g = 40, 3, 2
    rp, ci = workloads.longformer_mask(S, window=w, n_global=g)
    dense = np.zeros((S, S), bool)
    dense[np.repeat(np.arange(S), np.diff(rp)), ci] = True
    i, j = np.indices((S, S))
    assert np.array_equal(dense, (np.abs(i - j) <= w) | (i < g) | (j < g))
