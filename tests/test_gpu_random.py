"""Seeded random sweeps over shapes, densities and dtypes: every kernel against the
oracle on many small cases (sizes drawn so that empty matrices, single rows,
N = 1, odd widths and rows longer than a chunk all occur)."""
import numpy as np
import pytest

from conftest import random_csr
from gpu_util import hip_sddmm_coo, hip_sddmm_csr, hip_spmm, hip_spmv
from test_gpu_spgemm import hip_spgemm

pytestmark = pytest.mark.gpu
DTYPES = [np.float32, np.float64, np.int32, np.int64]


def draw_dense(rng, shape, dtype):
    if np.issubdtype(dtype, np.integer):
        return rng.integers(-1000, 1000, size=shape).astype(dtype)
    return rng.standard_normal(shape).astype(dtype)


def draw_density(rng, cols):
    return float(rng.choice([0.0, 1.0 / max(cols, 1), 0.02, 0.1, 0.5, 1.0]))


@pytest.mark.parametrize("seed", range(40))
def test_spmm_random(oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    M, K = int(rng.integers(1, 700)), int(rng.integers(1, 400))
    N = int(rng.choice([1, 2, 3, 7, 16, 31, 64, 65, 100, 128, 200, 256, 333]))
    dtype = DTYPES[seed % 4]
    rp, ci, v = random_csr(rng, M, K, draw_density(rng, K), dtype=dtype)
    B = draw_dense(rng, (K, N), dtype)
    fused = dtype == np.float32 and seed % 3 == 0
    bias = draw_dense(rng, (N,), dtype) if fused else None
    relu = fused and seed % 2 == 0
    got = hip_spmm(rp, ci, v, B, bias=bias, relu=relu)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got, oracle.spmm_csr_typed(rp, ci, v, B))
        return
    ref = oracle.spmm_fp64(rp, ci, v, B)
    if fused:
        ref = ref + bias.astype(np.float64)
        ref = np.maximum(ref, 0) if relu else ref
    assert oracle.rel_fro(got, ref) <= (1e-5 if dtype == np.float32 else 1e-13), (M, K, N)


@pytest.mark.parametrize("seed", range(24))
def test_spmv_random(oracle, seed):
    rng = np.random.default_rng(2000 + seed)
    M, K = int(rng.integers(1, 3000)), int(rng.integers(1, 900))
    dtype = DTYPES[seed % 4]
    rp, ci, v = random_csr(rng, M, K, draw_density(rng, K), dtype=dtype)
    x = draw_dense(rng, (K,), dtype)
    got = hip_spmv(rp, ci, v, x)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got, oracle.spmv_csr_typed(rp, ci, v, x))
    else:
        ref = oracle.spmm_fp64(rp, ci, v, x.reshape(-1, 1)).reshape(-1)
        assert oracle.rel_fro(got, ref) <= (1e-5 if dtype == np.float32 else 1e-13), (M, K)


@pytest.mark.parametrize("seed", range(24))
def test_sddmm_random(oracle, seed):
    rng = np.random.default_rng(3000 + seed)
    M, n_cols = int(rng.integers(1, 500)), int(rng.integers(1, 500))
    K = int(rng.choice([1, 3, 4, 8, 12, 17, 32, 64, 100, 128, 257]))
    rp, ci, s = random_csr(rng, M, n_cols, draw_density(rng, n_cols))
    rows = oracle.rows_of(rp)
    A, B = draw_dense(rng, (M, K), np.float32), draw_dense(rng, (n_cols, K), np.float32)
    ref = oracle.sddmm_fp64(rows, ci, s, A, B)
    r, c, val = hip_sddmm_csr(rp, ci, s, A, B, (M, n_cols))
    assert np.array_equal(r, rows) and np.array_equal(c, ci)
    assert oracle.rel_fro(val, ref) <= 1e-5, (M, n_cols, K)
    assert np.array_equal(hip_sddmm_coo(rows, ci, s, A, B, (M, n_cols)), val)


@pytest.mark.parametrize("seed", range(24))
def test_spgemm_random(oracle, seed):
    rng = np.random.default_rng(4000 + seed)
    M, K, N = (int(rng.integers(1, 400)) for _ in range(3))
    dtype = DTYPES[seed % 4]
    arp, aci, av = random_csr(rng, M, K, draw_density(rng, K), dtype=dtype)
    brp, bci, bv = random_csr(rng, K, N, draw_density(rng, N), dtype=dtype)
    rp, ci, v = hip_spgemm(arp, aci, av, brp, bci, bv, N)
    wrp, wci, wv = oracle.spgemm_csr_typed(arp, aci, av, brp, bci, bv, N)
    assert np.array_equal(rp, wrp) and np.array_equal(ci, wci), (M, K, N)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(v, wv)
    else:
        np.testing.assert_allclose(v, wv, rtol=1e-4 if dtype == np.float32 else 1e-12,
                                   atol=1e-3 if dtype == np.float32 else 1e-10)


@pytest.mark.parametrize("seed", range(8))
def test_spgemm_random_many_short_rows(oracle, seed):
    """More than 32,768 rows, so that wavefronts take four rows each (quarters for rows of at most
    32 products); mixes of empty, tiny and a few long rows, operands of different shapes."""
    rng = np.random.default_rng(4000 + seed)
    M = int(rng.integers(33_000, 60_000))
    K, N = int(rng.integers(50, 3000)), int(rng.integers(50, 5000))
    dtype = DTYPES[seed % 4]
    a_lens = rng.choice([0, 1, 2, 3, 5, 9], size=M, p=[0.2, 0.3, 0.2, 0.15, 0.1, 0.05])
    a_lens[rng.integers(0, M, 30)] = rng.integers(10, min(K, 200), 30)
    a_lens = np.minimum(a_lens, K)
    arp = np.concatenate([[0], np.cumsum(a_lens)]).astype(np.int32)
    aci = np.concatenate([np.sort(rng.choice(K, int(n), replace=False)) for n in a_lens if n] or
                         [np.zeros(0, np.int64)]).astype(np.int32)
    av = draw_dense(rng, aci.size, dtype)
    brp, bci, bv = random_csr(rng, K, N, float(rng.choice([0.002, 0.01, 0.05])), dtype=dtype)
    rp, ci, v = hip_spgemm(arp, aci, av, brp, bci, bv, N)
    wrp, wci, wv = oracle.spgemm_csr_typed(arp, aci, av, brp, bci, bv, N)
    assert np.array_equal(rp, wrp) and np.array_equal(ci, wci)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(v, wv)
    else:
        _, _, ref64 = oracle.spgemm_csr_typed(arp, aci, av.astype(np.float64), brp, bci, bv.astype(np.float64), N)
        assert oracle.rel_fro(v, ref64) <= (1e-5 if dtype == np.float32 else 1e-13)


def _rows_of(rng, rows, cols, lens, clustered):
    """Sorted distinct column indices for rows of the given lengths; clustered rows draw theirs
    from a window twice their length."""
    out = []
    for n in lens:
        n = int(min(n, cols))
        if clustered and n and rng.random() < 0.5:
            span = min(cols, 2 * n)
            start = int(rng.integers(0, cols - span + 1))
            out.append(start + np.sort(rng.choice(span, n, replace=False)))
        else:
            out.append(np.sort(rng.choice(cols, n, replace=False)))
    row_ptr = np.concatenate([[0], np.cumsum([c.size for c in out])]).astype(np.int32)
    return row_ptr, np.concatenate(out or [np.zeros(0, np.int64)]).astype(np.int32)


@pytest.mark.parametrize("seed", range(32))
def test_spgemm_random_across_the_tiers(oracle, seed):
    """Operands drawn so that result rows land in every tier (a few entries to tens of
    thousands), B from 100 to 1,048,576 columns wide (sums by column, LDS bitmap in one or more
    ranges, hash tables), columns spread or clustered, mostly short rows with a few heavy ones."""
    rng = np.random.default_rng(1000 + seed)
    dtype = DTYPES[seed % 4]
    M = int(rng.choice([3, 50, 700, 5000, 40000]))
    K = int(rng.choice([40, 900, 6000]))
    N = int(rng.choice([100, 3000, 20000, 140000, 600000, 1 << 20]))
    a_lens = rng.integers(0, 6, M)
    if rng.random() < 0.6:
        heavy = rng.choice(M, min(M, 6), replace=False)
        a_lens[heavy] = rng.integers(10, min(K, 400) + 1, heavy.size)
    b_lens = rng.integers(0, 2 * int(rng.choice([2, 20, 120])) + 1, K)
    arp, aci = _rows_of(rng, M, K, a_lens, False)
    brp, bci = _rows_of(rng, K, N, b_lens, rng.random() < 0.4)
    av, bv = draw_dense(rng, aci.size, dtype), draw_dense(rng, bci.size, dtype)
    rp, ci, v = hip_spgemm(arp, aci, av, brp, bci, bv, N)
    wrp, wci, wv = oracle.spgemm_csr_typed(arp, aci, av, brp, bci, bv, N)
    assert np.array_equal(rp, wrp) and np.array_equal(ci, wci), (M, K, N)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(v, wv)
    else:
        _, _, ref64 = oracle.spgemm_csr_typed(arp, aci, av.astype(np.float64), brp, bci, bv.astype(np.float64), N)
        assert oracle.rel_fro(v, ref64) <= (1e-5 if dtype == np.float32 else 1e-13)


@pytest.mark.parametrize("seed", range(8))
def test_coordinate_products_random(oracle, seed):
    """spmm_coo_float and spmspm_coo_float on shuffled, partly repeated coordinates."""
    import torch
    from gpu_util import dev, host
    from scorch_amd import scorch_ops_hip as H
    rng = np.random.default_rng(5000 + seed)
    M, K, N = int(rng.integers(1, 300)), int(rng.integers(1, 300)), int(rng.integers(1, 200))
    arp, aci, av = random_csr(rng, M, K, draw_density(rng, K))
    ar = np.repeat(np.arange(M, dtype=np.int32), np.diff(arp))
    if seed % 2:  # any order, some entries twice
        pick = np.concatenate([rng.permutation(ar.size), rng.integers(0, max(ar.size, 1), ar.size // 3)]) \
            if ar.size else np.zeros(0, np.int64)
        ar, aci, av = ar[pick], aci[pick], av[pick]
    B = draw_dense(rng, (K, N), np.float32)
    got = host(H.spmm_coo_float([M, N], [M, K], [[dev(ar)], [dev(aci)]], dev(av), [K, N], [[], []],
                                dev(B).reshape(-1)).storage.value).reshape(M, N)
    dense_a = np.zeros((M, K))
    np.add.at(dense_a, (ar, aci), av.astype(np.float64))
    ref = dense_a @ B.astype(np.float64)
    assert oracle.rel_fro(got, ref) <= 1e-5
    brp, bci, bv = random_csr(rng, K, N, draw_density(rng, N))
    br = np.repeat(np.arange(K, dtype=np.int32), np.diff(brp))
    shuffle = rng.permutation(br.size)
    out = H.spmspm_coo_float([M, N], [M, K], [[dev(ar)], [dev(aci)]], dev(av), [K, N],
                             [[dev(br[shuffle])], [dev(bci[shuffle])]], dev(bv[shuffle]))
    r, c = (host(level[0]) for level in out.storage.index.mode_indices)
    dense_b = np.zeros((K, N))
    dense_b[br, bci] = bv
    full = dense_a @ dense_b
    structure = (np.abs(dense_a) > 0).astype(np.float64) @ (np.abs(dense_b) > 0)
    wr, wc = np.nonzero(structure)                                # every structural entry, row-major
    assert np.array_equal(r, wr.astype(np.int32)) and np.array_equal(c, wc.astype(np.int32))
    assert oracle.rel_fro(host(out.storage.value), full[wr, wc]) <= 1e-5


@pytest.mark.parametrize("seed", range(16))
def test_softmax_random(oracle, seed):
    """Row lengths from a heavy-tailed draw (so that every tier of the kernel and
    the giant-row kernel meet rows), empty rows included, scale of either sign."""
    from gpu_util import dev, host
    from scorch_amd import scorch_ops_hip as H
    rng = np.random.default_rng(5000 + seed)
    M = int(rng.integers(1, 3000))
    lens = np.minimum(rng.zipf(1.6, size=M) - 1, int(rng.choice([40, 300, 3000, 12000]))).astype(np.int64)
    lens[rng.random(M) < 0.1] = 0
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    vals = (rng.standard_normal(int(rp[-1])) * float(rng.choice([0.1, 3.0, 30.0]))).astype(np.float32)
    scale = float(rng.choice([1.0, 0.125, -0.5]))
    got = host(H.softmax_csr_float(dev(rp), dev(vals), scale))
    want = oracle.softmax_csr_fp64(rp, vals, scale)
    assert got.shape == want.shape
    if want.size:
        np.testing.assert_allclose(got, want, rtol=3e-5, atol=1e-10)


@pytest.mark.parametrize("seed", range(12))
def test_attention_random_block_patterns(oracle, seed):
    """Random block masks (some block rows empty, some full), head counts that are
    and are not multiples of eight, sequence lengths from one block up."""
    import torch
    from gpu_util import dev
    from scorch_amd import scorch_ops_hip as H
    rng = np.random.default_rng(6000 + seed)
    nb = int(rng.choice([1, 2, 5, 9, 16]))
    heads = int(rng.choice([1, 3, 8, 16]))
    S = 64 * nb
    active = rng.random((nb, nb)) < float(rng.choice([0.15, 0.5, 1.0]))
    if nb > 2:
        active[int(rng.integers(nb)), :] = False
        active[int(rng.integers(nb)), :] = True
    r, c = np.nonzero(active)
    brp = np.concatenate([[0], np.cumsum(np.bincount(r, minlength=nb))]).astype(np.int32)
    bci = c.astype(np.int32)
    q, k, v = (torch.from_numpy((rng.standard_normal((heads, S, 64)) * float(rng.choice([0.3, 1.0, 3.0])))
                                .astype(np.float32)).to(torch.bfloat16) for _ in range(3))
    scale = float(rng.choice([0.125, 0.05, -0.125]))
    out = H.attn_blocksparse_bf16(q.cuda(), k.cuda(), v.cuda(), dev(brp), dev(bci), scale).float().cpu().numpy()
    ref = oracle.attention_blocksparse_fp64(q.float().numpy(), k.float().numpy(), v.float().numpy(),
                                            brp, bci, 64, scale)
    assert np.isfinite(out).all()
    empty_rows = np.nonzero(np.diff(brp) == 0)[0]
    for b in empty_rows:
        assert not out[:, 64 * b:64 * (b + 1)].any()
    if np.linalg.norm(ref) > 0:
        assert oracle.rel_fro(out, ref) <= 1e-2
