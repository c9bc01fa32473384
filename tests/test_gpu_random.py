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
