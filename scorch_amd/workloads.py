"""Seeded synthetic inputs for the five benchmark workloads.

All generators use ``numpy.random.Generator(PCG64(seed))`` so that the same
seed gives the same arrays on every host; index arrays are int32, sorted and
unique within a row.  The shapes and distributions follow the workloads the
reference's application benchmarks run (GCN normalisation:
bench/bench_gcn.py:233-268; sparse attention: bench/bench_sparse_transformer.py:
304-382; weight-sparse autoencoder: bench/bench_sparse_autoencoder.py:250-276),
scaled to the sizes this project measures.  Every generator takes its sizes as
arguments so that tests can run the same distribution at a small size.
"""
from __future__ import annotations

from typing import Dict

import numpy as np

SEEDS = {"spmm_uniform": 1001, "gcn_powerlaw": 1002, "sddmm_uniform": 1003,
         "attention_blocksparse": 1004, "sae_decoder": 1005}


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def csr_from_sorted_rows(rows: np.ndarray, n_rows: int) -> np.ndarray:
    """Row pointer (int32, n_rows + 1) for a row-sorted coordinate list."""
    counts = np.bincount(rows, minlength=n_rows)
    row_ptr = np.zeros(n_rows + 1, dtype=np.int64)
    np.cumsum(counts, out=row_ptr[1:])
    if row_ptr[-1] >= 2 ** 31:
        raise ValueError("nnz does not fit the int32 row pointer")
    return row_ptr.astype(np.int32)


def _dedupe_sorted(rows: np.ndarray, cols: np.ndarray, n_cols: int):
    """Sort (row, col) pairs and drop duplicates."""
    key = rows.astype(np.int64) * np.int64(n_cols) + cols.astype(np.int64)
    key = np.unique(key)
    return (key // n_cols).astype(np.int32), (key % n_cols).astype(np.int32)


def spmm_uniform(M: int = 4096, K: int = 4096, N: int = 64, density: float = 0.01,
                 seed: int = SEEDS["spmm_uniform"]) -> Dict[str, np.ndarray]:
    """Uniform-random CSR A (each entry present with probability ``density``,
    values U(-1, 1)) and dense B ~ N(0, 1)."""
    rng = _rng(seed)
    lengths = rng.binomial(K, density, size=M)
    rows = np.repeat(np.arange(M, dtype=np.int32), lengths)
    cols = rng.integers(0, K, size=rows.size, dtype=np.int64).astype(np.int32)
    rows, cols = _dedupe_sorted(rows, cols, K)
    vals = rng.uniform(-1.0, 1.0, size=rows.size).astype(np.float32)
    B = rng.standard_normal((K, N), dtype=np.float32)
    return {"M": M, "K": K, "N": N, "row_ptr": csr_from_sorted_rows(rows, M),
            "col_idx": cols, "vals": vals, "B": B}


def _degrees_with_mean(z: np.ndarray, mean_degree: float, cap: int, rng: np.random.Generator) -> np.ndarray:
    """Integer degrees proportional to ``z``, capped at ``cap``, whose mean after
    the cap is ``mean_degree``: the scale factor is found by bisection on the mean
    of the capped values, then rounded stochastically (floor(x + u), u ~ U[0, 1))."""
    if cap <= 0 or z.size == 0:
        return np.zeros(z.size, dtype=np.int64)
    target = min(mean_degree, float(cap))
    lo, hi = 0.0, 1.0
    while np.minimum(z * hi, cap).mean() < target and hi < 1e12:
        hi *= 2.0
    for _ in range(60):
        mid = 0.5 * (lo + hi)
        if np.minimum(z * mid, cap).mean() < target:
            lo = mid
        else:
            hi = mid
    scaled = np.minimum(z * hi, cap)
    return np.clip(np.floor(scaled + rng.random(z.size)).astype(np.int64), 0, cap)


def _distinct_neighbours(deg: np.ndarray, M: int, window: int, rng: np.random.Generator):
    """``deg[i]`` distinct neighbours for node i, uniform over the nodes (or over
    the ``window`` nodes around i): draw, drop repeats, and top up the rows that
    lost entries until none is short.  Returns row-sorted (rows, cols), int32."""
    def draw(rows):
        cols = rng.integers(0, M, size=rows.size, dtype=np.int64)
        if window > 0:
            cols = (rows.astype(np.int64) + cols % window - window // 2) % M
        return cols.astype(np.int32)

    rows = np.repeat(np.arange(M, dtype=np.int32), deg)
    rows, cols = _dedupe_sorted(rows, draw(rows), M)
    for _ in range(200):
        have = np.bincount(rows, minlength=M)
        short = np.nonzero(have < deg)[0]
        if short.size == 0:
            break
        r_new = np.repeat(short.astype(np.int32), (deg[short] - have[short]).astype(np.int64))
        rows, cols = _dedupe_sorted(np.concatenate([rows, r_new]), np.concatenate([cols, draw(r_new)]), M)
    return rows, cols


def gcn_powerlaw(M: int = 1 << 20, N: int = 128, seed: int = SEEDS["gcn_powerlaw"],
                 zipf_a: float = 2.1, mean_degree: float = 16.0,
                 max_degree: int = 50_000, window: int = 0) -> Dict[str, np.ndarray]:
    """Power-law graph with the GCN normalisation D^-1/2 (A + I) D^-1/2.

    Out-degrees are Zipf(``zipf_a``) draws capped at ``max_degree``, rescaled so
    that their mean *after* the cap is ``mean_degree`` (stochastic rounding);
    every node gets that many distinct neighbours, uniform over the nodes (drawn
    without replacement); a self-loop is added to every node that lacks one;
    ``deg`` is the row length of A + I and each entry is
    ``deg[row]^-1/2 * deg[col]^-1/2`` (the edge weight of
    bench/bench_gcn.py:248-258).  Features are N(0, 1).  At the default size:
    17,825,865 entries with the default seed (16 per node + the self-loops).

    ``window`` > 0 draws a node's neighbours from the ``window`` nodes around it
    (wrapping at the ends) instead of from all nodes, at most ``window`` of them:
    rows that lie close together then share neighbours.
    """
    rng = _rng(seed)
    cap = min(max_degree, M - 1) if M > 1 else 0
    if window > 0:
        cap = min(cap, window - 1)
    z = np.minimum(rng.zipf(zipf_a, size=M), max(cap, 1)).astype(np.float64)
    deg = _degrees_with_mean(z, mean_degree, cap, rng)
    rows, cols = _distinct_neighbours(deg, M, window, rng)
    loops = np.arange(M, dtype=np.int32)
    rows, cols = _dedupe_sorted(np.concatenate([rows, loops]), np.concatenate([cols, loops]), M)
    row_ptr = csr_from_sorted_rows(rows, M)
    d = np.diff(row_ptr).astype(np.float32)
    inv_sqrt = (1.0 / np.sqrt(d)).astype(np.float32)
    vals = (inv_sqrt[rows] * inv_sqrt[cols]).astype(np.float32)
    X = rng.standard_normal((M, N), dtype=np.float32)
    return {"M": M, "K": M, "N": N, "row_ptr": row_ptr, "col_idx": cols,
            "vals": vals, "B": X}


def sddmm_uniform(M: int = 65_536, n_cols: int = 65_536, per_row: int = 64, K: int = 64,
                  seed: int = SEEDS["sddmm_uniform"],
                  unit_mask: bool = True) -> Dict[str, np.ndarray]:
    """CSR mask with ``per_row`` distinct uniform columns in every row, dense A
    (M x K) and B (n_cols x K) ~ N(0, 1/8).  Mask values are 1 (``unit_mask``)
    or U(-1, 1)."""
    rng = _rng(seed)
    per_row = min(per_row, n_cols)
    # distinct columns per row: draw, dedupe, and top up rows that lost entries
    rows = np.repeat(np.arange(M, dtype=np.int32), per_row)
    cols = rng.integers(0, n_cols, size=rows.size, dtype=np.int64).astype(np.int32)
    rows, cols = _dedupe_sorted(rows, cols, n_cols)
    for _ in range(64):
        have = np.bincount(rows, minlength=M)
        short = np.nonzero(have < per_row)[0]
        if short.size == 0:
            break
        need = (per_row - have[short]).astype(np.int64)
        r_new = np.repeat(short.astype(np.int32), need)
        c_new = rng.integers(0, n_cols, size=r_new.size, dtype=np.int64).astype(np.int32)
        rows, cols = _dedupe_sorted(np.concatenate([rows, r_new]),
                                    np.concatenate([cols, c_new]), n_cols)
    row_ptr = csr_from_sorted_rows(rows, M)
    if unit_mask:
        vals = np.ones(rows.size, dtype=np.float32)
    else:
        vals = rng.uniform(-1.0, 1.0, size=rows.size).astype(np.float32)
    sigma = np.float32(np.sqrt(1.0 / 8.0))
    A = rng.standard_normal((M, K), dtype=np.float32) * sigma
    B = rng.standard_normal((n_cols, K), dtype=np.float32) * sigma
    return {"M": M, "n_cols": n_cols, "K": K, "row_ptr": row_ptr, "col_idx": cols,
            "row_idx": rows, "vals": vals, "A": A, "B": B}


def blocksparse_pattern(n_blocks: int, window: int = 4, stride: int = 8):
    """Block pattern of the sparse-transformer workload: block (bi, bj) is
    active iff bj <= bi and (bi - bj < window or (bi - bj) % stride == 0).
    Returns the block-CSR arrays (block_row_ptr, block_col_idx), int32."""
    bi = np.arange(n_blocks)[:, None]
    bj = np.arange(n_blocks)[None, :]
    active = (bj <= bi) & (((bi - bj) < window) | (((bi - bj) % stride) == 0))
    r, c = np.nonzero(active)
    return csr_from_sorted_rows(r.astype(np.int32), n_blocks), c.astype(np.int32)


def attention_blocksparse(S: int = 8192, H: int = 16, D: int = 64, block: int = 64,
                          seed: int = SEEDS["attention_blocksparse"],
                          window: int = 4, stride: int = 8) -> Dict[str, np.ndarray]:
    """Q, K, V ~ N(0, 1) of shape (H, S, D) in fp32 (the caller rounds to bf16)
    and the block mask shared by all heads.  Every entry of an active
    ``block`` x ``block`` tile is live (no triangle inside a tile)."""
    if S % block:
        raise ValueError("sequence length must be a multiple of the block size")
    rng = _rng(seed)
    q = rng.standard_normal((H, S, D), dtype=np.float32)
    k = rng.standard_normal((H, S, D), dtype=np.float32)
    v = rng.standard_normal((H, S, D), dtype=np.float32)
    brp, bci = blocksparse_pattern(S // block, window, stride)
    return {"S": S, "H": H, "D": D, "block": block, "q": q, "k": k, "v": v,
            "block_row_ptr": brp, "block_col_idx": bci,
            "scale": np.float32(1.0 / np.sqrt(D))}


def blocks_to_csr(block_row_ptr: np.ndarray, block_col_idx: np.ndarray, block: int):
    """Expand a block pattern to an element CSR pattern (row_ptr, col_idx)."""
    nb = block_row_ptr.size - 1
    counts = np.repeat(np.diff(block_row_ptr).astype(np.int64) * block, block)
    row_ptr = np.zeros(nb * block + 1, dtype=np.int64)
    np.cumsum(counts, out=row_ptr[1:])
    cols = []
    lane = np.arange(block, dtype=np.int32)
    for b in range(nb):
        bc = block_col_idx[block_row_ptr[b]:block_row_ptr[b + 1]].astype(np.int32)
        row_cols = (bc[:, None] * block + lane[None, :]).reshape(-1)
        cols.append(np.tile(row_cols, block))
    col_idx = np.concatenate(cols) if cols else np.zeros(0, np.int32)
    return row_ptr.astype(np.int32), col_idx.astype(np.int32)


def longformer_mask(S: int, window: int = 64, n_global: int = 1):
    """CSR pattern (row_ptr, col_idx; int32) of the Longformer-style attention mask of the
    reference's sparse-transformer benchmark (bench/bench_sparse_transformer.py:194-209): token
    i attends to the tokens within ``window`` positions on either side, and the first
    ``n_global`` tokens attend to and are attended by every token.  With the benchmark's
    settings (window 64, one global token) the mask has 62,782 entries at S = 512 and 532,286
    at S = 4096 (bench/README_sparse_transformer.md:78-81)."""
    i = np.arange(S, dtype=np.int64)
    lo = np.maximum(i - window, 0)
    hi = np.minimum(i + window, S - 1) + 1                  # the window, [lo, hi)
    n_global = min(n_global, S)
    extra = np.minimum(lo, n_global)                         # global columns left of the window
    lens = (hi - lo) + extra
    lens[:n_global] = S
    row_ptr = np.zeros(S + 1, dtype=np.int64)
    np.cumsum(lens, out=row_ptr[1:])
    cols = np.empty(int(row_ptr[-1]), dtype=np.int32)
    for r in range(S):
        seg = cols[row_ptr[r]:row_ptr[r + 1]]
        if r < n_global:
            seg[:] = np.arange(S, dtype=np.int32)
        else:
            seg[:extra[r]] = np.arange(extra[r], dtype=np.int32)
            seg[extra[r]:] = np.arange(lo[r], hi[r], dtype=np.int32)
    return row_ptr.astype(np.int32), cols


def sae_decoder(M: int = 4096, K: int = 16_384, N: int = 4096, k: int = 32,
                seed: int = SEEDS["sae_decoder"]) -> Dict[str, np.ndarray]:
    """Sparse-autoencoder decoder input: per row the top ``k`` of ReLU(N(0, 1))
    over K latent units (values are those activations, indices sorted), and a
    dense decoder weight W (K x N) ~ N(0, 1/64)."""
    rng = _rng(seed)
    k = min(k, K)
    cols = np.empty((M, k), dtype=np.int32)
    vals = np.empty((M, k), dtype=np.float32)
    step = max(1, min(M, (1 << 24) // max(K, 1)))
    for r0 in range(0, M, step):
        r1 = min(M, r0 + step)
        pre = np.maximum(rng.standard_normal((r1 - r0, K), dtype=np.float32), 0.0)
        top = np.argpartition(pre, K - k, axis=1)[:, K - k:]
        top.sort(axis=1)
        cols[r0:r1] = top
        vals[r0:r1] = np.take_along_axis(pre, top, axis=1)
    row_ptr = (np.arange(M + 1, dtype=np.int64) * k).astype(np.int32)
    W = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.125)
    return {"M": M, "K": K, "N": N, "row_ptr": row_ptr, "col_idx": cols.reshape(-1),
            "vals": vals.reshape(-1), "B": W}
