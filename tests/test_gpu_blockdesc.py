"""The block description of a CSR pattern as the device kernels build it
(scorch_hip_csr_block_count, scorch_hip_csr_block_fill, the extra fields of scorch_hip_csr_inspect):
bit for bit against a second construction with torch operations (tests/blockdesc_reference.py) and
against a direct reading of the dense mask."""
import numpy as np
import pytest
import torch

from blockdesc_reference import describe
from gpu_util import dev, host
from scorch_amd import native, workloads
from scorch_amd import scorch_ops_hip as H
from test_gpu_blocked import csr_of, pattern

pytestmark = pytest.mark.gpu

KINDS = ["blocks", "window", "causal", "window_global", "random30", "random2"]


def _inspect(rp, ci, n_cols):
    report = torch.full((H.INSPECT_REPORT_INTS,), -7, dtype=torch.int32, device="cuda")
    native.check(native.lib().scorch_hip_csr_inspect(rp.numel() - 1, n_cols, ci.numel(), rp.data_ptr(), ci.data_ptr(),
                                                     report.data_ptr(), torch.cuda.current_stream().cuda_stream))
    return report.tolist()


def _runs(rp, ci):
    """Maximal stretches of a row's entries that increase and lie in one aligned group of 64 columns."""
    runs = descents = 0
    for r in range(len(rp) - 1):
        row = ci[rp[r]:rp[r + 1]].astype(np.int64)
        if row.size:
            down = row[1:] <= row[:-1]
            descents += int(down.sum())
            runs += 1 + int((down | (row[1:] // 64 != row[:-1] // 64)).sum())
    return descents, runs


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("shape", [(256, 256), (192, 448), (1024, 1024)])
def test_description_equals_the_construction_by_torch_operations(kind, shape):
    rng = np.random.default_rng(100 * KINDS.index(kind) + shape[1])
    M, n_cols = shape
    rp, ci = csr_of(pattern(kind, M, n_cols, rng))
    pos, crd = dev(rp), dev(ci)
    report = _inspect(pos, crd, n_cols)
    assert report[:2] == [0, 0] and report[4:6] == list(_runs(rp, ci)) and report[6:] == [0, 0]
    brp, arrays = H._describe_blocks(pos, crd, M, n_cols)
    want = describe(pos, crd, M, n_cols)
    assert np.array_equal(brp, host(want["block_row_ptr"]))
    for name, expected in want.items():
        assert arrays[name].dtype == expected.dtype and torch.equal(arrays[name], expected), name
    # the run count bounds the blocks' fill from above
    n_active = int(brp[-1])
    assert ci.size / (64 * report[5]) >= ci.size / (4096 * n_active) - 1e-12


@pytest.mark.parametrize("n_block_cols", [257, 5000, 131_072])
def test_description_of_a_very_wide_pattern(n_block_cols):
    """More block columns than a workgroup has threads (the bitmap and its ranks are walked in
    strides and stretches), up to the most the kernels take: rows of a few hundred entries spread
    over the whole width, some clustered so that blocks hold more than one entry."""
    rng = np.random.default_rng(n_block_cols)
    M, n_cols = 128, 64 * n_block_cols
    rows = []
    for r in range(M):
        spread = rng.choice(n_cols, int(rng.integers(0, 300)), replace=False)
        home = 64 * int(rng.integers(0, n_block_cols))
        cluster = home + rng.choice(64, int(rng.integers(0, 40)), replace=False)
        rows.append(np.unique(np.concatenate([spread, cluster, [n_cols - 1] if r % 7 == 0 else []]).astype(np.int64)))
    rp = np.concatenate([[0], np.cumsum([len(x) for x in rows])]).astype(np.int32)
    ci = np.concatenate(rows).astype(np.int32)
    pos, crd = dev(rp), dev(ci)
    assert _inspect(pos, crd, n_cols)[:2] == [0, 0]
    brp, arrays = H._describe_blocks(pos, crd, M, n_cols)
    want = describe(pos, crd, M, n_cols)
    assert np.array_equal(brp, host(want["block_row_ptr"]))
    for name, expected in want.items():
        assert torch.equal(arrays[name], expected), name
    L = native.lib()
    too_wide = torch.zeros(3, dtype=torch.int32, device="cuda")
    assert L.scorch_hip_csr_block_count(64, 64 * (131_072 + 1), 0, too_wide.data_ptr(), None, too_wide.data_ptr(),
                                        None) == native.EUNSUPPORTED


def test_description_read_directly_from_the_mask():
    """Every stored entry is found at block_off + (stored columns below it); the work-item lists
    cover what they must; what the description is not built for is turned away."""
    rng = np.random.default_rng(0)
    M, n_cols = 192, 320
    mask = rng.random((M, n_cols)) < 0.3
    mask[64:128] = False                                          # a block row without blocks
    mask[:, 128:192] = False                                      # a block column without blocks
    mask[130, :] = False                                          # an empty row inside an active block row
    rp, ci = csr_of(mask)
    pos, crd = dev(rp), dev(ci)
    plan = H.csr_plan(pos, crd, M, n_cols)
    assert plan.sorted_rows and plan.runs == _runs(rp, ci)[1]
    bl = H._blocked_csr(plan, pos, crd, M, n_cols, 0.1)
    assert bl is not None and bl.n_block_rows == 3 and abs(bl.fill - ci.size / (bl.n_active * 4096)) < 1e-12
    cols = bl.block_col_idx.tolist()
    words = host(bl.block_words).reshape(-1, 64).view(np.uint64)
    offs = host(bl.block_off).reshape(-1, 64)
    stored_per_block = host(bl.block_nnz)
    spmm_items = sorted(bl.spmm_items.view(-1, 4).tolist())
    assert [it[0] for it in spmm_items] == [0, 1, 2] and spmm_items[1][1] == spmm_items[1][2]
    used = host(bl.block_cols).view(np.uint64)
    seen = np.zeros(ci.size, dtype=bool)
    for row_block, lo, hi, _ in spmm_items:
        assert cols[lo:hi] == sorted(cols[lo:hi]) and 2 not in cols[lo:hi]
        for b in range(lo, hi):
            block = mask[64 * row_block:64 * row_block + 64, 64 * cols[b]:64 * cols[b] + 64]
            assert int(used[b]) == sum(1 << c for c in range(64) if block[:, c].any())
            assert int(stored_per_block[b]) == int(block.sum())
            for r in range(64):
                row = 64 * row_block + r
                stored = [c for c in range(64) if mask[row, 64 * cols[b] + c]]
                assert int(words[b, r]) == sum(1 << c for c in stored)
                for rank, c in enumerate(stored):
                    at = offs[b, r] + rank
                    assert rp[row] <= at < rp[row + 1] and ci[at] == 64 * cols[b] + c and not seen[at]
                    seen[at] = True
    assert seen.all()
    for stretch, (items, n_items) in bl.sddmm_items.items():
        covered = sorted((lo, hi) for _, lo, hi, _ in items.view(-1, 4).tolist())
        assert len(covered) == n_items and covered[0][0] == 0 and covered[-1][1] == bl.n_active
        assert all(a[1] == b[0] for a, b in zip(covered, covered[1:])) and all(hi - lo <= stretch for lo, hi in covered)
    assert set(bl.sddmm_items) == set(H.BLOCKED_STRETCHES) and bl.sddmm_items[1][1] == bl.n_active
    # what the description is not built for
    assert H._blocked_csr(plan, pos, crd, M, n_cols, 0.5) is None                       # too thinly filled
    short_pos, short_crd = dev(rp[:-1]), dev(ci[:rp[-2]])
    assert H._blocked_csr(H.csr_plan(short_pos, short_crd, M - 1, n_cols), short_pos, short_crd, M - 1, n_cols,
                          0.0) is None
    backwards = ci.copy()
    backwards[rp[3]:rp[4]] = backwards[rp[3]:rp[4]][::-1]
    back = dev(backwards)
    unsorted = H.csr_plan(pos, back, M, n_cols)
    assert not unsorted.sorted_rows and H._blocked_csr(unsorted, pos, back, M, n_cols, 0.0) is None


def test_a_graph_is_turned_away_by_the_inspection_alone():
    """Operands that are not masks made of blocks -- a graph with power-law degrees, a band -- are
    told apart by the run count of their inspection: no kernel of the description runs, and the
    second product with them costs what the first did."""
    w = workloads.gcn_powerlaw(M=8192, N=64, seed=3, max_degree=2000)
    pos, crd = dev(w["row_ptr"]), dev(w["col_idx"])
    plan = H.csr_plan(pos, crd, 8192, 8192)
    assert plan.sorted_rows and crd.numel() < min(H.BLOCKED_MIN_FILL.values()) * 64 * plan.runs
    called = []
    original = H._describe_blocks
    H._describe_blocks = lambda *a, **k: called.append(a) or original(*a, **k)
    try:
        assert H._blocked_csr(plan, pos, crd, 8192, 8192, min(H.BLOCKED_MIN_FILL.values())) is None
        # a band of 9: rows of consecutive columns, one run each, but a 64 x 64 block holds 9 of 64 per row at best
        M = 4096
        i = np.arange(M)[:, None] + np.arange(-4, 5)[None, :]
        keep = (i >= 0) & (i < M)
        rp = np.concatenate([[0], np.cumsum(keep.sum(1))]).astype(np.int32)
        band_pos, band_crd = dev(rp), dev(i[keep].astype(np.int32))
        band = H.csr_plan(band_pos, band_crd, M, M)
        assert H._blocked_csr(band, band_pos, band_crd, M, M, min(H.BLOCKED_MIN_FILL.values())) is None
    finally:
        H._describe_blocks = original
    assert len(called) <= 1          # the band's runs are long enough to ask for the count pass; the graph's are not


def _mask_of(bm):
    """The dense mask a BlockMask stands for."""
    brp, bci, bmi = (host(t) for t in (bm.block_row_ptr, bm.block_col_idx, bm.block_mask_index))
    words = host(bm.block_masks).view(np.uint64).reshape(-1, 64)
    out = np.zeros((bm.S, bm.S), bool)
    for br in range(bm.S // 64):
        for i in range(brp[br], brp[br + 1]):
            bits = (np.ones((64, 64), bool) if bmi[i] < 0 else
                    ((words[bmi[i]][:, None] >> np.arange(64, dtype=np.uint64)[None, :]) & np.uint64(1)).astype(bool))
            out[64 * br:64 * br + 64, 64 * bci[i]:64 * bci[i] + 64] = bits
    return out


def test_block_mask_from_csr_round_trips_and_shares_equal_masks():
    rng = np.random.default_rng(40)
    S = 320
    mask = rng.random((S, S)) < 0.03
    mask[0:64, 64:128] = True                      # a full block
    mask[128:192, :] = False                       # an empty block row
    mask[64:128, 0:64] = np.tri(64, dtype=bool)    # two equal partial blocks
    mask[256:320, 192:256] = np.tri(64, dtype=bool)
    mask[100, 319] = True                          # bit 63 of a word
    rp, ci = csr_of(mask)
    bm = H.block_mask_from_csr(dev(rp), dev(ci), S)
    assert np.array_equal(_mask_of(bm), mask) and bm.nnz == int(mask.sum())
    brp, bci, bmi = (host(t) for t in (bm.block_row_ptr, bm.block_col_idx, bm.block_mask_index))
    at = {(br, int(bci[i])): int(bmi[i]) for br in range(5) for i in range(brp[br], brp[br + 1])}
    assert at[(0, 1)] == -1 and at[(1, 0)] == at[(4, 3)] >= 0 and brp[3] == brp[2]
    assert bm.n_masks < bm.n_active_blocks
    # repeated entries and columns out of order are tolerated
    rp2 = dev(np.array([0, 4] + [4] * 63, np.int32))
    bm2 = H.block_mask_from_csr(rp2, dev(np.array([7, 5, 5, 63], np.int32)), 64)
    assert bm2.nnz == 3 and (int(bm2.block_masks[0]) & 0xFFFFFFFFFFFFFFFF) == (1 << 5) | (1 << 7) | (1 << 63)
    with pytest.raises(ValueError):
        H.block_mask_from_csr(rp2, dev(np.array([5, 64, 7, 9], np.int32)), 64)
    with pytest.raises(ValueError):
        H.block_mask_from_csr(dev(rp), dev(ci), 100)
    # a mask without entries
    none = H.block_mask_from_csr(dev(np.zeros(129, np.int32)), dev(np.zeros(0, np.int32)), 128)
    assert none.n_active_blocks == 0 and none.nnz == 0 and host(none.block_row_ptr).tolist() == [0, 0, 0]


def test_longformer_mask_in_block_form():
    """The reference's Longformer pattern (window 64, one global token) at S = 4096: 314 active
    blocks, 6 distinct masks, and only the global token's block row is shared out."""
    rp, ci = workloads.longformer_mask(4096)
    bm = H.split_long_block_rows(H.block_mask_from_csr(dev(rp), dev(ci), 4096))
    assert (bm.n_active_blocks, bm.n_masks, bm.nnz) == (314, 6, 532286)
    assert bm.split_rows.tolist() == [0, 0, 7, 0] and bm.n_slots == 7
    items = host(bm.items).reshape(-1, 4)
    lengths = items[:, 2] - items[:, 1]
    assert (np.diff(lengths) <= 0).all() and lengths.max() <= 10          # longest first, none long
    covered = np.zeros(314, int)
    for _, lo, hi, _ in items:
        covered[lo:hi] += 1
    assert (covered == 1).all()
    assert sorted(items[items[:, 3] >= 0, 3].tolist()) == list(range(7))


def test_description_of_the_benchmark_attention_mask_at_full_size():
    """S = 8192 with the benchmark's block pattern (6.0 M entries): 1,466 fully stored blocks."""
    rp, ci = workloads.blocks_to_csr(*workloads.blocksparse_pattern(128), 64)
    pos, crd = dev(rp), dev(ci)
    brp, arrays = H._describe_blocks(pos, crd, 8192, 8192)
    assert int(brp[-1]) == 1466 and ci.size == 6_004_736
    assert bool((arrays["block_nnz"] == 4096).all()) and bool((arrays["block_words"] == -1).all())
    want = describe(pos, crd, 8192, 8192)
    for name, expected in want.items():
        assert torch.equal(arrays[name], expected), name
