"""Host-side logic that mirrors the reference's dispatch: format strings, the
tensor model, the prebuilt-kernel registry and the routing decisions of
matmul / einsum.  Mirrors tests/test_scorch/test_prebuilt_kernel_registry.py
and the format checks of the reference; runs without a GPU."""
import os

import numpy as np
import pytest
import torch

import scorch_amd as scorch
from scorch_amd import STensor, ops, parse_format, scorch_ops_hip
from scorch_amd.prebuilt_kernels import (execute_prebuilt_binary_kernel, resolve_prebuilt_fused,
                                         resolve_prebuilt_matmul)


def sparse_dense_pair(n=16, dtype=torch.float32, density=0.2, seed=0):
    g = torch.Generator().manual_seed(seed)
    a = torch.rand(n, n, generator=g, dtype=torch.float64) * (torch.rand(n, n, generator=g) < density)
    b = torch.rand(n, n, generator=g, dtype=torch.float64)
    if dtype in (torch.int32, torch.int64):
        a, b = (a * 10).round(), (b * 10).round()
    return a.to(dtype), b.to(dtype)


# ---- formats ------------------------------------------------------------------------
@pytest.mark.parametrize("spec,text", [("ds", "d,s"), ("dd", "d,d"), ("oo", "o,o"), ("d", "d"),
                                       (["dense", "compressed"], "d,s"), (["coord", "coordinate"], "o,o"),
                                       (["dense", "sparse"], "d,s"), (["d", "c"], "d,s")])
def test_parse_format_strings(spec, text):
    assert str(parse_format(spec)) == text


def test_parse_format_rejects_unknown_levels():
    with pytest.raises(ValueError):
        parse_format("dx")
    with pytest.raises(ValueError):
        parse_format(["dense", "singleton"])


def test_format_equality_and_density():
    assert parse_format("dd") == parse_format(["dense", "dense"])
    assert parse_format("ds") != parse_format("dd")
    assert parse_format("dd").is_dense() and not parse_format("ds").is_dense()
    assert parse_format(parse_format("oo")) is not None


# ---- tensor model -----------------------------------------------------------------------
def test_from_torch_dense_flattens_values():
    t = torch.arange(12, dtype=torch.float32).reshape(3, 4)
    s = STensor.from_torch(t)
    assert str(s.format) == "d,d" and s.shape == (3, 4) and s.dim() == 2
    assert s.index.mode_indices == [[], []]
    assert s.values.shape == (12,) and torch.equal(s.values, t.flatten())
    assert torch.equal(s.to_torch(), t)


def test_from_csr_shares_arrays_and_coerces_indices_to_int32():
    a, _ = sparse_dense_pair()
    csr = a.to_sparse_csr()
    assert csr.crow_indices().dtype == torch.int64
    s = STensor.from_csr(csr)
    pos, crd = s.index.mode_indices[1]
    assert str(s.format) == "d,s" and s.index.mode_indices[0] == []
    assert pos.dtype == torch.int32 and crd.dtype == torch.int32
    assert torch.equal(pos.long(), csr.crow_indices()) and torch.equal(crd.long(), csr.col_indices())
    assert s.values.data_ptr() == csr.values().data_ptr()
    assert s._nnz() == csr.values().numel()
    assert torch.equal(s.to_torch(), a)


def test_from_torch_sparse_layouts_and_from_coo():
    a, _ = sparse_dense_pair(seed=3)
    s_csr = scorch.from_torch(a.to_sparse_csr())
    s_coo = scorch.from_torch(a.to_sparse())
    assert str(s_csr.format) == "d,s" and str(s_coo.format) == "o,o"
    assert len(s_coo.index.mode_indices) == 2 and s_coo.index.mode_indices[0][0].dtype == torch.int32
    assert torch.equal(s_coo.to_torch(), a) and torch.equal(s_csr.to_torch(), a)
    raw = scorch.from_coo(indices=a.to_sparse().indices(), values=a.to_sparse().values(), shape=a.shape)
    assert torch.equal(raw.to_torch(), a)


def test_to_sparse_round_trips():
    a, _ = sparse_dense_pair(seed=4)
    d = STensor.from_torch(a)
    for fmt in ("ds", "oo"):
        s = d.to_sparse(fmt)
        assert str(s.format) == str(parse_format(fmt))
        assert torch.equal(s.to_torch(), a)
        assert torch.equal(s.to_dense().to_torch(), a)
    assert str(d.to_sparse("ds").to_sparse("oo").format) == "o,o"


def test_copy_is_deep_and_to_cpu_is_a_copy():
    a, _ = sparse_dense_pair(seed=5)
    s = STensor.from_torch(a).to_sparse("ds")
    c = s.copy()
    c.values.zero_()
    assert s.values.abs().sum() > 0
    assert s.to("cpu").index == s.index and not s.is_cuda


# ---- registry (reference: tests/test_scorch/test_prebuilt_kernel_registry.py) ---------------
@pytest.mark.parametrize("dtype,symbol", [(torch.float32, "spmm_csr_float_v2"),
                                          (torch.float64, "prebuilt_spmm_csr_f64"),
                                          (torch.int32, "prebuilt_spmm_csr_i32"),
                                          (torch.int64, "prebuilt_spmm_csr_i64")])
def test_resolve_prebuilt_spmm_symbol_per_dtype(dtype, symbol):
    a, b = sparse_dense_pair(dtype=dtype)
    resolved = resolve_prebuilt_matmul(STensor.from_torch(a).to_sparse("ds"), STensor.from_torch(b))
    assert resolved is not None and resolved.symbol_name == symbol
    assert str(resolved.output_format) == "d,d"
    assert resolved.fn is getattr(scorch_ops_hip, symbol)


def test_resolve_prebuilt_spmv_int64_symbol():
    a = torch.tensor([[1, 0, 2, 0], [0, 3, 0, 4], [0, 0, 0, 0], [5, 0, 0, 6]], dtype=torch.int64)
    x = torch.tensor([1, 2, 3, 4], dtype=torch.int64)
    resolved = resolve_prebuilt_matmul(STensor.from_torch(a).to_sparse("ds"), STensor.from_torch(x))
    assert resolved is not None and resolved.symbol_name == "prebuilt_spmv_csr_i64"
    assert str(resolved.output_format) == "d"


def test_resolve_prebuilt_gates():
    a, b = sparse_dense_pair()
    A, B = STensor.from_torch(a).to_sparse("ds"), STensor.from_torch(b)
    assert resolve_prebuilt_matmul(A, B, output_format="dd") is not None
    assert resolve_prebuilt_matmul(A, B, output_format="ds") is None          # requested format gate
    assert resolve_prebuilt_matmul(A, STensor.from_torch(b.double())) is None  # dtype equality gate
    assert resolve_prebuilt_matmul(B, B) is None                               # dense x dense: no entry
    assert resolve_prebuilt_matmul(A, STensor.from_torch(b.half())) is None
    # CSR x CSR produces CSR: a dense result cannot be requested from the prebuilt kernel
    # (reference: test_prebuilt_kernel_registry.py:41-51)
    assert resolve_prebuilt_matmul(A, A, output_format="dd") is None
    spgemm = resolve_prebuilt_matmul(A, A)
    assert spgemm.symbol_name == "prebuilt_spmspm_csr_f32" and str(spgemm.output_format) == "d,s"
    assert resolve_prebuilt_matmul(A, A, output_format="ds").symbol_name == "prebuilt_spmspm_csr_f32"
    # coordinate-format products, fp32 only (reference: prebuilt_kernels.py:64-79)
    coo = STensor.from_torch(a).to_sparse("oo")
    both = resolve_prebuilt_matmul(coo, coo)
    assert both.symbol_name == "spmspm_coo_float" and str(both.output_format) == "o,o"
    mixed = resolve_prebuilt_matmul(coo, B)
    assert mixed.symbol_name == "spmm_coo_float" and str(mixed.output_format) == "d,d"
    assert resolve_prebuilt_matmul(coo, coo, output_format="ds") is None
    coo64 = STensor.from_torch(a.double()).to_sparse("oo")
    assert resolve_prebuilt_matmul(coo64, coo64) is None


def test_resolve_prebuilt_fused():
    assert resolve_prebuilt_fused("d,s", "d,d", ("add", "relu"), torch.float32).symbol_name == \
        "spmm_csr_bias_relu_float"
    assert resolve_prebuilt_fused("d,s", "d,d", ("add",), torch.float32).symbol_name == "spmm_csr_bias_float"
    assert resolve_prebuilt_fused("d,s", "d,d", ("relu",), torch.float32) is None
    assert resolve_prebuilt_fused("d,s", "d,d", ("add",), torch.float64) is None
    assert resolve_prebuilt_fused("o,o", "d,d", ("add",), torch.float32) is None


def test_execute_prebuilt_packs_arguments_like_the_reference():
    a, b = sparse_dense_pair(n=8)
    A, B = STensor.from_torch(a).to_sparse("ds"), STensor.from_torch(b)
    seen = {}

    def fake_kernel(*args):
        seen["args"] = args
        return "result"

    td = {}
    result, shape = execute_prebuilt_binary_kernel(fake_kernel, A, B, time_dict=td)
    assert result == "result" and shape == (8, 8) and td["eval_time"] >= 0
    args = seen["args"]
    assert len(args) == 7 and args[0] == (8, 8) and args[1] == (8, 8) and args[4] == (8, 8)
    assert args[2] is A.index.mode_indices and args[3] is A.values and args[6] is B.values
    x = STensor.from_torch(b[:, 0].contiguous())
    _, shape = execute_prebuilt_binary_kernel(fake_kernel, A, x)
    assert shape == (8,)


# ---- routing ---------------------------------------------------------------------------------
def test_canonical_expression():
    assert ops._canonical("ik,kj->ij") == "ab,bc->ac" == ops._canonical("ij,jk->ik")
    assert ops._canonical("ij,ik,jk->ij") == ops._SDDMM_EXPR
    assert ops._canonical("ij,ik,kj->ij") == ops._SDDMM_EXPR_KJ


def test_dense_dense_matmul_uses_torch():
    _, b = sparse_dense_pair()
    assert torch.equal(scorch.matmul(b, b), torch.matmul(b, b))
    assert torch.equal(scorch.matmul(STensor.from_torch(b), STensor.from_torch(b)), torch.matmul(b, b))


def test_host_sparse_operands_are_refused_not_computed():
    a, b = sparse_dense_pair()
    A = STensor.from_torch(a).to_sparse("ds")
    with pytest.raises(RuntimeError, match="HIP devices only"):
        scorch.matmul(A, b)
    with pytest.raises(RuntimeError, match="HIP devices only"):
        scorch.matmul(A, b, use_cache=False)
    with pytest.raises(RuntimeError, match="HIP devices only"):
        scorch.einsum("ij,ik,jk->ij", A, b, b)
    with pytest.raises(RuntimeError, match="HIP devices only"):
        scorch.einsum("ij,ik,jk->ij", STensor.from_torch(a).to_sparse("oo"), b, b)


def test_expressions_outside_the_path_raise_not_implemented():
    a, b = sparse_dense_pair()
    A = STensor.from_torch(a).to_sparse("ds")
    with pytest.raises(RuntimeError, match="HIP devices only"):
        scorch.matmul(A, A)                      # CSR x CSR -> CSR has a kernel, on the device
    with pytest.raises(RuntimeError, match="HIP devices only"):
        scorch.matmul(A, A, format="dd")         # the same kernel, its result re-stored
    with pytest.raises(RuntimeError, match="HIP devices only"):
        scorch.matmul(A, b, format="ds")
    with pytest.raises(NotImplementedError):
        scorch.einsum("ij,ij->ij", A, A)
    with pytest.raises(NotImplementedError):
        scorch.matmul(A, STensor.from_torch(b.double()))   # operands of different types
    with pytest.raises(NotImplementedError):
        scorch.einsum("ijk,kl->ijl", STensor.from_torch(torch.rand(2, 3, 4)), A)
    with pytest.raises(NotImplementedError):
        scorch.einsum("ij,jk->ik", A, b, compile_only=True)
    with pytest.raises(NotImplementedError):
        scorch.spmm_bias_act(STensor.from_torch(a.double()).to_sparse("ds"), b.double(), b[0].double())


def test_device_module_rejects_host_and_mistyped_tensors():
    a, b = sparse_dense_pair(n=8)
    A, B = STensor.from_torch(a).to_sparse("ds"), STensor.from_torch(b)
    with pytest.raises(RuntimeError, match="HIP device"):
        scorch_ops_hip.spmm_csr_float_v2((8, 8), A.shape, A.index.mode_indices, A.values, B.shape,
                                         B.index.mode_indices, B.values)
    with pytest.raises(TypeError):
        scorch_ops_hip.spmm_csr_float_v2((8, 8), A.shape, A.index.mode_indices, A.values.double(),
                                         B.shape, B.index.mode_indices, B.values)
    with pytest.raises(ValueError, match="shape mismatch"):
        scorch_ops_hip.spmm_csr_float_v2((8, 9), A.shape, A.index.mode_indices, A.values, B.shape,
                                         B.index.mode_indices, B.values)
    with pytest.raises(ValueError, match="not a CSR"):
        scorch_ops_hip.spmm_csr_float_v2((8, 8), A.shape, [[], []], A.values, B.shape,
                                         B.index.mode_indices, B.values)


# ---- mode order (reference: src/scorch/stensor.py:785-896) -------------------------------------
@pytest.mark.parametrize("fmt", ["dd", "ds", "oo"])
def test_change_mode_order_transposes_storage(fmt):
    a, _ = sparse_dense_pair(n=12, seed=6)
    a = a[:, :9].contiguous()                                  # rectangular 12 x 9
    s = STensor.from_torch(a)
    s = s if fmt == "dd" else s.to_sparse(fmt)
    t = s.copy().change_mode_order([1, 0])
    assert t.shape == (9, 12) and t.index.mode_order == [1, 0] and str(t.format) == str(s.format)
    assert torch.equal(t.to_torch(), a)                         # logical tensor unchanged
    stored = STensor(shape=t.shape, index=type(t.index)(t.format, t.index.mode_indices), value=t.values)
    assert torch.equal(stored.to_torch(), a.t())                # physical storage is the transpose
    if fmt == "ds":
        pos, crd = t.index.mode_indices[1]
        assert pos.dtype == torch.int32 and pos[-1] == s._nnz()
        for r in range(9):
            seg = crd[pos[r]:pos[r + 1]]
            assert torch.all(seg[1:] > seg[:-1])                # sorted, unique
    back = t.change_mode_order([0, 1])
    assert back.shape == (12, 9) and torch.equal(back.to_torch(), a)
    assert back.change_mode_order([0, 1]) is back               # no-op when already there


def test_change_mode_order_sums_duplicate_coordinates():
    idx = torch.tensor([[0, 0, 1, 0], [2, 2, 0, 1]])
    vals = torch.tensor([1.0, 2.0, 5.0, 7.0])
    s = scorch.from_coo(indices=idx, values=vals, shape=(2, 3))
    t = s.change_mode_order([1, 0])
    assert t._nnz() == 3
    assert torch.equal(t.to_torch(), torch.tensor([[0.0, 7.0, 3.0], [5.0, 0.0, 0.0]]))


def test_change_mode_order_rejects_what_it_cannot_do():
    with pytest.raises(ValueError):
        STensor.from_torch(torch.rand(3, 3)).change_mode_order([0, 0])
    with pytest.raises(NotImplementedError):
        STensor.from_torch(torch.rand(2, 3, 4)).change_mode_order([2, 0, 1])


def test_check_csr_indices_names_what_is_wrong(monkeypatch):
    from scorch_amd.scorch_ops_hip import plans_enabled, tiled_operands_enabled
    from scorch_amd.utils import check_csr_indices
    pos = torch.tensor([0, 2, 2, 5], dtype=torch.int32)
    crd = torch.tensor([0, 3, 1, 2, 3], dtype=torch.int32)
    check_csr_indices(pos, crd, 4)                                   # well-formed: no exception
    with pytest.raises(ValueError, match=r"outside \[0, 3\)"):
        check_csr_indices(pos, crd, 3)
    with pytest.raises(ValueError, match="decreases"):
        check_csr_indices(torch.tensor([0, 3, 2, 5], dtype=torch.int32), crd, 4)
    with pytest.raises(ValueError, match=r"row_ptr\[-1\] = 4"):
        check_csr_indices(torch.tensor([0, 2, 2, 4], dtype=torch.int32), crd, 4)
    with pytest.raises(ValueError, match=r"row_ptr\[0\] = 1"):
        check_csr_indices(torch.tensor([1, 2, 2, 5], dtype=torch.int32), crd, 4)
    # operands are inspected (and planned) by default; both switches are opt-outs
    monkeypatch.delenv("SCORCH_HIP_PLAN", raising=False)
    monkeypatch.delenv("SCORCH_HIP_TILED", raising=False)
    assert plans_enabled() and tiled_operands_enabled()
    monkeypatch.setenv("SCORCH_HIP_PLAN", "0")
    monkeypatch.setenv("SCORCH_HIP_TILED", "0")
    assert not plans_enabled() and not tiled_operands_enabled()


# ---- the block form of an attention mask (torch ops, any device) ----

def _csr_of(mask):
    rp = np.concatenate([[0], np.cumsum(mask.sum(1))]).astype(np.int32)
    return torch.from_numpy(rp), torch.from_numpy(np.nonzero(mask)[1].astype(np.int32))


def _block_mask_of(active):
    """BlockMask of a mask made of whole 64 x 64 blocks, active[i, j] saying which."""
    nb = active.shape[0]
    brp = np.concatenate([[0], np.cumsum(active.sum(1))]).astype(np.int32)
    bci = np.nonzero(active)[1].astype(np.int32)
    return scorch_ops_hip.BlockMask(64 * nb, 64, torch.from_numpy(brp), torch.from_numpy(bci),
                                    torch.full((bci.size,), -1, dtype=torch.int32), torch.zeros(0, dtype=torch.int64),
                                    int(bci.size) * 4096)


def _mask_of(bm):
    """The dense mask a BlockMask stands for."""
    brp, bci, bmi = (t.numpy() for t in (bm.block_row_ptr, bm.block_col_idx, bm.block_mask_index))
    words = bm.block_masks.numpy().view(np.uint64).reshape(-1, 64)
    out = np.zeros((bm.S, bm.S), bool)
    for br in range(bm.S // 64):
        for i in range(brp[br], brp[br + 1]):
            bits = (np.ones((64, 64), bool) if bmi[i] < 0 else
                    ((words[bmi[i]][:, None] >> np.arange(64, dtype=np.uint64)[None, :]) & np.uint64(1)).astype(bool))
            out[64 * br:64 * br + 64, 64 * bci[i]:64 * bci[i] + 64] = bits
    return out


@pytest.mark.parametrize("longest", [1, 2, 5])
def test_split_long_block_rows_covers_every_block_once(longest):
    rng = np.random.default_rng(41 + longest)
    nb = 12
    active = rng.random((nb, nb)) < 0.5
    active[3, :] = True
    active[7, :] = False
    bm = scorch_ops_hip.split_long_block_rows(_block_mask_of(active), longest)
    items = bm.items.view(-1, 4).numpy()
    brp = bm.block_row_ptr.numpy()
    covered = np.zeros(bm.n_active_blocks, int)
    for row, lo, hi, slot in items:
        assert brp[row] <= lo <= hi <= brp[row + 1] and hi - lo <= longest
        assert lo < hi or brp[row] == brp[row + 1]       # only an empty block row has an empty item (it writes zeros)
        covered[lo:hi] += 1
        assert (slot >= 0) == (brp[row + 1] - brp[row] > longest)
    assert (covered == 1).all()
    for row, first, parts, _ in bm.split_rows.view(-1, 4).numpy():
        mine = items[items[:, 0] == row]
        assert sorted(mine[:, 3].tolist()) == list(range(first, first + parts))
    # a mask whose rows are all short enough is left alone
    bm = scorch_ops_hip.split_long_block_rows(_block_mask_of(active), nb)
    assert bm.items is None and bm.n_slots == 0


@pytest.mark.parametrize("longest,split", [(1, True), (3, True), (4, False), (16, True), (100, False)])
def test_work_items_by_array_operations_equal_the_plain_loops(longest, split):
    from blockdesc_reference import stretches
    rng = np.random.default_rng(longest)
    lens = rng.integers(0, 40, 57)
    lens[[3, 20]] = [0, 97]
    items, split_rows, n_slots = scorch_ops_hip._stretches(lens, longest, split)
    want_items, want_rows, want_slots = stretches(lens, longest, split)
    assert items.dtype == np.int32 and items.tolist() == [list(it) for it in want_items]
    assert split_rows.tolist() == [list(r) for r in want_rows] and n_slots == want_slots


def test_names_the_package_lacks_resolve_to_torch():
    """reference: src/scorch/__init__.py:14-18"""
    import scorch_amd as scorch
    assert scorch.float32 is torch.float32
    from scorch_amd import utils          # an own submodule wins over torch.utils
    assert utils.__name__ == "scorch_amd.utils"
    assert scorch.zeros(2, 3).shape == (2, 3)
    with pytest.raises(AttributeError, match="no_such_name"):
        scorch.no_such_name


def test_validate_accepts_well_formed_tensors_and_names_what_is_wrong():
    from scorch_amd import STensor
    dense = torch.tensor([[0.0, 2.0, 0.0], [1.0, 0.0, 3.0]])
    for fmt in ("dd", "ds", "oo"):
        t = STensor.from_torch(dense)
        (t if fmt == "dd" else t.to_sparse(fmt)).validate()
    i32 = lambda *v: torch.tensor(v, dtype=torch.int32)
    vals = torch.ones(3)
    STensor.from_csr_arrays(i32(0, 1, 3), i32(1, 0, 2), vals, (2, 3)).validate()
    with pytest.raises(ValueError, match="row pointers"):
        STensor.from_csr_arrays(i32(0, 2, 1), i32(1, 0, 2), vals, (2, 3)).validate()
    with pytest.raises(ValueError, match="row pointers"):
        STensor.from_csr_arrays(i32(0, 1, 2), i32(1, 0, 2), vals, (2, 3)).validate()
    with pytest.raises(ValueError, match=r"outside \[0, 3\)"):
        STensor.from_csr_arrays(i32(0, 1, 3), i32(1, 0, 3), vals, (2, 3)).validate()
    with pytest.raises(ValueError, match="lengths"):
        STensor.from_csr_arrays(i32(0, 1, 3, 3), i32(1, 0, 2), vals, (2, 3)).validate()
    coo = STensor.from_coo(indices=torch.tensor([[0, 1, 2], [1, 0, 2]]), values=vals, shape=(2, 3))
    with pytest.raises(ValueError, match=r"outside \[0, 2\)"):
        coo.validate()


def test_fp32_attention_schedule_covers_every_block_once_in_short_stretches():
    from scorch_amd import scorch_ops_hip as H
    nb = 64
    brp = torch.tensor(np.concatenate([[0], np.cumsum(np.arange(1, nb + 1))]), dtype=torch.int32)      # causal
    bci = torch.tensor(np.concatenate([np.arange(i + 1) for i in range(nb)]), dtype=torch.int32)
    bm = H.BlockMask(nb * 64, 64, brp, bci, None, None, int(bci.numel()) * 4096)
    items, split_rows, n_slots = H._fp32_schedule(bm)
    items = items.view(-1, 4).tolist()
    lengths = [e - b for _, b, e, _ in items]
    assert max(lengths) <= H.FP32_ATTENTION_STRETCH and lengths == sorted(lengths, reverse=True)
    covered = sorted(p for _, b, e, _ in items for p in range(b, e))
    assert covered == list(range(bci.numel()))
    for row, b, e, slot in items:
        assert brp[row] <= b < e <= brp[row + 1] and (slot >= 0) == (brp[row + 1] - brp[row] > H.FP32_ATTENTION_STRETCH)
    slots = sorted(slot for *_, slot in items if slot >= 0)
    assert slots == list(range(n_slots))
    for row, first, parts, _ in split_rows.view(-1, 4).tolist():
        assert [it[3] for it in items if it[0] == row and it[3] >= 0].__len__() == parts and first >= 0
    assert H._fp32_schedule(bm) is bm.schedule32                       # kept with the mask
    # rows of equal length: nothing to list
    even = H.BlockMask(256, 64, torch.arange(0, 17, 4, dtype=torch.int32), torch.arange(4, dtype=torch.int32).repeat(4),
                       None, None, 16 * 4096)
    assert H._fp32_schedule(even) == (None, None, 0)


# ---- the work split of the SpMM kernels, replayed on the host ---------------------------------------
def _kernel_constant(name, *files):
    import re
    for f in files:
        text = open(os.path.join(os.path.dirname(scorch_ops_hip.__file__), "csrc", f)).read()
        m = re.search(r"constexpr\s+int\s+" + name + r"\s*=\s*([^;]+);", text)
        if m:
            expr = m.group(1)
            for other in re.findall(r"k[A-Z]\w+", expr):
                expr = expr.replace(other, str(_kernel_constant(other, *files)))
            return int(eval(expr, {"__builtins__": {}}))
    raise KeyError(name)


def _spmm_split(M, nnz, N, elem, items_max=256, items_min=32, snap_items=64):
    """spmm_split of scorch_amd/csrc/spmm.hpp."""
    total = M + nnz
    tiles = max((N * elem + 1023) // 1024, 1)
    per_wave = total * tiles // 8192
    ipc = items_min
    while ipc < items_max and ipc * 2 <= per_wave:
        ipc *= 2
    return ipc, min(ipc, snap_items), -(-total // ipc)


def _chunk_boundary(d, M, total, row_ptr, snap):
    """chunk_boundary of scorch_amd/csrc/spmm.hpp: (rows finished, entries before) at merged position d."""
    if d >= total:
        return M, total - M
    keys = row_ptr[1:] + np.arange(M)                   # the position of row i's end marker
    x = int(np.searchsorted(keys, d, side="left"))      # rows whose marker lies before d
    y = d - x
    if x < M:
        begin, end = int(row_ptr[x]), int(row_ptr[x + 1])
        if begin < y and end + x + 1 - d <= snap:
            x, y = x + 1, end
    return x, y


def test_every_chunk_of_the_tiled_split_fits_the_staging_arrays():
    """The kernel for a dense operand stored by column tiles re-splits the work into a multiple of
    128 chunks of up to kTiledItemsMax items; a chunk's end may move forward to a row's end by up to
    kSnapItems more.  What a wavefront stages must fit kTiledSlots: replayed here for a matrix of 32
    entries per row with a hundred rows of 330 to 600."""
    files = ("spmm_tiled.hip", "spmm.hpp")
    items_max, snap_items = _kernel_constant("kTiledItemsMax", *files), _kernel_constant("kSnapItems", *files)
    slots = _kernel_constant("kTiledSlots", *files)
    assert slots >= items_max + snap_items
    rng = np.random.default_rng(3)
    M, N = 4096, 4096
    lens = np.full(M, 32, np.int64)
    lens[rng.choice(M, 100, replace=False)] = rng.integers(330, 601, 100)
    row_ptr = np.concatenate([[0], np.cumsum(lens)])
    nnz = int(row_ptr[-1])
    ipc, snap, spans = _spmm_split(M, nnz, N, 4, _kernel_constant("kItemsPerWave", *files))
    max_wgs = _kernel_constant("kTiledMaxWorkgroupsPerXcd", *files)
    assert 128 < spans <= max_wgs * 4
    even = spans // 128 * 128
    resplit = -(-(M + nnz) // even)
    assert even != spans and ipc < resplit <= items_max           # the case takes the re-split
    ipc, spans = resplit, -(-(M + nnz) // resplit)
    largest = 0
    for c in range(spans):
        x0, y0 = _chunk_boundary(c * ipc, M, M + nnz, row_ptr, snap)
        x1, y1 = _chunk_boundary((c + 1) * ipc, M, M + nnz, row_ptr, snap)
        assert 0 <= y1 - y0 and 0 <= x1 - x0
        largest = max(largest, y1 - y0, x1 - x0 + 2)
    assert largest > _kernel_constant("kItemsPerWave", *files) + snap_items   # more than the usual split stages
    assert largest <= slots


# ---- what the device module keeps beside tensors ----------------------------------------------------
def test_forget_and_mark_volatile_reach_every_tensor_of_an_operand():
    H = scorch_ops_hip
    dense = torch.arange(12.0).reshape(3, 4)
    A = STensor.from_torch(dense.to_sparse_csr(), "A")
    pos, crd = A.index.mode_indices[1]
    found = list(H._tensors_of([A, {"x": dense}, (None, 3)]))
    assert any(t is pos for t in found) and any(t is crd for t in found) and any(t is A.values for t in found)
    assert any(t is dense for t in found)
    before = (H._stamp(pos), H._stamp(crd))
    pos._scorch_plan = object()
    A.values._scorch_ones = (H._stamp(A.values), True)
    H.forget(A)
    assert not hasattr(pos, "_scorch_plan") and not hasattr(A.values, "_scorch_ones")
    assert H._stamp(pos) != before[0] and H._stamp(crd) != before[1]     # plans kept on a partner tensor go stale too
    assert not H.is_volatile(dense)
    dense._scorch_tiled = ("stale",)
    H.mark_volatile(dense)
    assert H.is_volatile(dense) and not hasattr(dense, "_scorch_tiled")
    flat = dense.flatten()
    flat._scorch_origin = dense            # what STensor.from_torch and matmul note on the flat view of a device tensor
    assert H.is_volatile(flat)
    H.mark_volatile(dense, volatile=False)
    assert not H.is_volatile(flat)
    result = H.Tensor(torch.zeros(3), [[], [pos, crd]])
    assert sum(1 for _ in H._tensors_of(result)) == 3


def test_writes_the_version_counter_misses_are_the_ones_forget_is_for():
    """The stamps follow PyTorch's version counter: in-place operations and writes through views
    change them, writes through .data do not -- which is what forget() exists for."""
    H = scorch_ops_hip
    t = torch.zeros(8)
    s0 = H._stamp(t)
    t.add_(1)
    s1 = H._stamp(t)
    assert s1 != s0
    t.view(2, 4)[0].mul_(2)
    s2 = H._stamp(t)
    assert s2 != s1
    t.data.add_(1)
    assert H._stamp(t) == s2
    H.forget(t)
    assert H._stamp(t) != s2


def test_when_attention_workgroups_take_two_items():
    """pair_attention_items on the shapes it was measured on (256 CUs): uneven or very short block
    rows, launches of 0.6 to 4 times what the chip holds at once, rows of 64 blocks at most."""
    pair = scorch_ops_hip.pair_attention_items
    nb = 128
    bi = np.arange(nb)
    c4 = np.array([int(((bi[:i + 1] >= i - 3) | ((i - bi[:i + 1]) % 8 == 0)).sum()) for i in range(nb)])   # the benchmark's mask
    assert c4.sum() == 1466
    causal = lambda n: np.arange(1, n + 1)
    assert pair(c4, 16, 64) and not pair(c4, 64, 64) and not pair(c4, 4, 64)
    assert pair(np.full(nb, 4), 16, 64) and not pair(np.full(nb, 12), 16, 64) and not pair(np.full(nb, 4), 64, 64)
    assert pair(causal(64), 16, 64) and pair(causal(64), 64, 64) and not pair(causal(64), 4, 64)
    assert not pair(causal(64), 128, 64)
    assert pair(causal(64), 32, 128) and pair(causal(64), 16, 32)
    assert not pair(causal(256), 8, 128)                       # rows of 128 blocks on average
    assert not pair(np.full(nb, nb), 16, 64)                   # dense
    assert not pair(np.array([5]), 16, 64) and not pair(c4, 16, 48)
    # the priority step: a quarter of the most a workgroup gets, where a CU holds two workgroups or more
    step = scorch_ops_hip.attention_priority_step
    assert step(c4, 16, 64, True) == 6 and step(c4, 16, 64, False) == 5        # pairs of 23 blocks; rows of 19
    assert step(c4, 4, 64, False) == 5 and step(c4, 2, 64, False) == 0          # 512 and 256 workgroups on 256 CUs
    assert step(causal(64), 16, 64, True) == 17 and step(causal(64), 4, 64, False) == 0
    assert step(causal(63), 16, 64, True) == 16                                 # 63 + 1, ..., the middle item alone
    assert step(np.full(nb, nb), 16, 64, False) == 32 and step(np.full(nb, 4), 64, 64, False) == 0   # eight rounds
    assert step(causal(256), 8, 128, False) == 0                                # four rounds of two workgroups per CU
    assert step(np.array([], np.int64), 16, 64, False) == 0 and step(c4, 16, 48, False) == 0
