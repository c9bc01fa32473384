"""Fused block-sparse attention in fp32 on the MI355X through the C ABI.

Tolerance: relative Frobenius error <= 1e-5 against an fp64 recomputation of the textbook masked
softmax (the reference's "dense" mode, bench/bench_sparse_transformer.py:330-335) on the same
inputs -- the fp32 bar -- and the same bound against this package's own fp32 SDDMM -> softmax ->
SpMM pipeline, the form in which the reference composes sparse attention (:354-372).  The reference
has no fused kernel, so nothing of its own pins this one beyond that composition.
"""
import numpy as np
import pytest
import torch

from gpu_util import dev
from scorch_amd import workloads
from scorch_amd import scorch_ops_hip as H

pytestmark = pytest.mark.gpu
TOL = 1e-5


def csr_of(mask_bool):
    rp = np.concatenate([[0], np.cumsum(mask_bool.sum(1))]).astype(np.int32)
    return rp, np.nonzero(mask_bool)[1].astype(np.int32)


def case(oracle, mask_bool, heads, D, seed, scale=None, spread=1.0):
    S = mask_bool.shape[0]
    rng = np.random.default_rng(seed)
    q, k, v = (rng.standard_normal((heads, S, D)).astype(np.float32) * spread for _ in range(3))
    scale = D ** -0.5 if scale is None else scale
    rp, ci = csr_of(mask_bool)
    out = H.sparse_attention_f32(dev(q), dev(k), dev(v), dev(rp), dev(ci), scale)
    assert out.dtype == torch.float32 and out.shape == (heads, S, D)
    ref = np.stack([oracle.attention_dense_fp64(q[h], k[h], v[h], mask_bool, scale) for h in range(heads)])
    return out.cpu().numpy(), ref


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("density", [0.03, 0.6])
def test_random_entry_masks(oracle, D, density):
    rng = np.random.default_rng(50 + D)
    mask = rng.random((320, 320)) < density
    mask[17, :] = False                                   # a query without any key: a zero row
    out, ref = case(oracle, mask, 3, D, 51)
    assert oracle.rel_fro(out, ref) <= TOL
    assert np.all(out[:, 17] == 0)


@pytest.mark.parametrize("D", [32, 64, 128])
def test_causal_mask(oracle, D):
    out, ref = case(oracle, np.tril(np.ones((448, 448), bool)), 2, D, 52)
    assert oracle.rel_fro(out, ref) <= TOL


@pytest.mark.parametrize("scale", [-0.7, 0.0, 3.0])
def test_negative_zero_and_large_scales(oracle, scale):
    rng = np.random.default_rng(53)
    mask = rng.random((256, 256)) < 0.3
    out, ref = case(oracle, mask, 2, 64, 54, scale=scale, spread=3.0)
    assert np.isfinite(out).all() and oracle.rel_fro(out, ref) <= TOL


def test_whole_blocks_without_bit_masks(oracle):
    """A pattern of whole 64 x 64 blocks handed over as such (no mask index, no bit masks): the
    benchmark's block pattern at a small size, with an empty block row."""
    w = workloads.attention_blocksparse(S=512, H=3, D=64, seed=55)
    brp, bci = w["block_row_ptr"].copy(), w["block_col_idx"]
    bm = H.BlockMask(512, 64, dev(brp), dev(bci), None, None, int(bci.size) * 4096)
    out = H.attn_blocksparse_f32(dev(w["q"]), dev(w["k"]), dev(w["v"]), bm, float(w["scale"])).cpu().numpy()
    rp, ci = workloads.blocks_to_csr(brp, bci, 64)
    dense = np.zeros((512, 512), bool)
    dense[np.repeat(np.arange(512), np.diff(rp)), ci] = True
    ref = np.stack([oracle.attention_dense_fp64(w["q"][h], w["k"][h], w["v"][h], dense, float(w["scale"]))
                    for h in range(3)])
    assert oracle.rel_fro(out, ref) <= TOL


def test_longformer_mask_reference_shape_against_the_three_launch_form():
    """The reference's attention benchmark at its own shape (S = 4096, 8 heads, D = 32, window 64 +
    one global token: bench/bench_sparse_transformer.py:117-141,194-209), whose global token's block
    row is shared out among workgroups: the fused fp32 kernel against the fp64 dense masked softmax
    and against SDDMM -> softmax -> SpMM in fp32."""
    S, heads, D = 4096, 8, 32
    rp, ci = workloads.longformer_mask(S)
    rng = np.random.default_rng(56)
    q, k, v = (torch.from_numpy(rng.standard_normal((heads, S, D)).astype(np.float32)).cuda() for _ in range(3))
    scale = D ** -0.5
    drp, dci = dev(rp), dev(ci)
    out = H.sparse_attention_f32(q, k, v, drp, dci, scale)
    assert H.attention_block_mask(drp, dci, S).schedule32[1].numel() > 0     # the shared-out row is exercised
    assert torch.equal(out, H.sparse_attention_f32(q, k, v, drp, dci, scale))
    dense = torch.zeros(S, S, dtype=torch.bool)
    dense[torch.from_numpy(np.repeat(np.arange(S), np.diff(rp))), torch.from_numpy(ci).long()] = True
    dense = dense.cuda()
    for h in range(heads):
        s = (q[h].double() @ k[h].double().T) * scale
        s.masked_fill_(~dense, float("-inf"))
        ref = torch.softmax(s, dim=-1) @ v[h].double()
        assert (torch.linalg.norm(out[h].double() - ref) / torch.linalg.norm(ref)).item() <= TOL
    unfused = H.sparse_attention_csr(drp, dci, q, k, v, scale)
    assert (torch.linalg.norm(out - unfused) / torch.linalg.norm(unfused)).item() <= TOL


def test_arguments_are_checked():
    bm = H.BlockMask(128, 64, dev(np.array([0, 1, 2], np.int32)), dev(np.array([0, 1], np.int32)), None, None, 8192)
    q = torch.zeros(1, 128, 64, device="cuda")
    with pytest.raises(TypeError, match="float32"):
        H.attn_blocksparse_f32(q.bfloat16(), q.bfloat16(), q.bfloat16(), bm, 1.0)
    with pytest.raises(ValueError, match="another sequence length"):
        H.attn_blocksparse_f32(q[:, :64], q[:, :64], q[:, :64], bm, 1.0)
    q48 = torch.zeros(1, 128, 48, device="cuda")
    with pytest.raises(RuntimeError, match="head dimensions 32, 64 and 128"):
        H.attn_blocksparse_f32(q48, q48, q48, bm, 1.0)


def test_keys_the_mask_leaves_out_may_hold_anything_in_k(oracle):
    """Padding keys that no query attends to: their rows of K may be NaN (their scores are replaced
    before they are looked at); their rows of V are multiplied by zero probabilities, so V has to be
    finite there.  Both fused kernels, against the fp64 result on clean operands."""
    S, heads, D = 256, 2, 64
    rng = np.random.default_rng(21)
    i, j = np.arange(S)[:, None], np.arange(S)[None, :]
    mask = j <= i
    padded = np.r_[50:64, 130:131, 192:256]         # part of a block, one key, a whole block column
    mask[:, padded] = False
    mask[padded, 0] = True                           # (the padded queries attend to the first key)
    q, k, v = (rng.standard_normal((heads, S, D)).astype(np.float32) for _ in range(3))
    k_bad = k.copy()
    k_bad[:, padded] = np.nan
    rp, ci = csr_of(mask)
    ref = np.stack([oracle.attention_dense_fp64(q[h], k[h], v[h], mask, D ** -0.5) for h in range(heads)])
    out32 = H.sparse_attention_f32(dev(q), dev(k_bad), dev(v), dev(rp), dev(ci), D ** -0.5).cpu().numpy()
    assert np.isfinite(out32).all() and oracle.rel_fro(out32, ref) <= TOL
    to16 = lambda a: dev(a).to(torch.bfloat16)
    out16 = H.sparse_attention_bf16(to16(q), to16(k_bad), to16(v), dev(rp), dev(ci), D ** -0.5).float().cpu().numpy()
    assert np.isfinite(out16).all() and oracle.rel_fro(out16, ref) <= 1e-2
