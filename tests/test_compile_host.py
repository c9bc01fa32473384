"""@scorch_amd.compile on the host: tracing and fusion analysis (mirrors
tests/test_scorch/test_compile.py:34-66 of the reference) and the choice of
runner.  No kernel runs here."""
import torch

import scorch_amd as scorch
from scorch_amd import STensor
from scorch_amd.trace import (_symbolic_trace, _try_prebuilt_fused, analyze_fx_graph, compile_fused)
from scorch_amd.trace import compile as scorch_compile


def csr_and_dense(n=64, k=16, density=0.1, seed=42, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    vals = (torch.rand(n, n, generator=g) * (torch.rand(n, n, generator=g) < density)).to(dtype)
    return STensor.from_csr(vals.to_sparse_csr(), "A"), torch.rand(n, k, generator=g).to(dtype)


def bias_relu(adj, x, bias):
    h = scorch.matmul(adj, x, format="dd")
    h = h + bias
    return torch.relu(h)


def test_trace_keeps_matmul_as_one_node_and_restores_it():
    before = scorch.matmul
    traced = _symbolic_trace(bias_relu)
    targets = [n.target for n in traced.graph.nodes if n.op == "call_function"]
    assert scorch.ops.matmul in targets and torch.relu in targets
    assert scorch.matmul is before and scorch.ops.matmul is before


def test_fusion_analysis_reads_the_chain():
    adj, x = csr_and_dense()
    spec = analyze_fx_graph(_symbolic_trace(bias_relu).graph, (adj, x, torch.rand(16)))
    assert [op.kind for op in spec.post_ops.ops] == ["add", "relu"]
    assert spec.extra_arg_indices == [2] and spec.matmul_arg_indices == [0, 1]
    assert spec.matmul_kwargs == {"format": "dd"} and spec.output_format == "dd"


def test_fusion_analysis_stops_at_a_non_elementwise_consumer():
    def fn(adj, x, bias):
        return (scorch.matmul(adj, x) + bias).sum()
    adj, x = csr_and_dense()
    spec = analyze_fx_graph(_symbolic_trace(fn).graph, (adj, x, torch.rand(16)))
    assert [op.kind for op in spec.post_ops.ops] == ["add"]
    assert not spec.complete and [n.op for n in spec.chain_nodes] == ["call_function"] * 2
    whole = analyze_fx_graph(_symbolic_trace(bias_relu).graph, (adj, x, torch.rand(16)))
    assert whole.complete and len(whole.chain_nodes) == 3


def test_what_follows_the_chain_is_run_from_the_graph(monkeypatch):
    """(matmul + c).sum(dim=1) * 2 returns a vector, not the product with its bias: the steps
    after the chain run on the chain's result.  The product itself is stubbed (no device here)."""
    from scorch_amd import trace
    adj, x = csr_and_dense()
    dense = adj.to_dense().to_torch()

    def fake_matmul(a, b, **kwargs):
        return dense @ (b.to_torch() if isinstance(b, STensor) else b)

    monkeypatch.setattr(trace.ops, "matmul", fake_matmul)
    monkeypatch.setattr(trace, "_try_prebuilt_fused", lambda spec, args: None)

    @scorch_compile
    def reduced(a, b, c):
        return (scorch.matmul(a, b, format="dd") + c).sum(dim=1) * 2.0

    @scorch_compile
    def two_consumers(a, b, c):
        h = scorch.matmul(a, b, format="dd")
        return torch.relu(h + c) - h

    c = torch.rand(16)
    out = reduced(adj, x, c)
    assert out.shape == (64,)
    torch.testing.assert_close(out, (dense @ x + c).sum(dim=1) * 2.0)
    torch.testing.assert_close(two_consumers(adj, x, c), torch.relu(dense @ x + c) - dense @ x)


def test_runner_choice():
    adj, x = csr_and_dense()
    bias = torch.rand(16)
    spec = analyze_fx_graph(_symbolic_trace(bias_relu).graph, (adj, x, bias))
    assert compile_fused(spec, (adj, x, bias)).fused_symbol == "spmm_csr_bias_relu_float"

    def bias_only(adj, x, bias):
        return scorch.matmul(adj, x) + bias
    spec = analyze_fx_graph(_symbolic_trace(bias_only).graph, (adj, x, bias))
    assert compile_fused(spec, (adj, x, bias)).fused_symbol == "spmm_csr_bias_float"

    def relu_only(adj, x):
        return torch.relu(scorch.matmul(adj, x))
    spec = analyze_fx_graph(_symbolic_trace(relu_only).graph, (adj, x))
    assert _try_prebuilt_fused(spec, (adj, x)) is None          # no fused kernel for relu alone
    assert compile_fused(spec, (adj, x)).fused_symbol is None

    adj64, x64 = csr_and_dense(dtype=torch.float64)
    spec = analyze_fx_graph(_symbolic_trace(bias_relu).graph, (adj64, x64, bias.double()))
    assert compile_fused(spec, (adj64, x64, bias.double())).fused_symbol is None   # fp32 only


def test_cache_key_separates_formats_and_dtypes():
    adj, x = csr_and_dense()
    key = scorch_compile._build_cache_key
    assert key((adj, x)) == key((adj, x.clone()))
    assert key((adj, x)) != key((adj, x.double()))
    assert key((adj, x)) != key((adj.to_sparse("oo"), x))
    assert key((adj, x, 3)) != key((adj, x, 3.0))
