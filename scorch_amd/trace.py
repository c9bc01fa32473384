"""``@scorch_amd.compile``: fuse ``matmul -> + bias [-> relu]`` into one kernel
(reference: src/scorch/trace.py).

The decorated function is traced once with torch.fx, with ``matmul`` kept as a
single node.  The chain of elementwise operations that consumes the product is
read off the graph; if it is ``add`` or ``add, relu`` on a CSR x dense fp32
product, the call is served by the fused SpMM kernel
(``spmm_csr_bias[_relu]_float``), which applies bias and activation when it
stores each row.  Any other chain runs as the plain ``matmul`` followed by the
same torch operations, one after the other -- what the reference's non-prebuilt
route amounts to (trace.py:304-358) -- so results are identical either way.
Whatever the function does after the chain (a reduction, an indexing step, a
second consumer of the product) is run from the traced graph on the chain's
result, so the decorated function always returns what the plain function would.
"""
from __future__ import annotations

import contextlib
import operator
import sys
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional

import torch
import torch.fx

from . import ops
from .prebuilt_kernels import resolve_prebuilt_fused
from .stensor import STensor


@dataclass
class PostOp:
    """One elementwise step applied to the product."""
    kind: str                           # "add", "mul", "relu", "sigmoid", "tanh"
    tensor_name: Optional[str] = None   # operand of a binary step


@dataclass
class PostOps:
    ops: List[PostOp] = field(default_factory=list)
    extra_tensors: List[str] = field(default_factory=list)


@dataclass
class FusionSpec:
    matmul_node: torch.fx.Node
    matmul_arg_indices: List[int]       # which arguments of the function feed the matmul
    matmul_kwargs: dict
    post_ops: PostOps
    extra_arg_indices: List[int]        # arguments that are operands of the post-ops
    output_format: Optional[str] = None
    chain_nodes: List[torch.fx.Node] = field(default_factory=list)   # matmul and the chain, in order
    complete: bool = True               # the chain's last node is what the function returns


_BINARY = {operator.add: "add", operator.mul: "mul", torch.add: "add", torch.mul: "mul"}
_UNARY = {torch.relu: "relu", torch.nn.functional.relu: "relu", torch.sigmoid: "sigmoid",
          torch.tanh: "tanh"}
_UNARY_FN = {"relu": torch.relu, "sigmoid": torch.sigmoid, "tanh": torch.tanh}


@contextlib.contextmanager
def _matmul_as_leaf(fn: Callable):
    """While active, every way the traced function can reach ``matmul``
    (``scorch_amd.matmul``, ``scorch_amd.ops.matmul``, a ``from ... import
    matmul`` in its module) resolves to a stand-in that records one
    ``call_function`` node targeting the real ``ops.matmul`` instead of being
    traced through."""
    real = ops.matmul

    def leaf(*args, **kwargs):
        for a in list(args) + list(kwargs.values()):
            if isinstance(a, torch.fx.Proxy):
                return a.tracer.create_proxy("call_function", real, args, kwargs)
        return real(*args, **kwargs)

    package = sys.modules[__package__]
    spots = [(package.__dict__, "matmul"), (ops.__dict__, "matmul")]
    fn_globals = getattr(fn, "__globals__", None)
    if fn_globals is not None and fn_globals.get("matmul") is real:
        spots.append((fn_globals, "matmul"))
    saved = [(d, k, d[k]) for d, k in spots if k in d]
    for d, k, _ in saved:
        d[k] = leaf
    try:
        yield
    finally:
        for d, k, v in saved:
            d[k] = v


def _symbolic_trace(fn: Callable) -> torch.fx.GraphModule:
    """torch.fx graph of ``fn`` with ``matmul`` as one opaque node."""
    with _matmul_as_leaf(fn):
        tracer = torch.fx.Tracer()
        graph = tracer.trace(fn)
        return torch.fx.GraphModule(tracer.root, graph)


def analyze_fx_graph(graph: torch.fx.Graph, real_args: tuple) -> FusionSpec:
    """Find the matmul node and the elementwise chain hanging off it."""
    placeholders = [n for n in graph.nodes if n.op == "placeholder"]
    index_of = {n: i for i, n in enumerate(placeholders)}
    matmul_node = next((n for n in graph.nodes
                        if n.op == "call_function" and n.target is ops.matmul), None)
    if matmul_node is None:
        raise ValueError("No scorch.matmul found in traced function")
    matmul_args = [index_of[a] for a in matmul_node.args
                   if isinstance(a, torch.fx.Node) and a in index_of]

    chain = PostOps()
    extra: List[int] = []
    node = matmul_node
    walked = [matmul_node]
    while len(node.users) == 1:
        (user,) = node.users
        if user.op != "call_function":
            break
        if user.target in _BINARY and len(user.args) == 2:
            other = user.args[1] if user.args[0] is node else user.args[0]
            if other not in index_of:
                break
            name = f"postop_{len(chain.extra_tensors)}"
            chain.ops.append(PostOp(_BINARY[user.target], name))
            chain.extra_tensors.append(name)
            extra.append(index_of[other])
        elif user.target in _UNARY:
            chain.ops.append(PostOp(_UNARY[user.target]))
        else:
            break
        node = user
        walked.append(node)
    kwargs = dict(matmul_node.kwargs)
    # the runners return the chain's result: that is the function's result only if the
    # chain's last node feeds the output node directly and nothing else
    users = list(node.users)
    complete = len(users) == 1 and users[0].op == "output" and users[0].args[0] is node
    return FusionSpec(matmul_node, matmul_args, kwargs, chain, extra, kwargs.get("format"), walked, complete)


class _Remainder(torch.fx.Interpreter):
    """Runs the traced function with the value of the chain's last node given: the
    nodes of the chain are not executed again, everything else is."""

    def __init__(self, module: torch.fx.GraphModule, spec: FusionSpec, value: Any):
        super().__init__(module)
        self._skip = set(spec.chain_nodes[:-1])
        self._tail = spec.chain_nodes[-1]
        self._value = value

    def run_node(self, n: torch.fx.Node) -> Any:
        if n is self._tail:
            return self._value
        if n in self._skip:
            return None     # consumed by the next node of the chain only
        return super().run_node(n)


def _as_stensor(x) -> STensor:
    return x if isinstance(x, STensor) else STensor.from_torch(x)


def _try_prebuilt_fused(spec: FusionSpec, args: tuple) -> Optional[Callable]:
    """Runner that serves the whole chain with one fused kernel, or None."""
    if len(spec.matmul_arg_indices) != 2:
        return None
    a, b = (args[i] for i in spec.matmul_arg_indices)
    if not isinstance(a, STensor):
        return None  # as in the reference, the fused route takes an STensor on the left
    if isinstance(b, STensor):
        b_format = str(b.format)
    elif isinstance(b, torch.Tensor):
        b_format = ",".join("d" * b.dim())
    else:
        return None
    kinds = tuple(op.kind for op in spec.post_ops.ops)
    resolved = resolve_prebuilt_fused(str(a.format), b_format, kinds, a.values.dtype)
    if resolved is None:
        return None
    a_idx, b_idx = spec.matmul_arg_indices
    bias_idx = spec.extra_arg_indices[0]
    kernel = resolved.fn

    def run(call_args: tuple) -> torch.Tensor:
        lhs, rhs = _as_stensor(call_args[a_idx]), _as_stensor(call_args[b_idx])
        rows, cols = lhs.shape[0], rhs.shape[1]
        out = kernel([rows, cols], list(lhs.shape), lhs.index.mode_indices, lhs.values, list(rhs.shape),
                     rhs.index.mode_indices, rhs.values, call_args[bias_idx])
        return out.storage.value.view(rows, cols)

    run.fused_symbol = resolved.symbol_name
    return run


def _unfused(spec: FusionSpec, args: tuple) -> Callable:
    """Runner: plain matmul, then the post-ops as torch operations."""
    a_idx, b_idx = spec.matmul_arg_indices[:2]
    kwargs = {k: v for k, v in spec.matmul_kwargs.items() if not k.startswith("_")}
    steps = list(spec.post_ops.ops)
    extra = list(spec.extra_arg_indices)

    def run(call_args: tuple):
        result = ops.matmul(call_args[a_idx], call_args[b_idx], **kwargs)
        operands = iter(call_args[i] for i in extra)
        for step in steps:
            if step.kind == "add":
                result = result + next(operands)
            elif step.kind == "mul":
                result = result * next(operands)
            else:
                result = _UNARY_FN[step.kind](result)
        return result

    run.fused_symbol = None
    return run


def compile_fused(spec: FusionSpec, args: tuple) -> Callable:
    return _try_prebuilt_fused(spec, args) or _unfused(spec, args)


class compile:
    """Decorator: ``@scorch_amd.compile`` on a function of the form
    ``matmul(a, b) [+ bias] [-> relu ...]``.  Traced on first call; one runner is
    cached per combination of argument formats and dtypes."""

    def __init__(self, fn: Callable):
        self.fn = fn
        self._fx_graph: Optional[torch.fx.GraphModule] = None
        self._cache: Dict[tuple, tuple] = {}

    def __call__(self, *args: Any) -> Any:
        if self._fx_graph is None:
            self._fx_graph = _symbolic_trace(self.fn)
        key = self._build_cache_key(args)
        cached = self._cache.get(key)
        if cached is None:
            spec = analyze_fx_graph(self._fx_graph.graph, args)
            cached = (compile_fused(spec, args), spec)
            self._cache[key] = cached
        runner, spec = cached
        result = runner(args)
        if spec.complete:
            return result
        return _Remainder(self._fx_graph, spec, result).run(*args)

    @staticmethod
    def _build_cache_key(args: tuple) -> tuple:
        key = []
        for a in args:
            if isinstance(a, STensor):
                key.append((str(a.format), a.dtype))
            elif isinstance(a, torch.Tensor):
                key.append((f"dense_{a.dim()}d", a.dtype))
            else:
                key.append(type(a))
        return tuple(key)
