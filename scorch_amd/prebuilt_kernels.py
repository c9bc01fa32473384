"""Registry of prebuilt kernels and the call that runs one
(reference: src/scorch/prebuilt_kernels.py).

The table below is the reference's (:37-93): (lhs rank, rhs rank, lhs format,
rhs format, output format) -> candidate symbol names per dtype, tried in
order.  What differs is the module the symbols are looked up in: the
reference looks in its pybind module ``scorch_ops``; here operands live on a
HIP device and the symbols come from ``scorch_ops_hip``, which provides every
family of the table (CSR x dense, CSR x CSR, COO x dense, COO x COO and the
matrix-vector products); a symbol that a module lacks resolves to ``None``,
as it does in the reference.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Any, Callable, List, Mapping, Optional, Sequence, Tuple, TYPE_CHECKING, Union

import torch

from . import scorch_ops_hip as native_ops
from .format import TensorFormat, parse_format

if TYPE_CHECKING:
    from .stensor import STensor

KernelFn = Callable[..., Any]


@dataclass(frozen=True)
class PrebuiltMatmulSpec:
    lhs_rank: int
    rhs_rank: int
    lhs_format: str
    rhs_format: str
    output_format: str
    symbol_by_dtype: Mapping[torch.dtype, Sequence[str]]


@dataclass(frozen=True)
class ResolvedPrebuiltKernel:
    fn: KernelFn
    output_format: TensorFormat
    symbol_name: str


def _typed(prefix: str, *extra_f32: str, first_f32: Sequence[str] = (), f64_alias: Sequence[str] = ()):
    return {
        torch.float32: tuple(first_f32) + (prefix + "f32",) + tuple(extra_f32),
        torch.float64: (prefix + "f64",) + tuple(f64_alias),
        torch.int32: (prefix + "i32",),
        torch.int64: (prefix + "i64",),
    }


_MATMUL_PREBUILT_SPECS: List[PrebuiltMatmulSpec] = [
    PrebuiltMatmulSpec(2, 2, "d,s", "d,d", "dd",
                       _typed("prebuilt_spmm_csr_", "spmm_csr_float", first_f32=("spmm_csr_float_v2",),
                              f64_alias=("spmm_csr_double",))),
    PrebuiltMatmulSpec(2, 2, "d,s", "d,s", "ds", _typed("prebuilt_spmspm_csr_", "spmspm_csr_float")),
    PrebuiltMatmulSpec(2, 2, "o,o", "o,o", "oo", {torch.float32: ("spmspm_coo_float",)}),
    PrebuiltMatmulSpec(2, 2, "o,o", "d,d", "dd", {torch.float32: ("spmm_coo_float",)}),
    PrebuiltMatmulSpec(2, 1, "d,s", "d", "d", _typed("prebuilt_spmv_csr_")),
]


def _resolve_symbol(candidates: Sequence[str]) -> Tuple[Optional[KernelFn], Optional[str]]:
    for name in candidates:
        fn = getattr(native_ops, name, None)
        if fn is not None:
            return fn, name
    return None, None


def resolve_prebuilt_matmul(a: "STensor", b: "STensor",
                            output_format: Optional[Union[TensorFormat, str, List[str]]] = None,
                            ) -> Optional[ResolvedPrebuiltKernel]:
    """First registry entry matching the operands' dtype, ranks, formats and the
    requested output format, or None (reference: prebuilt_kernels.py:104-137)."""
    if a.values.dtype != b.values.dtype:
        return None
    wanted = str(parse_format(output_format)) if output_format is not None else None
    a_fmt, b_fmt = str(a.format), str(b.format)
    for spec in _MATMUL_PREBUILT_SPECS:
        if (a.dim(), b.dim()) != (spec.lhs_rank, spec.rhs_rank):
            continue
        if (a_fmt, b_fmt) != (spec.lhs_format, spec.rhs_format):
            continue
        produced = parse_format(spec.output_format)
        if wanted is not None and wanted != str(produced):
            continue
        symbols = spec.symbol_by_dtype.get(a.values.dtype)
        if symbols is None:
            continue
        fn, name = _resolve_symbol(symbols)
        if fn is None:
            continue
        return ResolvedPrebuiltKernel(fn=fn, output_format=produced, symbol_name=name)
    return None


# ---- fused SpMM + post-ops ------------------------------------------------------
@dataclass(frozen=True)
class PrebuiltFusedSpec:
    lhs_format: str
    rhs_format: str
    post_op_kinds: Tuple[str, ...]
    symbol_by_dtype: Mapping[torch.dtype, Sequence[str]]


@dataclass(frozen=True)
class ResolvedPrebuiltFusedKernel:
    fn: KernelFn
    symbol_name: str


_FUSED_PREBUILT_SPECS: List[PrebuiltFusedSpec] = [
    PrebuiltFusedSpec("d,s", "d,d", ("add", "relu"), {torch.float32: ("spmm_csr_bias_relu_float",)}),
    PrebuiltFusedSpec("d,s", "d,d", ("add",), {torch.float32: ("spmm_csr_bias_float",)}),
]


def resolve_prebuilt_fused(a_format: str, b_format: str, post_op_kinds: Tuple[str, ...],
                           dtype: torch.dtype) -> Optional[ResolvedPrebuiltFusedKernel]:
    """Fused kernel for ``post_op_kinds`` applied to a CSR x dense product, or
    None (reference: prebuilt_kernels.py:176-195)."""
    for spec in _FUSED_PREBUILT_SPECS:
        if (a_format, b_format) != (spec.lhs_format, spec.rhs_format):
            continue
        if tuple(post_op_kinds) != spec.post_op_kinds:
            continue
        symbols = spec.symbol_by_dtype.get(dtype)
        if symbols is None:
            continue
        fn, name = _resolve_symbol(symbols)
        if fn is None:
            continue
        return ResolvedPrebuiltFusedKernel(fn=fn, symbol_name=name)
    return None


def _timed(call: Callable[[], Any], device: torch.device, time_dict: Optional[dict]) -> Any:
    """Run ``call``; with a time_dict, bracket it with device synchronisation so
    that "eval_time" covers the kernel and not just its launch."""
    if time_dict is None:
        return call()
    if device.type == "cuda":
        torch.cuda.synchronize(device)
    start = time.time()
    result = call()
    if device.type == "cuda":
        torch.cuda.synchronize(device)
    time_dict["eval_time"] = time.time() - start
    return result


def execute_prebuilt_binary_kernel(kernel_fn: KernelFn, a: "STensor", b: "STensor",
                                   time_dict: Optional[dict] = None) -> Tuple[Any, Tuple[int, ...]]:
    """Pack (result_shape, then shape / mode_indices / values of each operand)
    and call the kernel (reference: prebuilt_kernels.py:198-224)."""
    if b.dim() == 2:
        result_shape: Tuple[int, ...] = (a.shape[0], b.shape[1])
    elif b.dim() == 1:
        result_shape = (a.shape[0],)
    else:
        raise ValueError(f"Unsupported RHS rank for prebuilt matmul kernel: {b.dim()}")
    args: List[Any] = [result_shape]
    for operand in (a, b):
        args += [operand.shape, operand.index.mode_indices, operand.values]
    result = _timed(lambda: kernel_fn(*args), a.values.device, time_dict)
    return result, result_shape
