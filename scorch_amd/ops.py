"""matmul / einsum with the reference's call signatures, for device-resident
operands (reference: src/scorch/ops.py:248-423).

What is routed here: CSR x dense ``matmul`` (and its einsum spelling
"ij,jk->ik"), CSR x vector ``matmul``, and the SDDMM einsum "ij,ik,jk->ij"
with a coordinate or CSR mask.  Those are the expressions the reference serves
with prebuilt native kernels (plus the CSR-mask SDDMM its code generator
serves); here they run as HIP kernels.  Every other expression belongs to the
reference's compiler, which this package does not contain: it raises
``NotImplementedError`` rather than compute anything a different way.

There is no host path: a sparse operand that is not on a HIP device raises
``RuntimeError``.  (Dense x dense goes to ``torch.matmul`` on whatever device,
exactly as the reference does at ops.py:256-293.)
"""
from __future__ import annotations

from typing import Any, List, Optional, Union

import torch

from . import scorch_ops_hip
from .format import TensorFormat, parse_format
from .prebuilt_kernels import (_timed, execute_prebuilt_binary_kernel, resolve_prebuilt_fused,
                               resolve_prebuilt_matmul)
from .stensor import STensor
from .storage import TensorIndex

_SPMM_EXPR = "ab,bc->ac"
_SDDMM_EXPR = "ab,ac,bc->ab"       # "ij,ik,jk->ij": B indexed [j, k]
_SDDMM_EXPR_KJ = "ab,ac,cb->ab"    # "ij,ik,kj->ij": B indexed [k, j]


def _canonical(expression: str) -> str:
    """Rename subscripts by order of first appearance: "ik,kj->ij" -> "ab,bc->ac"."""
    names = {}
    out = []
    for ch in expression.replace(" ", ""):
        if ch.isalpha():
            if ch not in names:
                names[ch] = chr(ord("a") + len(names))
            out.append(names[ch])
        else:
            out.append(ch)
    return "".join(out)


def _not_on_device(device) -> RuntimeError:
    return RuntimeError("scorch_amd runs sparse kernels on HIP devices only; this operand is on "
                        f"{device}. Move it with STensor.to('cuda') (host tensors belong to the "
                        "reference's CPU kernels).")


def _require_device(*tensors: STensor) -> None:
    for t in tensors:
        if not t.values.is_cuda:
            raise _not_on_device(t.values.device)


def _wrap(result_cpp, shape, fmt) -> STensor:
    return STensor(shape=tuple(shape),
                   index=TensorIndex(mode_indices=result_cpp.storage.index.mode_indices,
                                     tensor_format=fmt),
                   value=result_cpp.storage.value)


def _not_prebuilt(what: str):
    return NotImplementedError(
        f"{what}: no prebuilt device kernel matches; the reference compiles such expressions with "
        "its code generator, which is outside this package")


def _run_prebuilt_matmul(a: STensor, b: STensor, requested_format, time_dict):
    resolved = resolve_prebuilt_matmul(a, b, output_format=requested_format)
    if resolved is None:
        return None
    _require_device(a, b)
    result_cpp, result_shape = execute_prebuilt_binary_kernel(resolved.fn, a, b, time_dict=time_dict)
    return _wrap(result_cpp, result_shape, resolved.output_format)


def _as_format(result: STensor, requested) -> STensor:
    """`result` re-stored in the requested format (on its device)."""
    if requested is None:
        return result
    fmt = parse_format(requested)
    if str(fmt) == str(result.format):
        return result
    if fmt.is_dense():
        return STensor.from_torch(result.to_torch().contiguous())
    return result.to_sparse(fmt)


def _run_converted_matmul(a: STensor, b: STensor, requested, time_dict) -> Optional[STensor]:
    """Matrix products of 2-D operands in any mix of "d,d", "d,s" and "o,o" (and a
    sparse matrix times a dense vector) that no registry entry takes as they
    are: the operands are re-stored, on the device, in the formats a prebuilt
    kernel takes, and its result in the format asked for.  The reference sends
    these combinations to its code generator (ops.py:358-367); the contraction
    is the same, so the values agree to rounding.  ``eval_time`` covers the
    kernel, as it does for a direct hit."""
    kinds = ("d,d", "d,s", "o,o")
    if a.dim() != 2 or str(a.format) not in kinds or a.values.dtype != b.values.dtype:
        return None
    if b.dim() == 1:
        if not b.format.is_dense() or a.format.is_dense():
            return None
        natural = _run_prebuilt_matmul(a.to_sparse("ds"), b, None, time_dict)
        return None if natural is None else _as_format(natural, requested)
    if b.dim() != 2 or str(b.format) not in kinds:
        return None
    if a.format.is_dense():
        if b.format.is_dense():
            return None
        # A B = (B^T A^T)^T with B^T in CSR, i.e. B stored by columns
        _require_device(a, b)
        bt = b.copy().to_sparse("ds").change_mode_order([1, 0])
        pos, crd = bt.index.mode_indices[1]
        bt = STensor.from_csr_arrays(pos, crd, bt.values, (b.shape[1], b.shape[0]))
        at = STensor.from_torch(a.to_torch(in_place=False).t().contiguous())
        natural = _run_prebuilt_matmul(bt, at, None, time_dict)
        if natural is None:
            return None
        natural = STensor.from_torch(natural.to_torch().t().contiguous())
    else:
        left = a.to_sparse("ds")
        right = b if b.format.is_dense() else b.to_sparse("ds")
        natural = _run_prebuilt_matmul(left, right, None, time_dict)
        if natural is None:
            return None
    return _as_format(natural, requested)


# The product this package is about -- a CSR STensor times a dense torch tensor, result dense --
# resolved once per (dtypes, ranks) through the registry and then called without wrapping the
# dense operand and the result in STensors (two nn.Module constructions, most of the general
# path's 30 us per call, against a kernel of a few microseconds).
_direct_matmul: dict = {}
_direct_fused: dict = {}


_dense_requests: dict = {}


def _requests_dense(requested, rank: int) -> bool:
    """Whether a ``format`` argument asks for what this route returns anyway: a dense result of
    this rank ("dd" for a matrix).  Strings are parsed once."""
    if requested is None:
        return True
    key = (requested, rank) if isinstance(requested, str) else None
    known = _dense_requests.get(key) if key is not None else None
    if known is None:
        try:
            fmt = parse_format(requested)
            known = fmt.is_dense() and fmt.get_order() == rank
        except Exception:
            known = False        # the general path words the error
        if key is not None:
            _dense_requests[key] = known
    return known


def _matmul_csr_dense_direct(a: STensor, b: torch.Tensor, kwargs) -> Optional[torch.Tensor]:
    if kwargs and not (set(kwargs) <= {"time_dict", "use_cache", "format", "output_format"}
                       and kwargs.get("use_cache", True)):
        return None
    if kwargs and not _requests_dense(kwargs.get("format", kwargs.get("output_format", None)), b.dim()):
        return None
    if b.layout != torch.strided or b.dim() not in (1, 2) or a.dim() != 2 or not b.is_cuda:
        return None
    if str(a.format) != "d,s" or a.index.mode_order != [0, 1] or not a.values.is_cuda:
        return None
    if a.shape[1] != b.shape[0]:
        return None          # the general path words the error
    key = (a.values.dtype, b.dtype, b.dim())
    fn = _direct_matmul.get(key)
    if fn is None:
        resolved = resolve_prebuilt_matmul(a, STensor.from_torch(b), output_format=None)
        if resolved is None or not resolved.output_format.is_dense():
            return None
        fn = _direct_matmul[key] = resolved.fn
    result_shape = (a.shape[0], b.shape[1]) if b.dim() == 2 else (a.shape[0],)
    values = b.reshape(-1)
    if values is not b and values.data_ptr() == b.data_ptr():
        values._scorch_origin = b    # a flat view: layouts cached for this operand live on the caller's tensor
    result = _timed(lambda: fn(result_shape, a.shape, a.index.mode_indices, a.values,
                               tuple(b.shape), [[] for _ in range(b.dim())], values),
                    a.values.device, kwargs.get("time_dict", None))
    return result.storage.value.view(result_shape)


def matmul(a: Union[torch.Tensor, STensor], b: Union[torch.Tensor, STensor],
           **kwargs: Any) -> Union[torch.Tensor, STensor]:
    """Matrix product.  Keyword arguments as in the reference: ``format`` /
    ``output_format``, ``use_cache``, ``time_dict``."""
    if isinstance(a, STensor) and isinstance(b, torch.Tensor):
        direct = _matmul_csr_dense_direct(a, b, kwargs)
        if direct is not None:
            return direct
    if isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor):
        sparse_a = a.layout != torch.strided
        sparse_b = b.layout != torch.strided
        if not (sparse_a or sparse_b):
            return torch.matmul(a, b)
        if a.layout == torch.sparse_coo and b.layout == torch.sparse_coo:
            a, b = a.to_sparse_csr(), b.to_sparse_csr()
    if isinstance(a, torch.Tensor):
        a = STensor.from_torch(a)
    if isinstance(b, torch.Tensor):
        b = STensor.from_torch(b)

    time_dict = kwargs.get("time_dict", None)
    requested = kwargs.get("format", kwargs.get("output_format", None))

    if a.format.is_dense() and b.format.is_dense():
        result = _timed(lambda: torch.matmul(a.to_torch(in_place=False), b.to_torch(in_place=False)),
                        a.values.device, time_dict)
        if requested is None or parse_format(requested).is_dense():
            return result
        return STensor.from_torch(result).to_sparse(parse_format(requested))

    # Sparse matrices stored in a non-default mode order are re-stored in the
    # default one first, as the reference does (ops.py:299-303,333-346).
    if a.dim() == 2 and b.dim() in (1, 2) and not (a.format.is_dense() and b.format.is_dense()):
        if a.index.mode_order != [0, 1]:
            a = a.copy().change_mode_order([0, 1])
        if b.dim() == 2 and b.index.mode_order != [0, 1]:
            b = b.copy().change_mode_order([0, 1])

    if kwargs.get("use_cache", True):
        result = _run_prebuilt_matmul(a, b, requested, time_dict)
        if result is None:
            result = _run_converted_matmul(a, b, requested, time_dict)
        if result is None:
            raise _not_prebuilt(f"matmul({a.format} x {b.format}, {a.values.dtype}, format={requested})")
    else:
        # the reference sends use_cache=False through einsum (ops.py:364-367)
        expr = "ij,jk->ik" if b.dim() == 2 else "ij,j->i"
        result = einsum(expr, a, b, **kwargs)

    if isinstance(result, STensor) and result.format.is_dense():
        result = result.to_torch()
    return result


def _sddmm(mask: STensor, A: STensor, B: STensor, time_dict) -> Optional[STensor]:
    if mask.values.dtype != torch.float32 or A.values.dtype != torch.float32 \
            or B.values.dtype != torch.float32:
        return None
    if str(A.format) != "d,d" or str(B.format) != "d,d":
        return None
    mask_fmt = str(mask.format)
    if mask_fmt == "o,o":
        fn = scorch_ops_hip.sddmm_coo_float_prebuilt
    elif mask_fmt == "d,s":
        fn = scorch_ops_hip.sddmm_csr_float
    else:
        return None
    _require_device(mask, A, B)
    result_cpp = _timed(lambda: fn(mask.shape, mask.shape, mask.index.mode_indices, mask.values,
                                   A.shape, A.index.mode_indices, A.values,
                                   B.shape, B.index.mode_indices, B.values),
                        mask.values.device, time_dict)
    # coordinate mask: the result keeps the mask's format and index tensors
    # (reference ops.py:416-423); CSR mask: all-coordinate result (ops.py:638-666)
    return _wrap(result_cpp, mask.shape, mask.format if mask_fmt == "o,o" else "oo")


_canonical_cache: dict = {}


def _sddmm_direct(mask, A, B, time_dict) -> Optional[STensor]:
    """The SDDMM with a sparse STensor mask and two dense fp32 torch tensors on the device: the
    kernel is called without wrapping the dense operands in STensors first."""
    if not (isinstance(mask, STensor) and isinstance(A, torch.Tensor) and isinstance(B, torch.Tensor)):
        return None
    if A.layout != torch.strided or B.layout != torch.strided or A.dim() != 2 or B.dim() != 2:
        return None
    if not (A.is_cuda and B.is_cuda and mask.values.is_cuda):
        return None
    if mask.values.dtype != torch.float32 or A.dtype != torch.float32 or B.dtype != torch.float32:
        return None
    mask_fmt = str(mask.format)
    if mask_fmt == "o,o":
        fn = scorch_ops_hip.sddmm_coo_float_prebuilt
    elif mask_fmt == "d,s" and mask.index.mode_order == [0, 1]:
        fn = scorch_ops_hip.sddmm_csr_float
    else:
        return None
    dense_index = [[], []]
    result_cpp = _timed(lambda: fn(mask.shape, mask.shape, mask.index.mode_indices, mask.values,
                                   tuple(A.shape), dense_index, A.reshape(-1),
                                   tuple(B.shape), dense_index, B.reshape(-1)),
                        mask.values.device, time_dict)
    return _wrap(result_cpp, mask.shape, mask.format if mask_fmt == "o,o" else "oo")


def einsum(expression: str, *tensors: Optional[Union[torch.Tensor, STensor]],
           compile_only: Optional[bool] = False, **kwargs: Any) -> Union[STensor, torch.Tensor]:
    """Einstein summation for the expressions that have a device kernel."""
    if compile_only:
        raise _not_prebuilt("einsum(compile_only=True)")
    canon = _canonical_cache.get(expression)
    if canon is None:
        canon = _canonical_cache[expression] = _canonical(expression)
    time_dict = kwargs.get("time_dict", None)
    requested = kwargs.get("format", kwargs.get("output_format", None))
    if canon == _SDDMM_EXPR and len(tensors) == 3 and requested is None:
        direct = _sddmm_direct(*tensors, time_dict)
        if direct is not None:
            return direct
    if canon in (_SPMM_EXPR, "ab,b->a") and len(tensors) == 2 and isinstance(tensors[0], STensor) \
            and isinstance(tensors[1], torch.Tensor) and tensors[1].dim() == (2 if canon == _SPMM_EXPR else 1):
        direct = _matmul_csr_dense_direct(tensors[0], tensors[1], kwargs)   # the same product as matmul's
        if direct is not None:
            return direct
    operands = tuple(STensor.from_torch(t) if isinstance(t, torch.Tensor) else t for t in tensors)

    if canon in (_SDDMM_EXPR, _SDDMM_EXPR_KJ) and len(operands) == 3:
        mask, A, B = operands
        if requested is not None and str(parse_format(requested)) != "o,o" \
                and str(parse_format(requested)) != str(mask.format):
            raise _not_prebuilt(f"SDDMM with output format {requested}")
        if canon == _SDDMM_EXPR_KJ:
            if not B.format.is_dense():
                raise _not_prebuilt("SDDMM with a sparse right operand")
            B = STensor.from_torch(B.to_torch().t().contiguous())
        result = _sddmm(mask, A, B, time_dict)
        if result is None:
            raise _not_prebuilt(f"einsum({expression!r}) with formats "
                                f"{[str(t.format) for t in operands]}")
        return result

    if canon == _SPMM_EXPR and len(operands) == 2:
        a, b = operands
        if a.format.is_dense() and b.format.is_dense():
            return torch.matmul(a.to_torch(in_place=False), b.to_torch(in_place=False))
        result = _run_prebuilt_matmul(a, b, requested, time_dict)
        if result is None:
            result = _run_converted_matmul(a, b, requested, time_dict)
        if result is None:
            raise _not_prebuilt(f"einsum({expression!r}) with formats {a.format} x {b.format}")
        return result.to_torch() if result.format.is_dense() else result

    if canon == "ab,b->a" and len(operands) == 2:
        a, b = operands
        result = _run_prebuilt_matmul(a, b, requested, time_dict)
        if result is None:
            result = _run_converted_matmul(a, b, requested, time_dict)
        if result is None:
            raise _not_prebuilt(f"einsum({expression!r}) with formats {a.format} x {b.format}")
        return result.to_torch() if result.format.is_dense() else result

    raise _not_prebuilt(f"einsum({expression!r})")


def spmv(a: STensor, b: STensor, output_format: Optional[Union[TensorFormat, str, List[str]]] = None,
         **kwargs: Any) -> STensor:
    """Sparse matrix times dense vector; an STensor in format "d", as the
    reference's function of this name returns (ops.py:48-136)."""
    if output_format is not None and not parse_format(output_format).is_dense():
        raise _not_prebuilt(f"spmv with output format {output_format}")
    time_dict = kwargs.get("time_dict", None)
    result = _run_prebuilt_matmul(a, b, None, time_dict)
    if result is None:
        result = _run_converted_matmul(a, b, None, time_dict)
    if result is None:
        raise _not_prebuilt(f"spmv({a.format} x {b.format}, {a.values.dtype})")
    return result


def matmul_wksp(a: Union[torch.Tensor, STensor], b: Union[torch.Tensor, STensor],
                output_format: Optional[Union[TensorFormat, str, List[str]]] = None,
                **kwargs: Any) -> STensor:
    """Matrix product of two sparse operands; torch tensors are made sparse
    first and the result is an STensor, "d,s" unless another format is asked for
    (reference: ops.py:139-245, a generated kernel with a row workspace; here
    the CSR x CSR kernel, which keeps a row's sums in LDS, does the work)."""
    if isinstance(a, torch.Tensor):
        a = STensor.from_torch(a).to_sparse()
    if isinstance(b, torch.Tensor):
        b = STensor.from_torch(b).to_sparse()
    fmt = parse_format("ds" if output_format is None else output_format)
    time_dict = kwargs.get("time_dict", None)
    result = _run_prebuilt_matmul(a, b, fmt, time_dict)
    if result is None:
        result = _run_converted_matmul(a, b, fmt, time_dict)
    if result is None:
        raise _not_prebuilt(f"matmul_wksp({a.format} x {b.format}, {a.values.dtype}, format={fmt})")
    return result


def precompile_kernels() -> None:
    """The reference generates and compiles its common matmul kernels ahead of
    use (ops.py:933-945).  Here they are built with the package; this loads
    the library so that a missing build shows up now and not at the first product."""
    from . import native
    native.lib()


def spmm_bias_act(a: STensor, b: Union[torch.Tensor, STensor], bias: torch.Tensor,
                  relu: bool = False) -> torch.Tensor:
    """``act(a @ b + bias)`` in one kernel: the call the reference's
    ``@scorch.compile`` makes when it recognises matmul -> add(bias) [-> relu]
    (src/scorch/trace.py:232-301).  Returns an (M, N) tensor."""
    kinds = ("add", "relu") if relu else ("add",)
    if isinstance(b, torch.Tensor) and b.layout == torch.strided and b.dim() == 2:
        # a dense torch operand is handed to the kernel as it is (no STensor around it)
        b_format, b_shape, b_index, b_values = "d,d", tuple(b.shape), [[], []], b.reshape(-1)
        if b_values is not b and b_values.data_ptr() == b.data_ptr():
            b_values._scorch_origin = b
    else:
        if isinstance(b, torch.Tensor):
            b = STensor.from_torch(b)
        b_format, b_shape, b_index, b_values = str(b.format), tuple(b.shape), b.index.mode_indices, b.values
    key = (str(a.format), b_format, kinds, a.values.dtype)
    fn = _direct_fused.get(key)
    if fn is None:
        resolved = resolve_prebuilt_fused(key[0], b_format, kinds, a.values.dtype)
        if resolved is None:
            raise _not_prebuilt(f"fused matmul+{'+'.join(kinds)} for {a.format} x {b_format}, {a.values.dtype}")
        fn = _direct_fused[key] = resolved.fn
    if b_values.dtype != a.values.dtype:
        raise _not_prebuilt(f"fused matmul+{'+'.join(kinds)} for {a.values.dtype} x {b_values.dtype}")
    for values in (a.values, b_values):
        if not values.is_cuda:
            raise _not_on_device(values.device)
    M, N = a.shape[0], b_shape[1]
    out = fn((M, N), a.shape, a.index.mode_indices, a.values, b_shape, b_index, b_values, bias)
    return out.storage.value.view(M, N)
