"""scorch_amd: Scorch's prebuilt CSR sparse x dense kernels (SpMM, SDDMM and
their neighbours) as hand-written HIP for AMD MI355X, behind Scorch's own
``matmul`` / ``einsum`` / ``STensor`` interface.

    import scorch_amd as scorch
    A = scorch.from_csr(torch_csr).to("cuda")
    C = scorch.matmul(A, B_cuda)                       # CSR x dense -> dense
    S = scorch.einsum("ij,ik,jk->ij", mask, Q, K)      # SDDMM
"""
from .format import LevelFormat, LevelType, TensorFormat, parse_format
from .stensor import STensor
from .storage import TensorIndex, TensorStorage
from .ops import einsum, matmul, matmul_wksp, precompile_kernels, spmm_bias_act, spmv
from .trace import compile

from_torch = STensor.from_torch
from_coo = STensor.from_coo
from_csr = STensor.from_csr



def __getattr__(name):
    """Names this package does not define resolve to torch's, as in the reference
    (src/scorch/__init__.py:14-18): ``scorch.float32``, ``scorch.rand(...)``."""
    import importlib
    import importlib.util
    import torch
    if not name.startswith("_") and importlib.util.find_spec(f"{__name__}.{name}") is not None:
        return importlib.import_module(f"{__name__}.{name}")    # a submodule not imported yet
    try:
        return getattr(torch, name)
    except AttributeError:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}") from None


__version__ = "0.1.0"

__all__ = ["STensor", "TensorFormat", "TensorIndex", "TensorStorage", "LevelFormat", "LevelType",
           "parse_format", "compile", "einsum", "matmul", "matmul_wksp", "precompile_kernels", "spmm_bias_act", "spmv", "from_torch", "from_coo", "from_csr",
           "__version__"]
