import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_PATH = os.path.join(ROOT, "tests", "golden", "golden_ref.npz")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    """GPU tests skip cleanly where there is no device."""
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def poisoned_device_buffers(request, monkeypatch):
    """Every GPU test runs with the package's fresh device buffers (results, workspaces, plans)
    filled with NaN (floating point) or 0x7f bytes (everything else) before a kernel sees them:
    a kernel that read memory it had not been given, or left part of a result unwritten, would
    show here and not only when recycled memory happens to hold something harmful."""
    if "gpu" not in request.keywords:
        return
    import torch
    from scorch_amd import scorch_ops_hip as H

    def poison(t):
        if t.is_cuda and t.numel():
            if t.dtype.is_floating_point:
                t.fill_(float("nan"))
            else:
                t.view(torch.uint8).fill_(0x7F)
        return t

    monkeypatch.setattr(H, "_empty", lambda *a, **k: poison(torch.empty(*a, **k)))
    monkeypatch.setattr(H, "_empty_like", lambda *a, **k: poison(torch.empty_like(*a, **k)))


class Golden:
    """Cases of tests/golden/golden_ref.npz: golden.case("spmm_rect") -> dict of arrays."""

    def __init__(self, path):
        self._z = np.load(path, allow_pickle=False)
        self.names = sorted({k.split("/")[0] for k in self._z.files})

    def case(self, name):
        prefix = name + "/"
        out = {k[len(prefix):]: self._z[k] for k in self._z.files if k.startswith(prefix)}
        if not out:
            raise KeyError(name)
        return out

    def cases(self, prefix):
        return [n for n in self.names if n.startswith(prefix)]


@pytest.fixture(scope="session")
def golden():
    return Golden(GOLDEN_PATH)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    return O


def random_csr(rng, M, K, density, dtype=np.float32, empty_rows=(), lo=-1.0, hi=1.0):
    """Random CSR pattern with sorted unique columns; returns (row_ptr, col_idx, vals)."""
    keep = rng.random((M, K)) < density
    for r in empty_rows:
        keep[r, :] = False
    rows, cols = np.nonzero(keep)
    row_ptr = np.zeros(M + 1, dtype=np.int32)
    np.cumsum(np.bincount(rows, minlength=M), out=row_ptr[1:])
    if np.issubdtype(np.dtype(dtype), np.integer):
        vals = rng.integers(-1000, 1000, size=rows.size).astype(dtype)
    else:
        vals = rng.uniform(lo, hi, size=rows.size).astype(dtype)
    return row_ptr, cols.astype(np.int32), vals
