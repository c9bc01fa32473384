"""A step of this package's calls recorded once as a HIP graph and replayed.

Every entry point of libscorch_hip only enqueues kernels on the caller's stream,
so a sequence of calls (the layers of a small GCN, the heads of an attention
block) can be captured with torch's graph support and replayed with one launch
instead of one per kernel plus the Python in between -- which is what a step on
a small operand is made of: the product of a 4,096 x 4,096 matrix takes the GPU
6 us and the host 8 to 18.

What has to happen before the capture, and what ``capture`` therefore does:
plans (index inspection, chunk boundaries, tiled copies, entry lists, block
masks) are built on an operand's first or second use and need a
synchronisation, which a capturing stream does not allow; the step is run
eagerly on a side stream first, ``warmup`` times, so that they exist.  The plans
of a sparse operand's index arrays (and of an attention mask) become part of the
recording: values may be rewritten in place between replays, index arrays may
not.  Nothing derived from an operand's *values* is recorded (the column-tile
copy of a wide dense operand, the verdict that a mask's values are all 1): a
recorded product runs from the operand itself and reads every value array it
was given.

A replay writes the results, and whatever the caller copied into the static
inputs arrived there, without PyTorch's version counters necessarily noticing.
``capture`` therefore marks the static inputs and the results volatile
(scorch_ops_hip.mark_volatile: eager calls that take them as operands keep
nothing derived from their values), and every replay bumps the results' version
counters, so that data other code derived from them is seen to be stale.

The reference has no counterpart: its kernels run on the host.
"""
from __future__ import annotations

from typing import Any, Callable

import torch

from . import scorch_ops_hip


class CapturedStep:
    """``fn(*args)`` as a replayable graph.  ``args`` are the static inputs: write new data
    into those tensors (``copy_``) and call ``replay()`` (or the object itself); the result is
    the same tensor object or structure on every replay, overwritten in place."""

    def __init__(self, fn: Callable[..., Any], *args: Any, warmup: int = 2):
        if not torch.cuda.is_available():
            raise RuntimeError("scorch_amd.graphs: no GPU")
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("scorch_amd.graphs: capture() called while the stream is already capturing")
        self.args = args
        scorch_ops_hip.mark_volatile(args)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(int(warmup), 2)):     # twice at least: some plans are built on the second use
                fn(*args)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.result = fn(*args)
        self._result_tensors = list(scorch_ops_hip._tensors_of(self.result))
        scorch_ops_hip.mark_volatile(self._result_tensors)

    def replay(self) -> Any:
        self.graph.replay()
        if self._result_tensors:
            # the replay has rewritten them in place behind the version counters' back
            torch.autograd.graph.increment_version(self._result_tensors)
        return self.result

    __call__ = replay


def capture(fn: Callable[..., Any], *args: Any, warmup: int = 2) -> CapturedStep:
    """Record ``fn(*args)`` as a HIP graph (see CapturedStep)."""
    return CapturedStep(fn, *args, warmup=warmup)
