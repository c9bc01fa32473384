"""Benchmark of the CSR sparse x dense kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--workload NAME]

With no --workload the line is the headline: CSR SpMM, fp32, on the GCN-style
power-law graph (1,048,576 nodes, N = 128 features), W untimed warm-up steps and
then exactly K timed steps between two device synchronisations.  A step is one
C = A @ B through the C ABI of libscorch_hip.so with A and B resident in HBM (the
output buffer comes from torch's caching allocator).  `value` is whole-job
GFLOP/s (2 * nnz * N flops per step, the reference's convention,
tools/benchmark_spmm_variants.py:127-129).  The same line carries, under
"configs", one record for each of the other four benchmark configurations
(SpMM 4096^2, SDDMM 65,536^2, fused block-sparse attention, the
sparse-autoencoder decoder), every one with the roofline of its dominant kernel
and the reference's CPU path timed on this host.  --workload NAME prints that
workload's record alone.

Per-kernel durations are measured in this process with HIP events on the launch
stream (scorch_hip_timing_begin / _end); what is computed once per operand
(index inspection, chunk boundaries, the column-tile copy of a reused dense
operand) happens in the warm-up calls, whose wall times are listed in
"warmup_ms".
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published
HEADLINE = "gcn_powerlaw"
CONFIG_WORKLOADS = ("spmm_uniform", "sddmm_uniform", "attention_blocksparse", "sae_decoder")

# Bytes through the L2-to-fabric boundary per launch of each configuration's
# dominant kernel at its default size: FETCH_SIZE (KiB, x 2.0: the factor a
# 1 GiB device copy gives for this counter on gfx950) + WRITE_SIZE (KiB, x 1.0)
# from two rocprofv3 --pmc runs of `python3 bench.py --workload NAME --no-cpu`
# (the factors are what the same counters read for a copy of known size,
# profiles/copy_calibration.md).  A measured constant holds for the default size
# and for the kernel as its source files stood when it was measured: "sha16" is
# the hash of those files then (source_hash below; `python bench.py
# --source-hashes` prints the current ones), and a record whose files have
# changed since reports "traffic": null until it is measured again.
_CSRC = "scorch_amd/csrc/"
_SPMM_SOURCES = (_CSRC + "spmm.hip", _CSRC + "spmm.hpp", _CSRC + "common.hpp")
MEASURED_TRAFFIC = {
    ("gcn_powerlaw", "merge"): {"bytes": 9_790_300_000, "sources": _SPMM_SOURCES, "sha16": "f03cdf8f7d11457c",
                                "profile": "profiles/spmm_merge_kernel_gcn_powerlaw.md"},
    ("spmm_uniform", "rows"): {"bytes": 10_830_000, "sources": (_CSRC + "spmm_rows.hip", _CSRC + "spmm.hpp",
                                                                _CSRC + "common.hpp"), "sha16": "36b7f160411c76eb",
                               "profile": "profiles/spmm_rows_kernel_uniform_4096.md"},
    ("sae_decoder", "tiled"): {"bytes": 344_100_000, "sources": (_CSRC + "spmm_tiled.hip", _CSRC + "spmm.hpp",
                                                                 _CSRC + "common.hpp"), "sha16": "ea9b5c43570e7930",
                               "profile": "profiles/spmm_tiled_kernel_sae_decoder.md"},
    ("sae_decoder", "merge"): {"bytes": 1_767_900_000, "sources": _SPMM_SOURCES, "sha16": "f03cdf8f7d11457c",
                               "profile": "profiles/spmm_tiled_kernel_sae_decoder.md"},
    ("sddmm_uniform", "listed"): {"bytes": 278_000_000, "sources": (_CSRC + "sddmm.hip", _CSRC + "common.hpp"),
                                  "sha16": "eed3747508604c18", "profile": "profiles/sddmm_kernels_uniform_65536.md"},
    ("sddmm_uniform", "plain"): {"bytes": 848_200_000, "sources": (_CSRC + "sddmm.hip", _CSRC + "common.hpp"),
                                 "sha16": "eed3747508604c18", "profile": "profiles/sddmm_kernels_uniform_65536.md"},
    ("attention_blocksparse", "fused"): {"bytes": 81_050_000, "sources": (_CSRC + "attn.hip", _CSRC + "common.hpp"),
                                         "sha16": "1c42d31b5c08e253", "profile": "profiles/attn_blocksparse_kernel_s8192_h16.md"},
}


def source_hash(files):
    """First 16 hex digits of the SHA-256 over the named files' bytes, in order."""
    import hashlib
    h = hashlib.sha256()
    for f in files:
        with open(os.path.join(ROOT, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def measured_traffic(name, path, default_size):
    rec = MEASURED_TRAFFIC.get((name, path))
    if rec is None or not default_size:
        return None, None
    if source_hash(rec["sources"]) != rec["sha16"]:
        return None, {"profile": rec["profile"], "stale": "the kernel's source files have changed since the "
                                                          "counters were read"}
    return rec["bytes"], {"sha16": rec["sha16"], "profile": rec["profile"]}


def spmm_algorithmic_bytes(M, K, N, nnz):
    """Every array touched once: col_idx + vals, row_ptr, B, C (fp32 / int32)."""
    return 8 * nnz + 4 * (M + 1) + 4 * K * N + 4 * M * N


def spmm_gather_bytes(M, N, nnz):
    """No-reuse model: a B row re-read for every nonzero."""
    return 8 * nnz + 4 * (M + 1) + 4 * nnz * N + 4 * M * N


# ---- CPU baselines: the reference's own kernels (oracle/_ref) on the host cores ------------------
# Protocol of the reference's benchmarks (bench/_utils.py:295-310): 3 warm-up calls, 10 timed,
# median.  Two figures where they differ: the kernel's loop alone, and the call as the reference's
# dispatch times it (src/scorch/prebuilt_kernels.py:217-222: the whole native call, which for SpMM
# allocates and zero-fills the result, csrc/spmm.h:2024-2025).
CPU_WARMUP, CPU_REPEATS = 3, 10


def _timed_calls(fn, repeats=CPU_REPEATS, warmup=CPU_WARMUP):
    times = []
    for i in range(warmup + repeats):
        t0 = time.perf_counter()
        out = fn()
        dt = time.perf_counter() - t0
        del out
        if i >= warmup:
            times.append(dt)
    return statistics.median(times)


_PROTOCOL = f"median of {CPU_REPEATS} calls after {CPU_WARMUP} warm-up calls"


def cpu_baseline_spmm(w):
    """Two timings on the host cores and the same inputs.  as_reference_times_it_ms: the
    reference's spmm_csr_float_v2 itself (oracle/_ref, compiled from the reference's sources;
    this repository's C restatement of it where that module is absent or this host cannot run
    it), the whole native call -- it allocates and zero-fills C.  kernel_only_ms: the
    restatement's loop into a result that is already allocated and zeroed (the compiled reference
    cannot be entered past its allocation).  `value` is computed from the first."""
    import numpy as np
    from oracle import oracle as O
    M, N, nnz = w["M"], w["N"], int(w["col_idx"].size)
    kind, whole = "port", None
    if O.have_ref():
        try:
            import torch
            mod = O.ref_module()
            pos, crd = torch.from_numpy(w["row_ptr"]), torch.from_numpy(w["col_idx"])
            val, Bf = torch.from_numpy(w["vals"]), torch.from_numpy(w["B"]).reshape(-1)
            args = ([M, N], [M, w["K"]], [[], [pos, crd]], val, [w["K"], N], [[], []], Bf)
            whole = _timed_calls(lambda: mod.spmm_csr_float_v2(*args))
            kind = "reference"
        except Exception as exc:  # module built against another torch
            print(f"[bench] reference module unusable here ({exc}); timing the C restatement", file=sys.stderr)
    if whole is None:
        whole = _timed_calls(lambda: O.spmm_csr_f32_v2(w["row_ptr"], w["col_idx"], w["vals"], w["B"]))
    out = np.zeros((M, N), dtype=np.float32)

    def loop_only():
        O.spmm_csr_f32_v2(w["row_ptr"], w["col_idx"], w["vals"], w["B"], out=out, zero_fill=False)

    loop = _timed_calls(loop_only)
    return {"value": round(2.0 * nnz * N / whole / 1e9, 3), "unit": "GFLOP/s", "cores": O.num_threads(),
            "kind": kind, "ms_per_step": round(whole * 1e3, 3),
            "as_reference_times_it_ms": round(whole * 1e3, 3), "kernel_only_ms": round(loop * 1e3, 3),
            "kernel_only_kind": "port",
            "sample": f"full workload (M={M}, nnz={nnz}, N={N}), {_PROTOCOL}; as_reference_times_it_ms: the "
                      "whole native call incl. allocating and zeroing C; kernel_only_ms: the restatement's "
                      "loop into a result allocated and zeroed beforehand"}


def cpu_baseline_sddmm(w):
    """The reference's sddmm_coo_float_prebuilt (oracle/_ref) or the C restatement of it, on the
    host cores, coordinate mask, same inputs: the whole call as the reference's dispatch times it
    (it allocates the result's values), and the restatement's loop alone."""
    from oracle import oracle as O
    nnz, K = int(w["col_idx"].size), w["K"]
    kind = "reference" if O.have_ref() else "port"

    def ref():
        return O.ref_sddmm_coo(w["row_idx"], w["col_idx"], w["vals"], w["A"], w["B"], (w["M"], w["n_cols"]))

    def port():
        return O.sddmm_coo_f32(w["row_idx"], w["col_idx"], w["vals"], w["A"], w["B"])

    try:
        whole = _timed_calls(ref if kind == "reference" else port)
    except Exception as exc:  # module built against another torch
        if kind == "port":
            raise
        print(f"[bench] reference module unusable here ({exc}); timing the C restatement", file=sys.stderr)
        kind, whole = "port", _timed_calls(port)
    loop = whole if kind == "port" else _timed_calls(port)
    return {"value": round((2.0 * nnz * K + nnz) / whole / 1e9, 3), "unit": "GFLOP/s", "cores": O.num_threads(),
            "kind": kind, "ms_per_step": round(whole * 1e3, 3),
            "as_reference_times_it_ms": round(whole * 1e3, 3), "kernel_only_ms": round(loop * 1e3, 3),
            "kernel_only_kind": "port",
            "sample": f"full workload (nnz={nnz}, K={K}), {_PROTOCOL}; as_reference_times_it_ms incl. wrapping "
                      "the operands and copying the result's index arrays; kernel_only_ms: the restatement's "
                      "loop with its result array"}


def cpu_baseline_attention(w, heads=4, pattern=None):
    """The per-head composition of the reference's attention benchmark
    (bench/bench_sparse_transformer.py:354-372) on the host cores, fp32, for a
    sample of the heads: its SDDMM and SpMM kernels (oracle/_ref, or the C
    restatements where that module is absent) with the CSR row softmax between
    them (the oracle's C restatement of the benchmark's torch composition)."""
    import numpy as np
    from oracle import oracle as O
    from scorch_amd import workloads
    S, D, H = w["S"], w["D"], w["H"]
    pos, crd = pattern if pattern is not None else workloads.blocks_to_csr(w["block_row_ptr"], w["block_col_idx"],
                                                                          w["block"])
    rows = np.repeat(np.arange(S, dtype=np.int32), np.diff(pos))
    ones = np.ones(crd.size, np.float32)
    kind = "reference" if O.have_ref() else "port"

    def head(h, use_ref):
        q, k, v = (np.ascontiguousarray(w[n][h]) for n in ("q", "k", "v"))
        if use_ref:
            s = O.ref_sddmm_coo(rows, crd, ones, q, k, (S, S))[2]
            p = O.softmax_csr_f32(pos, s, float(w["scale"]))
            return O.ref_spmm("spmm_csr_float_v2", pos, crd, p, v)
        s = O.sddmm_coo_f32(rows, crd, ones, q, k)
        p = O.softmax_csr_f32(pos, s, float(w["scale"]))
        return O.spmm_csr_f32_v2(pos, crd, p, v)

    try:
        head(0, kind == "reference")
    except Exception as exc:
        if kind == "port":
            raise
        print(f"[bench] reference module unusable here ({exc}); timing the C restatements", file=sys.stderr)
        kind = "port"
        head(0, False)
    times = []
    for h in range(heads):
        t0 = time.perf_counter()
        head(h, kind == "reference")
        times.append(time.perf_counter() - t0)
    per_head = statistics.median(times)
    nnz = int(crd.size)
    return {"value": round(4.0 * nnz * D / per_head / 1e12, 4), "unit": "TFLOP/s", "cores": O.num_threads(),
            "kind": kind, "ms_per_step": round(per_head * H * 1e3, 1),
            "as_reference_times_it_ms": round(per_head * H * 1e3, 1),
            "sample": f"{heads} of {H} heads after 1 warm-up head (nnz per head {nnz}), median; ms_per_step is the "
                      f"per-head time x {H}; SDDMM -> row softmax -> SpMM per head in fp32, each product the whole "
                      "native call as the reference times it; the softmax leg is the oracle's C restatement of "
                      "the benchmark's torch ops"}


# ---- device timing ----------------------------------------------------------------------------
_blocker = None


def _time_steps(fn, steps, warmup, rounds=3, min_round_ms=4.0):
    """GPU time per step of `fn`, HIP events on torch's current stream (the
    stream the kernels are launched on).  A few large device fills are queued
    first, so that the step launches are all enqueued before the GPU reaches the
    first of them: the interval is then the GPU's time for the steps, not the
    host's time to issue them.  Median of `rounds` such measurements.  A round of
    `steps` steps that lasts less than `min_round_ms` is a pilot only: the rounds
    that count then repeat the step until they last that long (a burst of a
    millisecond is over before the GPU's clocks have settled), with as many fills
    in front as the host needs to enqueue them."""
    import torch
    global _blocker
    if _blocker is None:
        _blocker = torch.empty(1 << 28, dtype=torch.float32, device="cuda")
    for _ in range(warmup):
        fn()

    def one_round(n):
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(3 + int(n * 0.012 / 0.15)):  # ~12 us of host time per call, ~0.15 ms per fill
            _blocker.fill_(1.0)
        start.record()
        for _ in range(n):
            fn()
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / n

    results = [one_round(steps)]
    n = steps
    if results[0] * steps < min_round_ms:
        n = min(int(min_round_ms / max(results[0], 1e-6)) + 1, 200 * steps)
        results = []
    while len(results) < rounds:
        results.append(one_round(n))
    global _last_timing
    _last_timing = {"steps": n, "rounds": len(results)}
    return statistics.median(results)


_last_timing = {"steps": 0, "rounds": 0}


def _timed_as():
    """How the last _time_steps call was timed: steps per round and rounds (median taken)."""
    return dict(_last_timing)


def _kernel_times(fn, samples):
    """Average duration (ms) of each kernel `fn` launches, in launch order: HIP events that the
    library records on the kernels' stream before, between and after them.  A kernel that only
    spins (no memory traffic, so the caches stay as the timed steps left them) is queued in front
    of every sample, so that the events and the kernels between them are all enqueued before the
    GPU reaches the first: an interval is then the kernel's time, without the host's time to
    issue it, which for a kernel of a few microseconds would be most of the figure."""
    import torch
    from scorch_amd import native

    def sample():
        torch.cuda._sleep(80_000)       # about 40 us
        fn()
    rows = [native.kernel_times(sample) for _ in range(samples)]
    width = min(len(r) for r in rows)
    return [sum(r[i] for r in rows) / len(rows) for i in range(width)]


def _warmup_calls(fn, warmup):
    """The warm-up calls one by one with their wall time (ms): the first builds
    whatever is computed once per operand."""
    import torch
    out = []
    for _ in range(warmup):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        out.append(round((time.perf_counter() - t0) * 1e3, 3))
    return out


def _vendor_time(call_name, fn, steps, warmup):
    """Times a torch routine on the same operands; an error becomes a field."""
    try:
        return {"call": call_name, "ms_per_step": round(_time_steps(fn, steps, warmup, rounds=1), 4)}
    except RuntimeError as err:
        return {"call": call_name, "error": str(err).splitlines()[0]}


def _hbm_roofline(kernel, kernel_ms, algo, traffic, provenance, extra=None):
    achieved = algo / (kernel_ms * 1e-3) / 1e9
    out = {"bound": "hbm", "kernel": kernel, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
           "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic, "algorithmic_bytes": algo,
           "kernel_ms_avg": round(kernel_ms, 5)}
    if provenance:
        out["traffic_measured_at"] = provenance
    if traffic is not None:
        # what the memory system moved per second for this kernel: the distance to the HBM peak that
        # remains once the re-reads the access pattern forces are counted
        out["traffic_gbps"] = round(traffic / (kernel_ms * 1e-3) / 1e9, 1)
    if extra:
        out.update(extra)
    return out


def _t(a):
    import numpy as np
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


# ---- the benchmark configurations ----------------------------------------------------------------
def run_spmm(name, args, headline=False):
    """CSR SpMM fp32: gcn_powerlaw (the headline), spmm_uniform, sae_decoder."""
    import torch
    from scorch_amd import scorch_ops_hip as H
    from scorch_amd import workloads
    t0 = time.time()
    if name == "gcn_powerlaw":
        w = workloads.gcn_powerlaw(M=args.rows, N=args.features, window=args.window)
        default_size = (args.rows, args.features, args.window) == (1 << 20, 128, 0)
    elif name == "spmm_uniform":
        w, default_size = workloads.spmm_uniform(), True
    else:
        w, default_size = workloads.sae_decoder(), True
    M, K, N, nnz = w["M"], w["K"], w["N"], int(w["col_idx"].size)
    print(f"[bench] generated {name}: M={M} K={K} nnz={nnz} N={N} in {time.time() - t0:.1f}s", file=sys.stderr)
    pos, crd, val, B = _t(w["row_ptr"]), _t(w["col_idx"]), _t(w["vals"]), _t(w["B"]).reshape(-1)
    call = ([M, N], [M, K], [[], [pos, crd]], val, [K, N], [[], []], B)
    fn = lambda: H.spmm_csr_float_v2(*call)

    warm = _warmup_calls(fn, args.warmup)
    if headline:
        # the contract's timed region: exactly K steps between two synchronisations, wall clock
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t_begin = time.perf_counter()
        start.record()
        for _ in range(args.steps):
            fn()
        stop.record()
        torch.cuda.synchronize()
        ms_per_step = (time.perf_counter() - t_begin) * 1e3 / args.steps
        event_ms = start.elapsed_time(stop) / args.steps
        timed = {"steps": args.steps, "rounds": 1}
    else:
        ms_per_step = event_ms = _time_steps(fn, args.steps, 0)
        timed = _timed_as()

    tiled = getattr(B, "_scorch_tiled", None) is not None
    plan = getattr(pos, "_scorch_plan", None)
    kernels = _kernel_times(fn, min(args.steps, 10))
    if tiled:
        path, names = "tiled", ["spmm_tiled_kernel<float,0>", "spmm_fixup_kernel<float,1,0>"]
    elif len(kernels) == 1:
        lanes = 64 if N % 4 else max(8, min(64, 1 << (max(N // 4, 1) - 1).bit_length()))
        path, names = "rows", [f"spmm_rows_kernel<float,{4 if N % 4 == 0 else 1},{lanes}>"]
    else:
        vec = 4 if N % 256 == 0 else 2 if N % 128 == 0 else 1
        path = "merge"
        names = [f"spmm_merge_kernel<float,{vec},0>" if N * 4 > 256 else "spmm_grouped_kernel<float,...>",
                 "spmm_fixup_kernel<float,...>"]
    dominant = max(range(len(kernels)), key=lambda i: kernels[i])
    # the named kernel's own duration: HIP events around its launch (a spin kernel queued in front
    # keeps the host's issue time out of it).  It still holds the dispatch of a launch that follows
    # an event, 2 to 3 us, which back-to-back launches hide and a profiler's kernel trace leaves
    # out: for a kernel of 5 us the figure is on the high side, the fraction on the low side.
    # kernel_ms_queued is the kernel's share of the time per step between the two events around
    # the timed region, where launches overlap each other's start and end.
    kernel_ms = kernels[dominant]
    queued_ms = event_ms * kernels[dominant] / sum(kernels)

    flops = 2.0 * nnz * N
    algo, gather = spmm_algorithmic_bytes(M, K, N, nnz), spmm_gather_bytes(M, N, nnz)
    traffic, provenance = measured_traffic(name, path, default_size)
    rec = {
        "metric": "CSR SpMM GFLOP/s + HBM GB/s (% peak), power-law 1M rows, N=128 fp32" if headline
                  else "CSR SpMM GFLOP/s",
        "value": round(flops / (ms_per_step * 1e-3) / 1e9, 2), "unit": "GFLOP/s",
        "n_gpus": 1, "steps": timed["steps"], "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "timed_rounds": timed["rounds"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": name + "_spmm_fp32" if name == "gcn_powerlaw" else name + "_fp32",
                   "rows": M, "cols": K, "nnz": nnz, "features": N,
                   "seed": workloads.SEEDS[name]},
        "warmup_ms": warm,
        "path": path,
        "longest_row": plan.max_row if plan is not None else None,
        "kernels_ms": {n: round(k, 5) for n, k in zip(names, kernels)},
        "event_ms_per_step": round(event_ms, 5),
        "hbm_gbps_algorithmic": round(algo / (ms_per_step * 1e-3) / 1e9, 1),
        "roofline": _hbm_roofline(names[dominant], kernel_ms, algo, traffic, provenance,
                                  {"kernel_ms_queued": round(queued_ms, 5),
                                   "gather_model_bytes": gather,
                                   "gather_model_gbps": round(gather / (kernel_ms * 1e-3) / 1e9, 1)}),
    }
    if name == "gcn_powerlaw":
        rec["config"].update({"degree": "zipf(2.1), mean 16 after the cap of 50000, distinct neighbours, + self-loops",
                              "values": "D^-1/2 (A+I) D^-1/2"})
        if args.window:
            rec["config"]["neighbour_window"] = args.window
    if not headline:
        # the same product through the C ABI's plan handles alone (what a C++ host of the reference would
        # call: one object per operand, one call per product, no Python-side plans)
        from scorch_amd.csr_plan import CsrPlanHandle, DensePlanHandle
        B2d = B.reshape(K, N)
        with CsrPlanHandle(pos, crd, K) as handle, DensePlanHandle(B2d) as dense:
            planned = (lambda: handle.spmm_dense(val, dense)) if tiled else (lambda: handle.spmm(val, B2d))
            rec["ms_per_step_plan_handle"] = round(_time_steps(planned, args.steps, 2), 5)
            torch.cuda.synchronize()
    if args.graph and not headline:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        rec["ms_per_step_graph_replay"] = round(_time_steps(graph.replay, args.steps, 2), 5)
    if args.vendor:
        A_t = torch.sparse_csr_tensor(pos, crd, val, size=(M, K))
        B2 = B.reshape(K, N)
        rec["vendor_library"] = _vendor_time("torch.sparse.mm(csr, dense)", lambda: torch.sparse.mm(A_t, B2),
                                             max(args.steps // 2, 2), 1)
    if not args.no_cpu:
        rec["cpu_baseline"] = cpu_baseline_spmm(w)
    return rec


def run_sddmm(args):
    import torch
    from scorch_amd import scorch_ops_hip as H
    from scorch_amd import workloads
    w = workloads.sddmm_uniform()
    M, n_cols, K, nnz = w["M"], w["n_cols"], w["K"], int(w["col_idx"].size)
    pos, crd, val, A, B = _t(w["row_ptr"]), _t(w["col_idx"]), _t(w["vals"]), _t(w["A"]), _t(w["B"])
    rows = _t(w["row_idx"])
    Af, Bf = A.reshape(-1), B.reshape(-1)
    csr = lambda: H.sddmm_csr_float([M, n_cols], [M, n_cols], [[], [pos, crd]], val, [M, K], [[], []], Af,
                                    [n_cols, K], [[], []], Bf)
    coo = lambda: H.sddmm_coo_float_prebuilt([M, n_cols], [M, n_cols], [[rows], [crd]], val, [M, K], [[], []], Af,
                                             [n_cols, K], [[], []], Bf)
    warm = _warmup_calls(csr, args.warmup)
    ms = _time_steps(csr, args.steps, 0)
    timed = _timed_as()
    kernel_ms = max(_kernel_times(csr, min(args.steps, 10)))   # HIP events around the launch (see run_spmm)
    ms_coo = _time_steps(coo, args.steps, 2)
    flops = 2.0 * nnz * K + nnz
    # every array once: row_ptr, col_idx, mask values, A, B, result values; the CSR-mask kernel
    # also writes the result's row coordinates, 4 more bytes per entry (not counted)
    algo = 4 * (M + 1) + 4 * nnz * 3 + 4 * M * K + 4 * n_cols * K
    gather = algo - 4 * n_cols * K + 4 * nnz * K
    plan = getattr(pos, "_scorch_plan", None)
    listed = plan is not None and plan.sddmm_lists is not None
    traffic, provenance = measured_traffic("sddmm_uniform", "listed" if listed else "plain", True)
    rec = {"metric": "CSR SDDMM GFLOP/s", "value": round(flops / ms / 1e6, 2), "unit": "GFLOP/s",
           "n_gpus": 1, "steps": timed["steps"], "timed_rounds": timed["rounds"], "warmup": args.warmup,
           "ms_per_step": round(ms, 5),
           "ms_per_step_coo_mask": round(ms_coo, 5), "higher_is_better": True, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "sddmm_uniform_fp32", "rows": M, "cols": n_cols, "nnz": nnz, "K": K,
                      "seed": workloads.SEEDS["sddmm_uniform"]},
           "warmup_ms": warm,
           "path": "listed" if listed else "plain",
           "roofline": _hbm_roofline("sddmm_listed_kernel<16,4>" if listed else "sddmm_kernel<16,4,false,false>",
                                     kernel_ms, algo, traffic, provenance,
                                     {"kernel_ms_queued": round(ms, 5),
                                      "row_coordinate_output_bytes": 4 * nnz, "gather_model_bytes": gather,
                                      "gather_model_gbps": round(gather / kernel_ms / 1e6, 1)})}
    if args.vendor:
        mask = torch.sparse_csr_tensor(pos, crd, val, size=(M, n_cols))
        Bt = B.t().contiguous()
        rec["vendor_library"] = _vendor_time("torch.sparse.sampled_addmm(mask, A, B^T, beta=0)",
                                             lambda: torch.sparse.sampled_addmm(mask, A, Bt, beta=0.0),
                                             max(args.steps // 2, 2), 1)
    if not args.no_cpu:
        rec["cpu_baseline"] = cpu_baseline_sddmm(w)
    return rec


def run_attention(args):
    import numpy as np
    import torch
    from scorch_amd import scorch_ops_hip as H
    from scorch_amd import workloads
    w = workloads.attention_blocksparse()
    Hh, S, D = w["H"], w["S"], w["D"]
    q, k, v = (_t(w[n]).to(torch.bfloat16) for n in ("q", "k", "v"))
    brp, bci = _t(w["block_row_ptr"]), _t(w["block_col_idx"])
    nnz = int(w["block_col_idx"].size) * w["block"] ** 2
    fn = lambda: H.attn_blocksparse_bf16(q, k, v, brp, bci, float(w["scale"]))
    warm = _warmup_calls(fn, args.warmup)
    ms = _time_steps(fn, args.steps, 0)
    timed = _timed_as()
    kernel_ms = max(_kernel_times(fn, min(args.steps, 10)))    # HIP events around the launch (see run_spmm)
    flops = 4.0 * nnz * D * Hh
    algo = 4 * Hh * S * D * 2 + 4 * (brp.numel() + bci.numel())
    achieved = flops / ms / 1e9
    kernel_achieved = flops / kernel_ms / 1e9
    traffic, provenance = measured_traffic("attention_blocksparse", "fused", True)
    rec = {"metric": "fused block-sparse attention TFLOP/s", "value": round(achieved, 2), "unit": "TFLOP/s",
           "n_gpus": 1, "steps": timed["steps"], "timed_rounds": timed["rounds"], "warmup": args.warmup,
           "ms_per_step": round(ms, 5),
           "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "attention_blocksparse_bf16", "S": S, "H": Hh, "D": D, "block": w["block"],
                      "active_blocks": int(bci.numel()), "nnz_per_head": nnz,
                      "seed": workloads.SEEDS["attention_blocksparse"]},
           "warmup_ms": warm,
           "roofline": {"bound": "mfma", "kernel": "attn_blocksparse_kernel<64, false, false>",
                        "achieved": round(kernel_achieved, 1),
                        "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": round(kernel_achieved / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": traffic,
                        "flops": flops, "algorithmic_bytes": algo, "kernel_ms_avg": round(kernel_ms, 5),
                        "kernel_ms_queued": round(ms, 5),
                        "hbm_gbps_algorithmic": round(algo / kernel_ms / 1e6, 1),
                        **({"traffic_measured_at": provenance} if provenance else {})}}
    # the same attention at the reference's precision: fp32 operands, probabilities and sums, one kernel
    q32, k32, v32 = q.float(), k.float(), v.float()
    bm32 = H.BlockMask(S, w["block"], brp, bci, None, None, nnz)
    ms32 = _time_steps(lambda: H.attn_blocksparse_f32(q32, k32, v32, bm32, float(w["scale"])), max(args.steps // 2, 2), 2)
    rec["fused_fp32"] = {"kernel": "attn32::attn_f32_kernel<64>", "ms_per_step": round(ms32, 5),
                         "tflops": round(flops / ms32 / 1e9, 1), "peak_tflops_fp32_matrix": 157.3,
                         "frac": round(flops / ms32 / 1e9 / 157.3, 4)}
    # (a) the composition the reference's benchmark uses, in fp32, on this package's own kernels:
    # SDDMM -> row softmax -> SpMM over the mask as a CSR operand (bench_sparse_transformer.py:354-372),
    # one launch each for all heads; the two products go to the block kernels (this mask is made of
    # whole 64 x 64 blocks)
    pos_np, crd_np = workloads.blocks_to_csr(w["block_row_ptr"], w["block_col_idx"], w["block"])
    pos, crd = _t(pos_np), _t(crd_np)

    def unfused():
        return H.sparse_attention_csr(pos, crd, q32, k32, v32, float(w["scale"]))

    rec["unfused_fp32_pipeline"] = _vendor_time("SDDMM -> softmax -> SpMM, one launch each for all heads "
                                                "(this package, fp32)", unfused, max(args.steps // 4, 2), 2)
    if args.vendor:
        ones = torch.ones(crd.numel(), device="cuda")
        qf, kf, vf = q32, k32, v32

        def unfused_per_head():
            outs = []
            for h in range(Hh):
                sc = H.sddmm_csr_float([S, S], [S, S], [[], [pos, crd]], ones, [S, D], [[], []],
                                       qf[h].reshape(-1), [S, D], [[], []], kf[h].reshape(-1))
                p = H.softmax_csr_float(pos, sc.storage.value, float(w["scale"]))
                outs.append(H.spmm_csr_float_v2([S, D], [S, S], [[], [pos, crd]], p, [S, D], [[], []],
                                                vf[h].reshape(-1)).storage.value)
            return outs

        rec["unfused_fp32_pipeline_per_head"] = _vendor_time(
            "SDDMM -> softmax -> SpMM per head from a Python loop, as the reference's benchmark runs it "
            "(this package, fp32)", unfused_per_head, max(args.steps // 4, 2), 1)
        # (b) torch's dense attention with the same mask
        import torch.nn.functional as F
        blk = w["block"]
        rows_b = np.repeat(np.arange(brp.numel() - 1), np.diff(w["block_row_ptr"]))
        dense_blocks = np.zeros((S // blk, S // blk), bool)
        dense_blocks[rows_b, w["block_col_idx"]] = True
        mask = torch.from_numpy(np.kron(dense_blocks, np.ones((blk, blk), bool))).cuda()
        rec["vendor_library"] = _vendor_time(
            "F.scaled_dot_product_attention(bf16, dense boolean mask)",
            lambda: F.scaled_dot_product_attention(q[None], k[None], v[None], attn_mask=mask[None, None],
                                                   scale=float(w["scale"])), max(args.steps // 4, 2), 1)
    if not args.no_cpu:
        rec["cpu_baseline"] = cpu_baseline_attention(w)
    return rec


# ---- workloads beside the five configurations -------------------------------------------------------
def run_extra(args):
    import numpy as np
    import torch
    from scorch_amd import scorch_ops_hip as H
    from scorch_amd import workloads
    base = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": "f32", "data": "synthetic",
            "higher_is_better": True}
    if args.workload == "gcn_forward":
        # The two-layer GCN forward pass of the reference's graph benchmark
        # (bench/bench_gcn.py:320-357) on the headline graph: linear -> A_hat x -> + bias
        # -> relu -> linear -> A_hat x -> + bias -> log_softmax, once with the separate
        # steps and once through @compile, which routes matmul + bias (+ relu) to the fused kernel.
        import torch.nn.functional as F
        import scorch_amd as scorch
        w = workloads.gcn_powerlaw(M=args.rows, N=args.features)
        M, nnz = w["M"], int(w["col_idx"].size)
        hidden, classes = 128, 64
        adj = scorch.STensor.from_csr_arrays(_t(w["row_ptr"]), _t(w["col_idx"]), _t(w["vals"]), (M, M))
        x0 = _t(w["B"])
        gen = torch.Generator(device="cuda").manual_seed(5)
        weights = {"w1": torch.randn(hidden, args.features, device="cuda", generator=gen) * 0.1,
                   "b1": torch.randn(hidden, device="cuda", generator=gen) * 0.1,
                   "w2": torch.randn(classes, hidden, device="cuda", generator=gen) * 0.1,
                   "b2": torch.randn(classes, device="cuda", generator=gen) * 0.1}

        def unfused():
            h = F.linear(x0, weights["w1"])
            h = scorch.matmul(adj, h, format="dd") + weights["b1"]
            h = F.linear(F.relu(h), weights["w2"])
            return F.log_softmax(scorch.matmul(adj, h, format="dd") + weights["b2"], dim=1)

        @scorch.compile
        def spmm_bias_relu(a, h, bias):
            return torch.relu(scorch.matmul(a, h, format="dd") + bias)

        @scorch.compile
        def spmm_bias(a, h, bias):
            return scorch.matmul(a, h, format="dd") + bias

        def fused():
            h = spmm_bias_relu(adj, F.linear(x0, weights["w1"]), weights["b1"])
            return F.log_softmax(spmm_bias(adj, F.linear(h, weights["w2"]), weights["b2"]), dim=1)

        a_t = torch.sparse_csr_tensor(adj.index.mode_indices[1][0], adj.index.mode_indices[1][1], adj.values,
                                      size=(M, M))

        def vendor():
            h = F.relu(torch.sparse.mm(a_t, F.linear(x0, weights["w1"])) + weights["b1"])
            return F.log_softmax(torch.sparse.mm(a_t, F.linear(h, weights["w2"])) + weights["b2"], dim=1)

        err = float((fused() - unfused()).abs().max())
        ms_fused = _time_steps(fused, args.steps, args.warmup)
        ms_unfused = _time_steps(unfused, args.steps, args.warmup)
        out = {"metric": "two-layer GCN forward passes per second", "value": round(1e3 / ms_fused, 2),
               "unit": "1/s", "ms_per_step": round(ms_fused, 4), "ms_per_step_unfused": round(ms_unfused, 4),
               "max_abs_difference_fused_unfused": err, **base,
               "config": {"workload": "gcn_forward_fp32", "rows": M, "nnz": nnz, "features": args.features,
                          "hidden": hidden, "classes": classes}}
        if args.vendor:
            out["vendor_library"] = _vendor_time("torch.sparse.mm in the same forward pass", vendor,
                                                 max(args.steps // 2, 2), 1)
        return out
    if args.workload == "copy_calibration":
        # 1 GiB read and 1 GiB written by a plain elementwise kernel: what the memory counters
        # (FETCH_SIZE, WRITE_SIZE) read for a known amount of traffic gives the factor by which the
        # counters of the other workloads are scaled.
        n = 1 << 28
        x = torch.ones(n, device="cuda")
        y = torch.empty_like(x)
        ms = _time_steps(lambda: torch.mul(x, 2.0, out=y), args.steps, args.warmup)
        return {"metric": "copy GB/s (read + write)", "value": round(8.0 * n / ms / 1e6, 1), "unit": "GB/s",
                "ms_per_step": round(ms, 4), **base,
                "config": {"workload": "copy_calibration", "bytes_read": 4 * n, "bytes_written": 4 * n}}
    if args.workload == "attention_longformer":
        # The reference's sparse-transformer benchmark shape (bench/bench_sparse_transformer.py:49-60,
        # 194-209): embedding 256 in 8 heads (head dimension 32), Longformer mask with a window of 64 on
        # either side and one global token, fp32; SDDMM -> row softmax -> SpMM, one launch each for all heads.
        S, heads, D = (args.rows if args.rows != 1 << 20 else 4096), 8, 32
        rp_np, ci_np = workloads.longformer_mask(S)
        rp, ci = _t(rp_np), _t(ci_np)
        gen = torch.Generator(device="cuda").manual_seed(7)
        q, k, v = (torch.randn(heads, S, D, device="cuda", generator=gen) for _ in range(3))
        scale = D ** -0.5
        fn = lambda: H.sparse_attention_csr(rp, ci, q, k, v, scale)
        ms = _time_steps(fn, args.steps, args.warmup)
        nnz = int(ci_np.size)
        out = {"metric": "sparse attention (SDDMM -> softmax -> SpMM) GFLOP/s", "unit": "GFLOP/s",
               "value": round(heads * (4.0 * nnz * D + 5.0 * nnz) / ms / 1e6, 2), "ms_per_step": round(ms, 5), **base,
               "config": {"workload": "attention_longformer_fp32", "S": S, "H": heads, "D": D, "window": 64,
                          "global_tokens": 1, "nnz_per_head": nnz}}
        # the same mask through the fused bf16 kernel: 64 x 64 blocks with per-block bit masks
        qb, kb, vb = (t.to(torch.bfloat16) for t in (q, k, v))
        bm = H.attention_block_mask(rp, ci, S)
        ms_fused = _time_steps(lambda: H.sparse_attention_bf16(qb, kb, vb, rp, ci, scale), args.steps, args.warmup)
        diff = (H.sparse_attention_bf16(qb, kb, vb, rp, ci, scale).float() - fn()).norm() / fn().norm()
        out["fused_bf16"] = {"ms_per_step": round(ms_fused, 5), "active_blocks": bm.n_active_blocks,
                             "distinct_block_masks": bm.n_masks,
                             "live_share_of_active_blocks": round(bm.density_in_blocks, 4),
                             "rel_fro_vs_fp32_pipeline": float(diff)}
        # ... and through the fused fp32 kernel (fp32 operands, probabilities and sums)
        ms_fused32 = _time_steps(lambda: H.sparse_attention_f32(q, k, v, rp, ci, scale), args.steps, args.warmup)
        diff32 = (H.sparse_attention_f32(q, k, v, rp, ci, scale) - fn()).norm() / fn().norm()
        out["fused_fp32"] = {"ms_per_step": round(ms_fused32, 5), "rel_fro_vs_fp32_pipeline": float(diff32)}
        if args.vendor:
            import torch.nn.functional as F
            rows = torch.repeat_interleave(torch.arange(S, device="cuda"), (rp[1:] - rp[:-1]).long())
            live = torch.zeros(S, S, dtype=torch.bool, device="cuda")
            live[rows, ci.long()] = True
            out["vendor_library"] = _vendor_time(
                "F.scaled_dot_product_attention(fp32, dense boolean mask)",
                lambda: F.scaled_dot_product_attention(q[None], k[None], v[None], attn_mask=live[None, None],
                                                       scale=scale), max(args.steps // 4, 2), 1)
        if not args.no_cpu:
            w = {"S": S, "H": heads, "D": D, "q": q.cpu().numpy(), "k": k.cpu().numpy(), "v": v.cpu().numpy(),
                 "scale": scale}
            out["cpu_baseline"] = cpu_baseline_attention(w, heads=2, pattern=(rp_np, ci_np))
        return out
    if args.workload == "softmax_rows":
        # every row --row-length entries long, or a causal mask (row i has i + 1) with --row-length 0
        M = args.rows if args.rows != 1 << 20 else 8192
        lens = np.full(M, args.row_length, np.int64) if args.row_length > 0 else np.arange(1, M + 1, dtype=np.int64)
        pos = _t(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32))
        nnz = int(lens.sum())
        val = torch.randn(nnz, device="cuda")
        ms = _time_steps(lambda: H.softmax_csr_float(pos, val, 1.0), args.steps, args.warmup)
        algo = 8 * nnz + 4 * (M + 1)
        return {"metric": "CSR row softmax GFLOP/s (4 flops per entry)", "value": round(4.0 * nnz / ms / 1e6, 2),
                "unit": "GFLOP/s", "ms_per_step": round(ms, 4), **base,
                "config": {"workload": "softmax_rows_fp32", "rows": M, "nnz": nnz,
                           "row_length": args.row_length if args.row_length > 0 else "causal"},
                "algorithmic_bytes": algo, "hbm_gbps_algorithmic": round(algo / ms / 1e6, 1),
                "hbm_frac_algorithmic": round(algo / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    if args.workload in ("spmv_powerlaw", "softmax_powerlaw"):
        w = workloads.gcn_powerlaw(M=args.rows, N=1)
        M, nnz = w["M"], int(w["col_idx"].size)
        pos, crd, val = _t(w["row_ptr"]), _t(w["col_idx"]), _t(w["vals"])
        x = _t(w["B"]).reshape(-1)
        if args.workload == "spmv_powerlaw":
            fn = lambda: H.prebuilt_spmv_csr_f32([M], [M, M], [[], [pos, crd]], val, [M], [[]], x)
            algo, flops, name = 8 * nnz + 4 * (M + 1) + 8 * M, 2.0 * nnz, "CSR SpMV GFLOP/s"
        else:
            fn = lambda: H.softmax_csr_float(pos, val, 1.0)
            algo, flops, name = 8 * nnz + 4 * (M + 1), 4.0 * nnz, "CSR row softmax GFLOP/s (4 flops per entry)"
        ms = _time_steps(fn, args.steps, args.warmup)
        out = {"metric": name, "value": round(flops / ms / 1e6, 2), "unit": "GFLOP/s", "ms_per_step": round(ms, 4),
               **base, "config": {"workload": args.workload + "_fp32", "rows": M, "nnz": nnz},
               "algorithmic_bytes": algo, "hbm_gbps_algorithmic": round(algo / ms / 1e6, 1),
               "hbm_frac_algorithmic": round(algo / ms / 1e6 / HBM_PEAK_GBPS, 4)}
        if args.workload == "softmax_powerlaw":
            # the same through a plan handle, which knows the pattern's longest row and leaves out the
            # launches no row of that length needs
            from scorch_amd.csr_plan import CsrPlanHandle
            with CsrPlanHandle(pos, crd, M) as plan:
                assert torch.equal(plan.softmax(val, 1.0), fn())
                out["ms_per_step_plan_handle"] = round(_time_steps(lambda: plan.softmax(val, 1.0), args.steps,
                                                                   args.warmup), 4)
                out["longest_row"] = plan.info()["longest_row"]
        if args.vendor and args.workload == "spmv_powerlaw":
            A_t = torch.sparse_csr_tensor(pos, crd, val, size=(M, M))
            out["vendor_library"] = _vendor_time("torch.mv(csr, x)", lambda: torch.mv(A_t, x), args.steps, 1)
        return out
    if args.workload == "spgemm_powerlaw":
        # A @ A for the power-law graph at 1/8 of the headline size (the square of the
        # full graph has billions of products)
        rows = args.rows if args.rows != 1 << 20 else 1 << 17
        w = workloads.gcn_powerlaw(M=rows, N=4, max_degree=5000)
        M = w["M"]
        pos, crd, val = _t(w["row_ptr"]), _t(w["col_idx"]), _t(w["vals"])
        fn = lambda: H.prebuilt_spmspm_csr_f32([M, M], [M, M], [[], [pos, crd]], val, [M, M], [[], [pos, crd]], val)
        nnz_c = int(fn().storage.value.numel())
        deg = (pos[1:] - pos[:-1]).long()
        products = int(deg[crd.long()].sum().item())
        ms = _time_steps(fn, args.steps, args.warmup, rounds=1)
        out = {"metric": "CSR SpGEMM GFLOP/s (2 flops per product)", "value": round(2.0 * products / ms / 1e6, 2),
               "unit": "GFLOP/s", "ms_per_step": round(ms, 4), **base,
               "config": {"workload": "spgemm_powerlaw_fp32", "rows": M, "nnz_a": int(crd.numel()),
                          "products": products, "nnz_c": nnz_c},
               "note": "symbolic + numeric passes and the host read of nnz(C) between them"}
        if args.vendor:
            A_t = torch.sparse_csr_tensor(pos, crd, val, size=(M, M))
            out["vendor_library"] = _vendor_time("torch.sparse.mm(csr, csr)", lambda: torch.sparse.mm(A_t, A_t),
                                                 max(2, args.steps // 4), 1)
        return out
    raise ValueError(args.workload)


def run_workload(name, args, headline=False):
    if name in ("gcn_powerlaw", "spmm_uniform", "sae_decoder"):
        return run_spmm(name, args, headline)
    if name == "sddmm_uniform":
        return run_sddmm(args)
    if name == "attention_blocksparse":
        return run_attention(args)
    return run_extra(args)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--rows", type=int, default=1 << 20, help="nodes of the graph (default: the headline size)")
    ap.add_argument("--features", type=int, default=128)
    ap.add_argument("--window", type=int, default=0,
                    help="gcn_powerlaw: draw a node's neighbours from this many nodes around it instead of from "
                         "all nodes (same degrees; shows what the kernel does when rows share neighbours)")
    ap.add_argument("--row-length", type=int, default=0,
                    help="softmax_rows: entries per row (0: a causal mask, row i has i + 1 entries)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--headline-only", action="store_true", help="skip the records of the other four configurations")
    ap.add_argument("--workload", default=None,
                    choices=[HEADLINE, *CONFIG_WORKLOADS, "spgemm_powerlaw", "spmv_powerlaw", "softmax_powerlaw",
                             "softmax_rows", "gcn_forward", "attention_longformer", "copy_calibration"],
                    help="print this workload's record alone (default: the headline line with all configurations)")
    ap.add_argument("--vendor", action="store_true",
                    help="also time torch's own sparse routine on the same operands")
    ap.add_argument("--graph", action="store_true",
                    help="also capture one step in a HIP graph and time its replay (SpMM side workloads)")
    ap.add_argument("--source-hashes", action="store_true",
                    help="print the current hash of every kernel's source files named in MEASURED_TRAFFIC and exit")
    args = ap.parse_args()
    if args.source_hashes:
        for key, rec in MEASURED_TRAFFIC.items():
            now = source_hash(rec["sources"])
            print(f"{key}: {now}" + ("" if now == rec["sha16"] else f"  (recorded: {rec['sha16'] or 'none'})"))
        return 0
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU leg (the kernel shards by rows "
              "of A, every GPU writing its own rows of C, with no reduction). Run with --gpus 1.", file=sys.stderr)
        return 2

    import torch
    from scorch_amd import native

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        return 1
    if not os.path.exists(native.library_path()):
        print("libscorch_hip.so is not built (python __graft_entry__.py)", file=sys.stderr)
        return 1
    torch.cuda.set_device(0)

    if args.workload is not None:
        print(json.dumps(run_workload(args.workload, args, headline=args.workload == HEADLINE)))
        return 0
    result = run_workload(HEADLINE, args, headline=True)
    if not args.headline_only:
        result["configs"] = []
        for name in CONFIG_WORKLOADS:
            torch.cuda.empty_cache()
            # the CPU leg of the configuration before leaves its OpenMP workers spinning for a moment; the
            # first calls of the next one are host-bound and would be timed against them
            time.sleep(0.2)
            try:
                result["configs"].append(run_workload(name, args))
            except Exception as exc:  # one configuration failing must not lose the headline line
                result["configs"].append({"config": {"workload": name}, "error": f"{type(exc).__name__}: {exc}"})
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
