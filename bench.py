"""Headline benchmark: CSR SpMM, fp32, on the GCN-style power-law graph
(1,048,576 nodes, N = 128 features) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

A step is one C = A @ B through the C ABI of libscorch_hip.so with A, B
resident in HBM (the output buffer comes from torch's caching allocator).
Prints ONE JSON line: whole-job GFLOP/s (2 * nnz * N flops per step, the
reference's convention, tools/benchmark_spmm_variants.py:127-129), the memory
roofline of the dominant kernel and the CPU baseline timed on this host.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0   # MI355X HBM3E, published
WORKLOAD = "gcn_powerlaw_spmm_fp32"

# Bytes through the L2-to-fabric boundary per launch of the dominant kernel at
# the headline size: FETCH_SIZE (4,292,650 KiB x 2.0, the factor a 1 GiB copy
# kernel gives for this counter) + WRITE_SIZE (539,816 KiB x 1.0) from two
# rocprofv3 --pmc runs of this script.  It is a measured constant, valid for
# the default workload only; the summary with the commands is
# profiles/spmm_merge_kernel_gcn_powerlaw.md.
MEASURED_TRAFFIC_BYTES = 9_344_118_000


def algorithmic_bytes(M, K, N, nnz):
    """Every array touched once: col_idx + vals, row_ptr, B, C (fp32 / int32)."""
    return 8 * nnz + 4 * (M + 1) + 4 * K * N + 4 * M * N


def gather_bytes(M, N, nnz):
    """No-reuse model: a B row re-read for every nonzero."""
    return 8 * nnz + 4 * (M + 1) + 4 * nnz * N + 4 * M * N


def cpu_baseline(w, repeats=5):
    """The reference's spmm_csr_float_v2 (oracle/_ref, compiled from the
    reference's sources) or, where that module is absent, this repository's C
    restatement of it, timed on the host cores on the same inputs.  The timed
    region is the whole native call, as the reference's own eval_time is: it
    includes allocating and zero-filling C."""
    from oracle import oracle as O
    M, N, nnz = w["M"], w["N"], int(w["col_idx"].size)
    flops = 2.0 * nnz * N
    kind, times = "port", []
    if O.have_ref():
        try:
            import torch
            mod = O.ref_module()
            pos, crd = torch.from_numpy(w["row_ptr"]), torch.from_numpy(w["col_idx"])
            val, Bf = torch.from_numpy(w["vals"]), torch.from_numpy(w["B"]).reshape(-1)
            args = ([M, N], [M, w["K"]], [[], [pos, crd]], val, [w["K"], N], [[], []], Bf)
            for i in range(repeats + 1):
                t0 = time.perf_counter()
                out = mod.spmm_csr_float_v2(*args)
                dt = time.perf_counter() - t0
                del out
                if i:
                    times.append(dt)
            kind = "reference"
        except Exception as exc:  # module built for another host
            print(f"[bench] reference module unusable here ({exc}); timing the C restatement",
                  file=sys.stderr)
            times = []
    if not times:
        import numpy as np
        out = np.empty((M, N), dtype=np.float32)
        for i in range(repeats + 1):
            t0 = time.perf_counter()
            O.spmm_csr_f32_v2(w["row_ptr"], w["col_idx"], w["vals"], w["B"], out=out)
            dt = time.perf_counter() - t0
            if i:
                times.append(dt)
    med = statistics.median(times)
    return {"value": round(flops / med / 1e9, 3), "unit": "GFLOP/s", "cores": O.num_threads(),
            "kind": kind, "ms_per_step": round(med * 1e3, 3),
            "sample": f"full workload (M={M}, nnz={nnz}, N={N}), median of {repeats} calls after 1 "
                      "warm-up, whole native call incl. allocating and zeroing C"}


def cpu_baseline_sddmm(w, repeats=5):
    """The reference's sddmm_coo_float_prebuilt (oracle/_ref) or the C
    restatement of it, on the host cores, coordinate mask, same inputs."""
    from oracle import oracle as O
    nnz, K = int(w["col_idx"].size), w["K"]
    kind = "reference" if O.have_ref() else "port"
    times = []
    for i in range(repeats + 1):
        t0 = time.perf_counter()
        try:
            if kind == "reference":
                O.ref_sddmm_coo(w["row_idx"], w["col_idx"], w["vals"], w["A"], w["B"], (w["M"], w["n_cols"]))
            else:
                O.sddmm_coo_f32(w["row_idx"], w["col_idx"], w["vals"], w["A"], w["B"])
        except Exception as exc:  # module built for another host
            if kind == "port":
                raise
            print(f"[bench] reference module unusable here ({exc}); timing the C restatement", file=sys.stderr)
            kind = "port"
            continue
        if i:
            times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {"value": round((2.0 * nnz * K + nnz) / med / 1e9, 3), "unit": "GFLOP/s", "cores": O.num_threads(),
            "kind": kind, "ms_per_step": round(med * 1e3, 3),
            "sample": f"full workload (nnz={nnz}, K={K}), median of {len(times)} calls after 1 warm-up, "
                      "incl. wrapping the operands"}


def _time_steps(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def _vendor_time(call_name, fn, steps, warmup):
    """Times a torch routine on the same operands; an error becomes a field."""
    try:
        return {"call": call_name, "ms_per_step": round(_time_steps(fn, steps, warmup), 4)}
    except RuntimeError as err:
        return {"call": call_name, "error": str(err).splitlines()[0]}


def vendor_spmm(pos, crd, val, B2d, steps, warmup):
    """torch.sparse.mm on the same CSR operands (torch routes it to the ROCm
    sparse library): a second GPU implementation timed beside ours.  Returns a
    JSON-ready dict; never part of `value`."""
    import torch
    M = pos.numel() - 1
    A = torch.sparse_csr_tensor(pos, crd, val, size=(M, B2d.shape[0]))
    try:
        ms = _time_steps(lambda: torch.sparse.mm(A, B2d), steps, warmup)
    except RuntimeError as err:                       # e.g. unsupported size
        return {"call": "torch.sparse.mm(csr, dense)", "error": str(err).splitlines()[0]}
    return {"call": "torch.sparse.mm(csr, dense)", "ms_per_step": round(ms, 4)}


def side_workload(args, dev) -> int:
    """Times one of the other workloads (not the headline metric): same JSON
    shape, HIP-event time per step, algorithmic and gather-model bandwidth."""
    import torch
    from scorch_amd import workloads
    from scorch_amd import scorch_ops_hip as H
    t = lambda a: torch.from_numpy(a).to(dev)
    if args.workload == "attention_blocksparse":
        w = workloads.attention_blocksparse()
        Hh, S, D = w["H"], w["S"], w["D"]
        q, k, v = (t(w[n]).to(torch.bfloat16) for n in ("q", "k", "v"))
        brp, bci = t(w["block_row_ptr"]), t(w["block_col_idx"])
        nnz = int(w["block_col_idx"].size) * w["block"] ** 2
        fn = lambda: H.attn_blocksparse_bf16(q, k, v, brp, bci, float(w["scale"]))
        ms = _time_steps(fn, args.steps, args.warmup)
        flops = 4.0 * nnz * D * Hh
        algo = 4 * Hh * S * D * 2 + 4 * (brp.numel() + bci.numel())
        extra = {}
        if args.vendor:
            # (a) the composition the reference's benchmark uses, per head and in fp32, on this
            # package's own kernels: SDDMM -> row softmax -> SpMM (bench_sparse_transformer.py:354-372)
            import numpy as np
            blk = w["block"]
            rows_b = np.repeat(np.arange(brp.numel() - 1), np.diff(w["block_row_ptr"]))
            dense_blocks = np.zeros((S // blk, S // blk), bool)
            dense_blocks[rows_b, w["block_col_idx"]] = True
            mask = torch.from_numpy(np.kron(dense_blocks, np.ones((blk, blk), bool))).to(dev)
            csr = mask.to(torch.float32).to_sparse_csr()
            pos, crd = csr.crow_indices().to(torch.int32), csr.col_indices().to(torch.int32)
            ones = torch.ones(crd.numel(), device=dev)
            qf, kf, vf = q.float(), k.float(), v.float()

            def unfused():
                outs = []
                for h in range(Hh):
                    sc = H.sddmm_csr_float([S, S], [S, S], [[], [pos, crd]], ones, [S, D], [[], []],
                                           qf[h].reshape(-1), [S, D], [[], []], kf[h].reshape(-1))
                    p = H.softmax_csr_float(pos, sc.storage.value, float(w["scale"]))
                    outs.append(H.spmm_csr_float_v2([S, D], [S, S], [[], [pos, crd]], p, [S, D], [[], []],
                                                    vf[h].reshape(-1)).storage.value)
                return outs

            extra["unfused_fp32_pipeline"] = _vendor_time("SDDMM -> softmax -> SpMM per head (this package, fp32)",
                                                          unfused, max(args.steps // 4, 2), 1)
            # (b) torch's dense attention with the same mask
            import torch.nn.functional as F
            extra["vendor_library"] = _vendor_time(
                "F.scaled_dot_product_attention(bf16, dense boolean mask)",
                lambda: F.scaled_dot_product_attention(q[None], k[None], v[None], attn_mask=mask[None, None],
                                                       scale=float(w["scale"])), max(args.steps // 4, 2), 1)
        print(json.dumps({**extra,
                          "metric": "fused block-sparse attention TFLOP/s", "value": round(flops / ms / 1e9, 2),
                          "unit": "TFLOP/s", "ms_per_step": round(ms, 4), "n_gpus": 1, "steps": args.steps,
                          "warmup": args.warmup, "dtype": "bf16", "data": "synthetic",
                          "higher_is_better": True,
                          "config": {"workload": "attention_blocksparse_bf16", "S": S, "H": Hh, "D": D,
                                     "block": w["block"], "active_blocks": int(bci.numel()),
                                     "nnz_per_head": nnz},
                          "mfma_frac_of_2.5PFLOPs": round(flops / ms / 1e9 / 2500.0, 4),
                          "algorithmic_bytes": algo, "hbm_gbps_algorithmic": round(algo / ms / 1e6, 1)}))
        return 0
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
        adj = scorch.STensor.from_csr_arrays(t(w["row_ptr"]), t(w["col_idx"]), t(w["vals"]), (M, M))
        x0 = t(w["B"])
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
               "max_abs_difference_fused_unfused": err, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
               "dtype": "f32", "data": "synthetic", "higher_is_better": True,
               "config": {"workload": "gcn_forward_fp32", "rows": M, "nnz": nnz, "features": args.features,
                          "hidden": hidden, "classes": classes}}
        if args.vendor:
            out["vendor_library"] = _vendor_time("torch.sparse.mm in the same forward pass", vendor, args.steps,
                                                 args.warmup)
        print(json.dumps(out))
        return 0
    if args.workload == "softmax_rows":
        # every row --row-length entries long, or a causal mask (row i has i + 1) with --row-length 0
        import numpy as np
        M = args.rows if args.rows != 1 << 20 else 8192
        lens = np.full(M, args.row_length, np.int64) if args.row_length > 0 else np.arange(1, M + 1, dtype=np.int64)
        pos = t(np.concatenate([[0], np.cumsum(lens)]).astype(np.int32))
        nnz = int(lens.sum())
        val = torch.randn(nnz, device="cuda")
        ms = _time_steps(lambda: H.softmax_csr_float(pos, val, 1.0), args.steps, args.warmup)
        algo = 8 * nnz + 4 * (M + 1)
        print(json.dumps({"metric": "CSR row softmax GFLOP/s (4 flops per entry)",
                          "value": round(4.0 * nnz / ms / 1e6, 2), "unit": "GFLOP/s", "ms_per_step": round(ms, 4),
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": "f32",
                          "data": "synthetic", "higher_is_better": True,
                          "config": {"workload": "softmax_rows_fp32", "rows": M, "nnz": nnz,
                                     "row_length": args.row_length if args.row_length > 0 else "causal"},
                          "algorithmic_bytes": algo, "hbm_gbps_algorithmic": round(algo / ms / 1e6, 1),
                          "hbm_frac_algorithmic": round(algo / ms / 1e6 / HBM_PEAK_GBPS, 4)}))
        return 0
    if args.workload in ("spmv_powerlaw", "softmax_powerlaw"):
        w = workloads.gcn_powerlaw(M=args.rows, N=1)
        M, nnz = w["M"], int(w["col_idx"].size)
        pos, crd, val = t(w["row_ptr"]), t(w["col_idx"]), t(w["vals"])
        x = t(w["B"]).reshape(-1)
        if args.workload == "spmv_powerlaw":
            fn = lambda: H.prebuilt_spmv_csr_f32([M], [M, M], [[], [pos, crd]], val, [M], [[]], x)
            algo, flops, name = 8 * nnz + 4 * (M + 1) + 8 * M, 2.0 * nnz, "CSR SpMV GFLOP/s"
        else:
            fn = lambda: H.softmax_csr_float(pos, val, 1.0)
            algo, flops, name = 8 * nnz + 4 * (M + 1), 4.0 * nnz, "CSR row softmax GFLOP/s (4 flops per entry)"
        ms = _time_steps(fn, args.steps, args.warmup)
        vendor = None
        if args.vendor and args.workload == "spmv_powerlaw":
            A_t = torch.sparse_csr_tensor(pos, crd, val, size=(M, M))
            vendor = _vendor_time("torch.mv(csr, x)", lambda: torch.mv(A_t, x), args.steps, args.warmup)
        print(json.dumps({**({"vendor_library": vendor} if vendor else {}),
                          "metric": name, "value": round(flops / ms / 1e6, 2), "unit": "GFLOP/s",
                          "ms_per_step": round(ms, 4), "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                          "dtype": "f32", "data": "synthetic", "higher_is_better": True,
                          "config": {"workload": args.workload + "_fp32", "rows": M, "nnz": nnz},
                          "algorithmic_bytes": algo, "hbm_gbps_algorithmic": round(algo / ms / 1e6, 1),
                          "hbm_frac_algorithmic": round(algo / ms / 1e6 / HBM_PEAK_GBPS, 4)}))
        return 0
    if args.workload == "spgemm_powerlaw":
        # A @ A for the power-law graph at 1/8 of the headline size (the square of the
        # full graph has billions of products)
        rows = args.rows if args.rows != 1 << 20 else 1 << 17
        w = workloads.gcn_powerlaw(M=rows, N=4, max_degree=5000)
        M = w["M"]
        pos, crd, val = t(w["row_ptr"]), t(w["col_idx"]), t(w["vals"])
        fn = lambda: H.prebuilt_spmspm_csr_f32([M, M], [M, M], [[], [pos, crd]], val, [M, M],
                                               [[], [pos, crd]], val)
        out = fn()
        nnz_c = int(out.storage.value.numel())
        deg = (pos[1:] - pos[:-1]).long()
        products = int(deg[crd.long()].sum().item())
        ms = _time_steps(fn, args.steps, args.warmup)
        vendor = None
        if args.vendor:
            A_t = torch.sparse_csr_tensor(pos, crd, val, size=(M, M))
            vendor = _vendor_time("torch.sparse.mm(csr, csr)", lambda: torch.sparse.mm(A_t, A_t),
                                  max(2, args.steps // 4), 1)
        print(json.dumps({"metric": "CSR SpGEMM GFLOP/s (2 flops per product)",
                          "value": round(2.0 * products / ms / 1e6, 2), "unit": "GFLOP/s",
                          "ms_per_step": round(ms, 4), "n_gpus": 1, "steps": args.steps,
                          "warmup": args.warmup, "dtype": "f32", "data": "synthetic",
                          "higher_is_better": True,
                          "config": {"workload": "spgemm_powerlaw_fp32", "rows": M, "nnz_a": int(crd.numel()),
                                     "products": products, "nnz_c": nnz_c},
                          "note": "symbolic + numeric passes and the host read of nnz(C) between them",
                          **({"vendor_library": vendor} if vendor else {})}))
        return 0
    if args.workload == "sddmm_uniform":
        w = workloads.sddmm_uniform()
        M, n_cols, K, nnz = w["M"], w["n_cols"], w["K"], int(w["col_idx"].size)
        pos, crd, val, A, B = t(w["row_ptr"]), t(w["col_idx"]), t(w["vals"]), t(w["A"]), t(w["B"])
        rows = t(w["row_idx"])
        csr = lambda: H.sddmm_csr_float([M, n_cols], [M, n_cols], [[], [pos, crd]], val, [M, K], [[], []],
                                        A.reshape(-1), [n_cols, K], [[], []], B.reshape(-1))
        coo = lambda: H.sddmm_coo_float_prebuilt([M, n_cols], [M, n_cols], [[rows], [crd]], val, [M, K],
                                                 [[], []], A.reshape(-1), [n_cols, K], [[], []],
                                                 B.reshape(-1))
        ms = _time_steps(csr, args.steps, args.warmup)
        ms_coo = _time_steps(coo, args.steps, args.warmup)
        flops = 2.0 * nnz * K + nnz
        algo = 4 * (M + 1) + 4 * nnz * 3 + 4 * M * K + 4 * n_cols * K + 4 * nnz   # + row output
        gather = algo - 4 * n_cols * K + 4 * nnz * K
        out = {"metric": "CSR SDDMM GFLOP/s", "value": round(flops / ms / 1e6, 2), "unit": "GFLOP/s",
               "ms_per_step": round(ms, 4), "ms_per_step_coo_mask": round(ms_coo, 4),
               "config": {"workload": "sddmm_uniform_fp32", "rows": M, "cols": n_cols, "nnz": nnz, "K": K}}
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_baseline_sddmm(w)
        if args.vendor:
            mask = torch.sparse_csr_tensor(pos, crd, val, size=(M, n_cols))
            Bt = B.t().contiguous()
            out["vendor_library"] = _vendor_time(
                "torch.sparse.sampled_addmm(mask, A, B^T, beta=0)",
                lambda: torch.sparse.sampled_addmm(mask, A, Bt, beta=0.0), args.steps, args.warmup)
    else:
        w = workloads.spmm_uniform() if args.workload == "spmm_uniform" else workloads.sae_decoder()
        M, K, N, nnz = w["M"], w["K"], w["N"], int(w["col_idx"].size)
        pos, crd, val, B = t(w["row_ptr"]), t(w["col_idx"]), t(w["vals"]), t(w["B"]).reshape(-1)
        fn = lambda: H.spmm_csr_float_v2([M, N], [M, K], [[], [pos, crd]], val, [K, N], [[], []], B)
        ms = _time_steps(fn, args.steps, args.warmup)
        flops = 2.0 * nnz * N
        algo, gather = algorithmic_bytes(M, K, N, nnz), gather_bytes(M, N, nnz)
        out = {"metric": "CSR SpMM GFLOP/s", "value": round(flops / ms / 1e6, 2), "unit": "GFLOP/s",
               "ms_per_step": round(ms, 4),
               "config": {"workload": args.workload + "_fp32", "rows": M, "cols": K, "nnz": nnz,
                          "features": N}}
        if args.graph:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                fn()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                fn()
            out["ms_per_step_graph_replay"] = round(_time_steps(graph.replay, args.steps, args.warmup), 4)
        if args.vendor:
            out["vendor_library"] = vendor_spmm(pos, crd, val, B.reshape(K, N), args.steps, args.warmup)
        if not args.no_cpu:
            out["cpu_baseline"] = cpu_baseline(w)
    out.update({"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "dtype": "f32",
                "data": "synthetic", "higher_is_better": True,
                "algorithmic_bytes": algo, "hbm_gbps_algorithmic": round(algo / ms / 1e6, 1),
                "hbm_frac_algorithmic": round(algo / ms / 1e6 / HBM_PEAK_GBPS, 4),
                "gather_model_bytes": gather, "gather_model_gbps": round(gather / ms / 1e6, 1)})
    print(json.dumps(out))
    return 0


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
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--workload", default="gcn_powerlaw",
                    choices=["gcn_powerlaw", "spmm_uniform", "sae_decoder", "sddmm_uniform",
                             "attention_blocksparse", "spgemm_powerlaw", "spmv_powerlaw",
                             "softmax_powerlaw", "softmax_rows", "gcn_forward"],
                    help="gcn_powerlaw is the headline line; the others time the parity workloads")
    ap.add_argument("--vendor", action="store_true",
                    help="also time torch's own sparse routine on the same operands (SpMM, SDDMM, SpGEMM, SpMV)")
    ap.add_argument("--graph", action="store_true",
                    help="also capture one step in a HIP graph and time its replay (SpMM side workloads)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU leg (the kernel shards by rows "
              "of A, every GPU writing its own rows of C, with no reduction). Run with --gpus 1.", file=sys.stderr)
        return 2

    import torch
    from scorch_amd import native, workloads
    from scorch_amd import scorch_ops_hip as H

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        return 1
    if not os.path.exists(native.library_path()):
        print("libscorch_hip.so is not built (python __graft_entry__.py)", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.workload != "gcn_powerlaw":
        return side_workload(args, dev)

    t0 = time.time()
    w = workloads.gcn_powerlaw(M=args.rows, N=args.features, window=args.window)
    M, K, N, nnz = w["M"], w["K"], w["N"], int(w["col_idx"].size)
    print(f"[bench] generated {WORKLOAD}: M={M} nnz={nnz} N={N} in {time.time() - t0:.1f}s", file=sys.stderr)

    pos = torch.from_numpy(w["row_ptr"]).to(dev)
    crd = torch.from_numpy(w["col_idx"]).to(dev)
    val = torch.from_numpy(w["vals"]).to(dev)
    B = torch.from_numpy(w["B"]).to(dev).reshape(-1)
    call = ([M, N], [M, K], [[], [pos, crd]], val, [K, N], [[], []], B)

    for _ in range(args.warmup):
        out = H.spmm_csr_float_v2(*call)
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t_begin = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        out = H.spmm_csr_float_v2(*call)
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t_begin
    ms_per_step = wall * 1e3 / args.steps
    event_ms_per_step = start.elapsed_time(stop) / args.steps

    # per-kernel durations: events around each kernel, on the launch stream
    L = native.lib()
    stream = torch.cuda.current_stream(dev).cuda_stream
    ws_bytes = L.scorch_hip_spmm_csr_workspace_bytes(M, nnz, N, 4)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    C = out.storage.value
    kernel_ms = (ctypes.c_float * 2)()
    merge_ms, fixup_ms = [], []
    for _ in range(args.steps):
        native.check(L.scorch_hip_spmm_csr_f32_timed(M, K, N, nnz, pos.data_ptr(), crd.data_ptr(),
                                                     val.data_ptr(), B.data_ptr(), C.data_ptr(),
                                                     ws.data_ptr(), ws.numel(), stream, kernel_ms))
        merge_ms.append(kernel_ms[0])
        fixup_ms.append(kernel_ms[1])
    merge_avg = sum(merge_ms) / len(merge_ms)
    fixup_avg = sum(fixup_ms) / len(fixup_ms)

    flops = 2.0 * nnz * N
    algo = algorithmic_bytes(M, K, N, nnz)
    achieved = algo / (merge_avg * 1e-3) / 1e9
    result = {
        "metric": "CSR SpMM GFLOP/s + HBM GB/s (% peak), power-law 1M rows, N=128 fp32",
        "value": round(flops / (ms_per_step * 1e-3) / 1e9, 2),
        "unit": "GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": WORKLOAD, "rows": M, "cols": K, "nnz": nnz, "features": N,
                   "degree": "zipf(2.1) scaled to mean 16, cap 50000, + self-loops",
                   "values": "D^-1/2 (A+I) D^-1/2", "seed": workloads.SEEDS["gcn_powerlaw"],
                   **({"neighbour_window": args.window} if args.window else {})},
        "hbm_gbps_algorithmic": round(algo / (ms_per_step * 1e-3) / 1e9, 1),
        "hbm_frac_algorithmic": round(algo / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "event_ms_per_step": round(event_ms_per_step, 4),
        "roofline": {
            "bound": "hbm", "kernel": "spmm_merge_kernel<float,2,0>" if N == 128 else "spmm_merge_kernel",
            "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES if (M, N) == (1 << 20, 128) else None,
            "algorithmic_bytes": algo, "gather_model_bytes": gather_bytes(M, N, nnz),
            "gather_model_gbps": round(gather_bytes(M, N, nnz) / (merge_avg * 1e-3) / 1e9, 1),
            "kernel_ms_avg": round(merge_avg, 4), "fixup_kernel_ms_avg": round(fixup_avg, 4),
        },
    }
    if args.vendor:
        result["vendor_library"] = vendor_spmm(pos, crd, val, B.reshape(K, N), args.steps, args.warmup)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
