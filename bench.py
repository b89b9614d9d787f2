#!/usr/bin/env python3
"""Throughput of the scatter / segment / gather hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs C1,C2,...]

Headline (`value`): configuration C5 of BASELINE.json, the largest one and the
only one whose tensors do not fit the 256 MB memory-side cache -- N = 2.4 M
nodes, E = 62.4 M edges (out-degree Zipf(1.8), mean 26), bf16 features
[., 128]. One step = gather_csr (node -> edge) + segment_csr mean (edge ->
node) + the backward of that mean, through the registered operators
(torch.ops.torch_scatter.*; the backward through autograd). Reported as
effective HBM GB/s: algorithmic bytes (every input and output tensor counted
once, 3 x 16.6 GB) divided by the wall time of K steps, inputs resident in HBM.

The same JSON line carries
  roofline      the dominant kernel of the step (the CSR reduction of the mean,
                ts::csr_reduce_kernel<bf16, 8, MEAN>), timed with HIP events on
                the launch stream, against the 8 TB/s peak; `traffic` = HBM bytes
                per launch from the tracked counter profile;
  cpu_baseline  the reference's CPU kernels (oracle/_ref, else the C oracle)
                timed on the host on a 1/4-scale slice of the same workload,
                one thread;
  configs       effective GB/s of every op of configurations C1..C5, timed the
                same way (events around back-to-back launches; inputs under
                256 MB also cold, with 1 GiB written between launches); the X-*
                rows are extra shapes (sorted index given to scatter, one value
                per entry, fused composites).

Hardware probes and dispatcher sweeps: python3 -m benchmark.hw_probes.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_GBS = 8000.0  # MI355X HBM3E


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--configs", default="C1,C2,C2m,C3,C4,C5,X",
                    help="comma list of side configurations to time (the C5 headline is always run)")
    ap.add_argument("--iters", type=int, default=20, help="launches per op in the per-config table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    return ap.parse_args()


def event_time(fn, iters, warm=3):
    """Average seconds per call, HIP events on the current stream."""
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e-3 / iters


def graph_time(fn, iters):
    """Average seconds per call when `iters` calls in a row are captured in one HIP graph (a caller that captures a
    whole step: no launch gaps between the kernels), the graph replayed four times between two events; None if the
    call cannot be captured. (A graph of one call alone is slower than eager launches: 28 against 17 us for the
    small scatter, the cost of starting a graph.)"""
    import torch
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(iters):
                fn()
        graph.replay()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(4):
            graph.replay()
        b.record()
        torch.cuda.synchronize()
        t = a.elapsed_time(b) * 1e-3 / (4 * iters)
        del graph
        return t
    except Exception as e:  # noqa: BLE001 -- a bench row, not a test
        print(f"[bench] graph capture failed: {e}", file=sys.stderr)
        return None


def cold_time(fn, iters):
    """Median seconds of a call that finds nothing of its inputs in a cache: 1 GiB is written between the
    launches (the memory-side cache holds 256 MB), each launch timed on its own."""
    import torch
    flush = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    ts_ = []
    for _ in range(max(iters, 5)):
        flush.zero_()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        ts_.append(a.elapsed_time(b) * 1e-3)
    del flush
    return sorted(ts_)[len(ts_) // 2]


CACHE_BYTES = 256 << 20  # inputs below this size stay in the memory-side cache from launch to launch


def gbs(nbytes, seconds):
    return nbytes / seconds / 1e9


def entry(nbytes, seconds, elems):
    g = gbs(nbytes, seconds)
    return {"GBps": round(g, 1), "pct_of_peak": round(100 * g / PEAK_GBS, 1), "us": round(seconds * 1e6, 1),
            "Gelem_per_s": round(elems / seconds / 1e9, 2), "MB": round(nbytes / 1e6, 1)}


# kernels behind every op of the table (the first one dominates), for the per-op roofline entries
KERNELS = {
    "segment_csr_sum": ["ts::csr_reduce_kernel"], "segment_csr_mean": ["ts::csr_reduce_kernel"],
    "segment_csr_max": ["ts::csr_reduce_kernel"], "segment_coo_max": ["ts::csr_reduce_kernel", "ts::coo_to_indptr_kernel"],
    "segment_coo_sum": ["ts::csr_reduce_kernel", "ts::coo_to_indptr_kernel"],
    "gather_csr": ["ts::csr_gather_kernel"], "gather_coo": ["ts::coo_gather_kernel"],
    "segment_csr_mean_backward": ["ts::csr_gather_kernel<DIV>"],
}


def with_roofline(e, kernels):
    """The table entry of an op plus its roofline: every kernel of the op is HBM-bound, the time is that of
    the whole launch sequence of the op (HIP events around back-to-back calls)."""
    e = dict(e)
    e["roofline"] = {"bound": "hbm", "kernels": kernels, "achieved": e["GBps"], "peak": PEAK_GBS, "unit": "GB/s",
                     "frac": round(e["GBps"] / PEAK_GBS, 4), "algorithmic_bytes": int(e["MB"] * 1e6), "us": e["us"]}
    return e


def bench_csr_config(ts, wl, w, dev, iters, ops, uniform=False, cold=False):
    """segment / gather ops of one CSR-shaped workload through the operators."""
    import torch
    s = torch.empty(0, dtype=w.dtype).element_size()
    src = wl.edge_values(w, dev, uniform=uniform)
    indptr = w.indptr.to(dev)
    index = w.index.to(dev)
    out = torch.empty((w.N, w.K), dtype=w.dtype, device=dev)
    res = {"N": w.N, "E": w.E, "K": w.K, "dtype": str(w.dtype).replace("torch.", ""),
           "mean_degree": round(w.E / w.N, 2)}
    EK = w.E * w.K
    with torch.no_grad():
        for op in ops:
            if op in ("segment_csr_sum", "segment_csr_mean"):
                r = op.rsplit("_", 1)[1]
                t = event_time(lambda: ts.segment_csr(src, indptr, out, r), iters)
                res[op] = entry(wl.bytes_segment(w.E, w.N, w.K, s), t, EK)
            elif op == "segment_csr_max":
                t = event_time(lambda: ts.segment_max_csr(src, indptr, out), iters)
                res[op] = entry(wl.bytes_segment(w.E, w.N, w.K, s, True), t, EK)
            elif op == "segment_coo_max":
                t = event_time(lambda: ts.segment_max_coo(src, index, None, w.N), iters)
                res[op] = entry(wl.bytes_segment(w.E, w.N, w.K, s, True, coo=True), t, EK)
            elif op == "segment_coo_sum":
                t = event_time(lambda: ts.segment_sum_coo(src, index, None, w.N), iters)
                res[op] = entry(wl.bytes_segment(w.E, w.N, w.K, s, coo=True), t, EK)
            elif op == "gather_csr":
                t = event_time(lambda: ts.gather_csr(out, indptr, src), iters)
                res[op] = entry(wl.bytes_gather(w.E, w.N, w.K, s), t, EK)
            elif op == "gather_coo":
                t = event_time(lambda: ts.gather_coo(out, index, src), iters)
                res[op] = entry(wl.bytes_gather(w.E, w.N, w.K, s, coo=True), t, EK)
            elif op == "segment_csr_mean_backward":
                from pytorch_scatter_amd import capi
                t = event_time(lambda: capi.segment_mean_csr_backward(out, indptr, src, 1, w.N, w.E, w.K, 0), iters)
                res[op] = entry(wl.bytes_gather(w.E, w.N, w.K, s), t, EK)
            res[op] = with_roofline(res[op], KERNELS.get(op, []))
        if cold and w.E * w.K * s < CACHE_BYTES:
            # small enough to sit in the memory-side cache between launches: also the time from HBM
            for op in ops:
                if op in ("segment_csr_sum", "segment_csr_mean"):
                    r = op.rsplit("_", 1)[1]
                    t = cold_time(lambda: ts.segment_csr(src, indptr, out, r), max(iters // 2, 5))
                    res[op + "_cold"] = entry(wl.bytes_segment(w.E, w.N, w.K, s), t, EK)
                elif op == "gather_csr":
                    t = cold_time(lambda: ts.gather_csr(out, indptr, src), max(iters // 2, 5))
                    res[op + "_cold"] = entry(wl.bytes_gather(w.E, w.N, w.K, s), t, EK)
            # and the same calls replayed from a HIP graph: what a caller with a launch-bound loop gets
            for op in ops:
                if op in ("segment_csr_sum", "segment_csr_mean"):
                    r = op.rsplit("_", 1)[1]
                    t = graph_time(lambda: ts.segment_csr(src, indptr, out, r), iters)
                    if t is not None:
                        res[op + "_graph_replay"] = entry(wl.bytes_segment(w.E, w.N, w.K, s), t, EK)
                elif op == "gather_csr":
                    t = graph_time(lambda: ts.gather_csr(out, indptr, src), iters)
                    if t is not None:
                        res[op + "_graph_replay"] = entry(wl.bytes_gather(w.E, w.N, w.K, s), t, EK)
    del src, out
    torch.cuda.empty_cache()
    return res


def bench_scatter_config(ts, wl, w, dev, iters, reduces):
    import torch
    src = wl.scatter_values(w, dev)
    index = w.index.to(dev)
    res = {"N": w.N, "E": w.E, "K": w.K, "dtype": "float32"}
    with torch.no_grad():
        for r in reduces:
            if r == "sum":
                t = event_time(lambda: ts.scatter_sum(src, index, 0, None, w.N), iters)
                res["scatter_sum"] = entry(wl.bytes_scatter(w.E, w.N, w.K, 4), t, w.E * w.K)
                if w.E * w.K * 4 < CACHE_BYTES:
                    t = cold_time(lambda: ts.scatter_sum(src, index, 0, None, w.N), max(iters // 2, 5))
                    res["scatter_sum_cold"] = entry(wl.bytes_scatter(w.E, w.N, w.K, 4), t, w.E * w.K)
                if w.E * w.K * 4 < (64 << 20):   # launch-bound sizes: the same call replayed from a HIP graph
                    t = graph_time(lambda: ts.scatter_sum(src, index, 0, None, w.N), iters)
                    if t is not None:
                        res["scatter_sum_graph_replay"] = entry(wl.bytes_scatter(w.E, w.N, w.K, 4), t, w.E * w.K)
            else:
                fn = ts.scatter_max if r == "max" else ts.scatter_min
                t = event_time(lambda: fn(src, index, 0, None, w.N), iters)
                res["scatter_" + r] = entry(wl.bytes_scatter(w.E, w.N, w.K, 4, True), t, w.E * w.K)
                if w.E * w.K * 4 < CACHE_BYTES:
                    t = cold_time(lambda: fn(src, index, 0, None, w.N), max(iters // 2, 5))
                    res["scatter_" + r + "_cold"] = entry(wl.bytes_scatter(w.E, w.N, w.K, 4, True), t, w.E * w.K)
            key = "scatter_" + r
            res[key] = with_roofline(res[key], ["ts::scatter_* (see profiles/bench_kernel_trace_stats.txt)"])
    del src
    torch.cuda.empty_cache()
    return res


def bench_sorted_config(ts, wl, w, dev, iters):
    """The same scatter through an index sorted once (SortedIndex + scatter_sorted): the one-time sort, then
    sum / max as a segmented reduction over permuted rows. Bytes as for scatter plus 4 per entry for perm."""
    import torch
    src = wl.scatter_values(w, dev)
    index = w.index.to(dev)
    res = {"N": w.N, "E": w.E, "K": w.K, "dtype": "float32"}
    t = event_time(lambda: ts.SortedIndex(index, w.N), max(iters // 2, 3))
    res["sort_index_us"] = round(t * 1e6, 1)
    plan = ts.SortedIndex(index, w.N)
    with torch.no_grad():
        t = event_time(lambda: ts.scatter_sorted(src, plan, 0, "sum"), iters)
        res["scatter_sorted_sum"] = entry(wl.bytes_scatter(w.E, w.N, w.K, 4) + 4 * w.E, t, w.E * w.K)
        t = event_time(lambda: ts.scatter_sorted(src, plan, 0, "max"), iters)
        res["scatter_sorted_max"] = entry(wl.bytes_scatter(w.E, w.N, w.K, 4, True) + 4 * w.E, t, w.E * w.K)
    del src, plan
    torch.cuda.empty_cache()
    return res


def bench_softmax_config(ts, wl, w, dev, iters, K):
    """scatter_softmax and scatter_std over the destination index of the C3 graph with K values per entry (attention
    heads), sorted and in random order; bytes: src read once, index read once, result written once."""
    import torch
    index = w.index.to(dev)
    shuffled = index[torch.randperm(w.E, device=dev)]
    src = torch.randn((w.E, K), device=dev)
    grad = torch.randn((w.E, K), device=dev)
    res = {"N": w.N, "E": w.E, "K": K, "dtype": "float32"}
    fwd_bytes = 2 * w.E * K * 4 + w.E * 8
    bwd_bytes = 3 * w.E * K * 4 + w.E * 8
    for name, idx in (("sorted", index), ("unsorted", shuffled)):
        with torch.no_grad():
            t = event_time(lambda: ts.scatter_softmax(src, idx, 0, w.N), iters)
        res[f"softmax_{name}"] = entry(fwd_bytes, t, w.E * K)
        x = src.clone().requires_grad_(True)
        y = ts.scatter_softmax(x, idx, 0, w.N)
        t = event_time(lambda: torch.autograd.grad(y, x, grad, retain_graph=True), iters)
        res[f"softmax_backward_{name}"] = entry(bwd_bytes, t, w.E * K)
        del x, y
        # std: src read twice (group sums, then squared deviations), index twice, N*K result
        with torch.no_grad():
            t = event_time(lambda: ts.scatter_std(src, idx, 0, None, w.N), iters)
        res[f"std_{name}"] = entry(2 * (w.E * K * 4 + w.E * 8) + w.N * K * 4, t, w.E * K)
        x = src.clone().requires_grad_(True)
        y = ts.scatter_std(x, idx, 0, None, w.N)
        gn = grad[:w.N].contiguous()
        t = event_time(lambda: torch.autograd.grad(y, x, gn, retain_graph=True), iters)
        res[f"std_backward_{name}"] = entry(2 * w.E * K * 4 + w.E * 8, t, w.E * K)
        del x, y
        # logsumexp: src and index read once, N*K result
        with torch.no_grad():
            t = event_time(lambda: ts.scatter_logsumexp(src, idx, 0, None, w.N), iters)
        res[f"logsumexp_{name}"] = entry(w.E * K * 4 + w.E * 8 + w.N * K * 4, t, w.E * K)
    del src, grad
    torch.cuda.empty_cache()
    return res


def load_ref_ops():
    """The reference's own CPU kernels (oracle/_ref) as torch.ops.ts_ref, or None when they are not built."""
    import torch
    ref_path = os.path.join(ROOT, "oracle", "_ref", "libts_ref_cpu.so")
    if not os.path.exists(ref_path):
        return None
    try:
        torch.ops.load_library(ref_path)
        return torch.ops.ts_ref
    except Exception:  # built against another torch: the C restatement serves instead
        return None


def cpu_baseline(wl, scale=1.0 / 4):
    """The three ops of the C5 step on the host, single thread, on a slice of the workload (the same
    generator with N scaled down: same degree distribution, same cap rule, bf16): the reference's own CPU kernels
    when oracle/_ref is built, else the C restatement. The backward follows csrc/segment_csr.cpp:93-109: gather
    of the gradient, gather of the counts, one division."""
    import torch
    torch.set_num_threads(1)
    w = wl.c5_gnn(scale)
    g = torch.Generator().manual_seed(0)
    x = torch.randn((w.N, w.K), generator=g).to(w.dtype)
    src = torch.empty((w.E, w.K), dtype=w.dtype)
    for s0 in range(0, w.E, 1 << 20):
        src[s0:s0 + (1 << 20)] = torch.randn((min(1 << 20, w.E - s0), w.K), generator=g).to(w.dtype)
    grad = torch.randn((w.N, w.K), generator=g).to(w.dtype)
    out = torch.empty((w.N, w.K), dtype=w.dtype)
    msg = torch.empty_like(src)
    count = (w.indptr[1:] - w.indptr[:-1]).to(w.dtype)
    ops = load_ref_ops()
    kind = "reference" if ops is not None else "port"
    if ops is not None:
        def run():
            ops.gather_csr(x, w.indptr, msg)
            ops.segment_csr(src, w.indptr, out, "mean")
            ops.gather_csr(grad, w.indptr, msg)
            msg.true_divide_(ops.gather_csr(count, w.indptr, None).unsqueeze(-1))
    else:
        import ts_oracle

        def run():
            ts_oracle.gather_csr(x, w.indptr, msg)
            ts_oracle.segment_csr(src, w.indptr, out, "mean")
            ts_oracle.gather_csr(grad, w.indptr, msg)
            msg.true_divide_(ts_oracle.gather_csr(count, w.indptr, None).unsqueeze(-1))
    run()
    reps = 4
    t0 = time.perf_counter()
    for _ in range(reps):
        run()
    dt = (time.perf_counter() - t0) / reps
    s = 2
    nbytes = 2 * wl.bytes_gather(w.E, w.N, w.K, s) + wl.bytes_segment(w.E, w.N, w.K, s)
    return {"value": round(gbs(nbytes, dt), 3), "unit": "GB/s", "cores": 1, "kind": kind,
            "host_cores_available": os.cpu_count(),
            "sample": f"1/{round(1 / scale)} slice of C5 (N={w.N}, E={w.E}, K={w.K}, bf16: the same generator with "
                      f"the node count scaled), {reps} passes of gather_csr + segment_csr mean + mean backward "
                      f"(gather, gather of counts, divide), {dt * 1e3:.0f} ms per pass"}


def cpu_baselines_other(wl):
    """The reference's CPU kernels (oracle/_ref, else the C oracle) on the other configurations, one thread: C1 in
    full (the configuration BASELINE.json names "on CPU reference"), C2 in full, C4 with one value per entry in
    full, C3 on a slice of 1/16 of its segments (the full input is 4.6 GB)."""
    import torch
    torch.set_num_threads(1)
    ops = load_ref_ops()
    kind = "reference" if ops is not None else "port"
    import ts_oracle

    def scatter(src, index, N, reduce):
        idx = index.view(-1, 1).expand_as(src)
        if ops is not None:
            return ops.scatter(src, idx, 0, None, N, reduce)
        return ts_oracle.scatter(src, idx, 0, None, N, reduce)

    def segment_coo(src, index, N, reduce):
        if ops is not None:
            return ops.segment_coo(src, index, None, N, reduce)
        return ts_oracle.segment_coo(src, index, None, N, reduce)

    def timed(fn, reps):
        fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps

    out = {}
    g = torch.Generator().manual_seed(0)
    w1 = wl.c1_scatter_sum()
    src = torch.randn((w1.E, w1.K), generator=g)
    dt = timed(lambda: scatter(src, w1.index, w1.N, "sum"), 20)
    out["C1"] = {"value": round(gbs(wl.bytes_scatter(w1.E, w1.N, w1.K, 4), dt), 3), "unit": "GB/s", "cores": 1,
                 "kind": kind, "host_cores_available": os.cpu_count(),
                 "sample": f"full C1 (scatter sum, E={w1.E}, N={w1.N}, K={w1.K}, fp32), 20 passes, {dt * 1e3:.2f} ms per pass"}
    w4 = wl.c4_scatter_minmax(1)
    src = torch.randn((w4.E, 1), generator=g)
    dt = timed(lambda: scatter(src, w4.index, w4.N, "max"), 3)
    out["C4-K1"] = {"value": round(gbs(wl.bytes_scatter(w4.E, w4.N, 1, 4, True), dt), 3), "unit": "GB/s", "cores": 1,
                    "kind": kind, "host_cores_available": os.cpu_count(),
                    "sample": f"full C4 with one value per entry (scatter max + arg, E={w4.E}, N={w4.N}), 3 passes, "
                              f"{dt * 1e3:.1f} ms per pass"}
    w2 = wl.c2_segment_csr()
    src = torch.randn((w2.E, w2.K), generator=g)
    o2, b2 = torch.empty((w2.N, w2.K)), torch.empty((w2.E, w2.K))

    def c2_step():
        for r in ("sum", "mean"):
            (ops.segment_csr if ops is not None else ts_oracle.segment_csr)(src, w2.indptr, o2, r)
        (ops.gather_csr if ops is not None else ts_oracle.gather_csr)(o2, w2.indptr, b2)
    dt = timed(c2_step, 5)
    out["C2"] = {"value": round(gbs(2 * wl.bytes_segment(w2.E, w2.N, w2.K, 4) + wl.bytes_gather(w2.E, w2.N, w2.K, 4), dt), 3),
                 "unit": "GB/s", "cores": 1, "kind": kind, "host_cores_available": os.cpu_count(),
                 "sample": f"full C2 (segment_csr sum + mean + gather_csr, E={w2.E}, N={w2.N}, K={w2.K}, fp32), 5 passes, "
                           f"{dt * 1e3:.1f} ms per pass"}
    w3 = wl.c3_segment_coo(scale=1.0 / 16)
    src = torch.rand((w3.E, w3.K), generator=g) * 2 - 1
    dt = timed(lambda: segment_coo(src, w3.index, w3.N, "max"), 3)
    out["C3"] = {"value": round(gbs(wl.bytes_segment(w3.E, w3.N, w3.K, 4, True, coo=True), dt), 3), "unit": "GB/s",
                 "cores": 1, "kind": kind, "host_cores_available": os.cpu_count(),
                 "sample": f"1/16 of C3 (segment_coo max + arg, E={w3.E}, N={w3.N}, K={w3.K}, fp32), 3 passes, "
                           f"{dt * 1e3:.1f} ms per pass"}
    return out


def measured_traffic(key):
    """HBM bytes per launch of a kernel as the tracked counter profile states them (a line
    `<key>: <number>` in profiles/csr_reduce_pmc_traffic.txt), or None."""
    import re
    try:
        text = open(os.path.join(ROOT, "profiles", "csr_reduce_pmc_traffic.txt")).read()
    except OSError:
        return None
    m = re.search(r"^" + re.escape(key) + r":\s*([0-9.eE+]+)", text, re.M)
    return float(m.group(1)) if m else None


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; every box of this run has a single MI355X, "
              "so --gpus above 1 is not supported (segment / gather ops would shard by node range "
              "without any exchange).", file=sys.stderr)
        sys.exit(2)
    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    import pytorch_scatter_amd as ts
    from pytorch_scatter_amd import workloads as wl
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # ---------------- headline: C5 through the registered operators (HBM-resident: 16.6 GB per op)
    w5 = wl.c5_gnn()
    indptr = w5.indptr.to(dev)
    g = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn((w5.N, w5.K), generator=g, device=dev).to(w5.dtype)          # node features
    grad_out = torch.randn((w5.N, w5.K), generator=g, device=dev).to(w5.dtype)   # gradient of the mean
    src = wl.edge_values(w5, dev).requires_grad_(True)                           # edge features
    msg = torch.empty((w5.E, w5.K), dtype=w5.dtype, device=dev)                  # node -> edge messages
    out = torch.empty((w5.N, w5.K), dtype=w5.dtype, device=dev)
    op_bytes = {"gather_csr": wl.bytes_gather(w5.E, w5.N, w5.K, 2),
                "segment_csr_mean": wl.bytes_segment(w5.E, w5.N, w5.K, 2),
                "segment_csr_mean_backward": wl.bytes_gather(w5.E, w5.N, w5.K, 2)}
    step_bytes = sum(op_bytes.values())

    def step():
        with torch.no_grad():
            ts.gather_csr(x, indptr, msg)
        y = ts.segment_csr(src, indptr, None, "mean")
        (gin,) = torch.autograd.grad(y, src, grad_out)   # the fused gather-and-divide kernel, 16 GB written
        return gin

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    # dominant kernel: the CSR reduction of the mean (one launch per call), HIP events on the launch stream
    with torch.no_grad():
        t_kernel = event_time(lambda: ts.segment_csr(src, indptr, out, "mean"), max(args.steps, 10))
    kernel_bytes = op_bytes["segment_csr_mean"]
    # HBM bytes per launch of this kernel from rocprofv3 --pmc (memory-side read / write requests by size):
    # read from the tracked profile, null if that file does not state it
    traffic = measured_traffic("traffic_bytes_per_launch_c5_mean")
    roofline = {"bound": "hbm", "kernel": "ts::csr_reduce_kernel<bf16, 8, MEAN> (segment_csr mean of C5)",
                "achieved": round(gbs(kernel_bytes, t_kernel), 1), "peak": PEAK_GBS, "unit": "GB/s",
                "frac": round(gbs(kernel_bytes, t_kernel) / PEAK_GBS, 4), "traffic": traffic,
                "algorithmic_bytes_per_launch": kernel_bytes, "us_per_launch": round(t_kernel * 1e6, 1)}
    del src, msg, out, x, grad_out
    torch.cuda.empty_cache()
    w2 = wl.c2_segment_csr()

    # ---------------- side table: every configuration
    want = set(args.configs.split(",")) if args.configs else set()
    table = {}
    it = args.iters
    if "C1" in want:
        table["C1"] = bench_scatter_config(ts, wl, wl.c1_scatter_sum(), dev, it, ["sum"])
    if "C2" in want:
        table["C2"] = bench_csr_config(ts, wl, w2, dev, it, ["segment_csr_sum", "segment_csr_mean", "gather_csr"],
                                       cold=True)
    if "C2m" in want:
        table["C2-mean16"] = bench_csr_config(ts, wl, wl.c2_segment_csr(mean16=True), dev, it,
                                              ["segment_csr_sum", "segment_csr_mean", "gather_csr"], cold=True)
    if "C3" in want:
        table["C3"] = bench_csr_config(ts, wl, wl.c3_segment_coo(), dev, it, ["segment_coo_max"], uniform=True)
    if "C4" in want:
        for K in (1, 32):
            table[f"C4-K{K}"] = bench_scatter_config(ts, wl, wl.c4_scatter_minmax(K), dev, max(it // 2, 3),
                                                     ["max", "min"])
    if "C5" in want:
        table["C5"] = bench_csr_config(ts, wl, wl.c5_gnn(), dev, max(it // 2, 3),
                                       ["gather_csr", "segment_csr_mean", "segment_csr_mean_backward"])

    if "X" in want:
        # not BASELINE configurations: the graph of C3 with a sorted index given to scatter (the usual
        # message-passing call) and with one value per entry (attention scores, degrees)
        import dataclasses
        w3 = wl.c3_segment_coo()
        sw = wl.ScatterWorkload("X-sorted-K64", w3.index, w3.N, w3.E, 64, torch.float32)
        table["X-sorted-K64"] = bench_scatter_config(ts, wl, sw, dev, max(it // 2, 3), ["sum", "max"])
        # the same entries in random order: the hubs of a power-law index no longer form runs and every
        # entry of a hub meets the others on one address unless the kernel keeps its hot rows in LDS
        g = torch.Generator().manual_seed(0)
        wz = wl.c4_scatter_minmax(1)
        zipf_index = wz.index[torch.randperm(wz.E, generator=g)] * 10 % 1_000_000
        sz = wl.ScatterWorkload("X-zipf-unsorted-K8", zipf_index, 1_000_000, wz.E, 8, torch.float32)
        table["X-zipf-unsorted-K8"] = bench_scatter_config(ts, wl, sz, dev, max(it // 2, 3), ["sum", "max"])
        sw32 = dataclasses.replace(wl.c4_scatter_minmax(32), name="X-zipf-unsorted-K32")
        table["X-zipf-unsorted-K32"] = bench_scatter_config(ts, wl, sw32, dev, max(it // 2, 3), ["sum"])
        # few entries per output row (ten on average), unsorted: uniform index and the Zipf index from above
        uni = torch.randint(0, 1_000_000, (wz.E,), generator=g)
        su = wl.ScatterWorkload("X-uniform-deg10-K64", uni, 1_000_000, wz.E, 64, torch.float32)
        table["X-uniform-deg10-K64"] = bench_scatter_config(ts, wl, su, dev, max(it // 2, 3), ["sum", "max"])
        # narrow rows under the same uniform index: two floats per entry (values travel in binned words), and one
        # float per entry at a tenth of the size (a table per workgroup, handed over in slabs)
        su2 = wl.ScatterWorkload("X-uniform-deg10-K2", uni, 1_000_000, wz.E, 2, torch.float32)
        table["X-uniform-deg10-K2"] = bench_scatter_config(ts, wl, su2, dev, max(it // 2, 3), ["sum"])
        su1 = wl.ScatterWorkload("X-uniform-deg10-K1-1M", uni[:1_000_000] % 100_000, 100_000, 1_000_000, 1, torch.float32)
        table["X-uniform-deg10-K1-1M"] = bench_scatter_config(ts, wl, su1, dev, max(it // 2, 3), ["sum"])
        sz64 = wl.ScatterWorkload("X-zipf-unsorted-K64", zipf_index, 1_000_000, wz.E, 64, torch.float32)
        table["X-zipf-unsorted-K64"] = bench_scatter_config(ts, wl, sz64, dev, max(it // 2, 3), ["sum", "max"])
        table["X-sorted-plan-C4-K32"] = bench_sorted_config(ts, wl, wl.c4_scatter_minmax(32), dev, max(it // 2, 3))
        ss = wl.ScatterWorkload("X-sorted-plan-C3-shuffled-K64", w3.index[torch.randperm(w3.E, generator=g)], w3.N, w3.E,
                                64, torch.float32)
        table["X-sorted-plan-C3-shuffled-K64"] = bench_sorted_config(ts, wl, ss, dev, max(it // 2, 3))
        table["X-softmax-K8"] = bench_softmax_config(ts, wl, w3, dev, max(it // 2, 3), 8)
        table["X-narrow-K1"] = bench_csr_config(ts, wl, dataclasses.replace(w3, K=1, name="X-narrow-K1"), dev, it,
                                                ["segment_csr_sum", "segment_csr_max", "segment_coo_sum",
                                                 "gather_csr", "gather_coo"], uniform=True)

    cpu = None if args.no_cpu else cpu_baseline(wl)
    cpu_other = None if args.no_cpu else cpu_baselines_other(wl)

    line = {
        "metric": "effective HBM GB/s, gather_csr + segment_csr mean + mean backward (BASELINE config C5), 1 MI355X",
        "value": round(gbs(step_bytes, dt), 1),
        "unit": "GB/s",
        "pct_of_8TBps_peak": round(100 * gbs(step_bytes, dt) / PEAK_GBS, 1),
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "C5: gather_csr (node->edge) + segment_csr mean (edge->node) + mean backward; "
                               "N=2.4M nodes, out-degree Zipf(1.8) capped for mean 26, features bf16 [., 128], "
                               "numpy default_rng(0)",
                   "N": w5.N, "E": w5.E, "K": w5.K, "algorithmic_bytes_per_step": step_bytes,
                   "algorithmic_bytes_per_op": op_bytes,
                   "api": "torch.ops.torch_scatter.* (eager; backward through autograd)"},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "cpu_baselines_other_configs": cpu_other,
        "configs": table,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
