#!/usr/bin/env python3
"""Throughput of the scatter / segment / gather hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs C1,C2,...]

Headline (`value`): configuration C2 of BASELINE.json -- segment_csr sum,
segment_csr mean and gather_csr of the result back to the edges, 100000
segments with Zipf(2.0) degrees, fp32 [E, 64] -- as effective HBM GB/s:
algorithmic bytes (every input and output tensor counted once) divided by the
wall time of K steps, inputs resident in HBM, called through the registered
operators (torch.ops.torch_scatter.*). One step = the three ops once.

The same JSON line carries
  roofline      the dominant kernel of the headline (the CSR reduction), timed
                with HIP events on the launch stream, against the 8 TB/s peak;
  cpu_baseline  the reference's CPU kernels (oracle/_ref, else the C oracle)
                timed on the host for the same workload, one thread;
  configs       effective GB/s of every op of configurations C1..C5, timed the
                same way (events around back-to-back launches); the X-* rows are
                extra shapes (sorted index given to scatter, one value per entry).
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
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--configs", default="C1,C2,C2m,C3,C4,C5,X",
                    help="comma list of side configurations to time (C2 is always run)")
    ap.add_argument("--iters", type=int, default=20, help="launches per op in the per-config table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--probe-scatter", action="store_true",
                    help="launch sequence for the L2 / atomic counters of the scatter kernels (see probe_scatter)")
    ap.add_argument("--probe-ceilings", action="store_true",
                    help="plain read / write / copy / mixed streams over several GiB: what the memory system of this "
                         "device sustains (the ceilings the kernels are held against), nothing else is run")
    ap.add_argument("--probe-atomics", action="store_true",
                    help="rate of device-scope 64-bit atomics on scattered and on neighbouring addresses")
    ap.add_argument("--sweep-thresholds", action="store_true",
                    help="time scatter sum / max just either side of every size threshold of the dispatcher and "
                         "flag neighbours that differ by more than 1.5x")
    ap.add_argument("--sweep-orders", action="store_true",
                    help="scatter sum / max for one shape under a sorted, a shuffled and a skewed index, fp32 and bf16; "
                         "flags a sorted index that is slower than a shuffled one and 16-bit types far behind fp32")
    ap.add_argument("--probe", action="store_true",
                    help="counter-collection mode for rocprofv3 --pmc: a few launches of the dominant kernels "
                         "next to copies of known size, nothing timed")
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
    del src, grad
    torch.cuda.empty_cache()
    return res


def cpu_baseline(wl, w):
    """The same three ops of C2 on the host, single thread: the reference's own
    CPU kernels when oracle/_ref is built, else the C restatement."""
    import torch
    torch.set_num_threads(1)
    g = torch.Generator().manual_seed(0)
    src = torch.randn((w.E, w.K), generator=g, dtype=torch.float32)
    out = torch.empty((w.N, w.K), dtype=torch.float32)
    back = torch.empty_like(src)
    kind = "port"
    ref_path = os.path.join(ROOT, "oracle", "_ref", "libts_ref_cpu.so")
    run = None
    if os.path.exists(ref_path):
        try:
            torch.ops.load_library(ref_path)
            ops = torch.ops.ts_ref

            def run():
                ops.segment_csr(src, w.indptr, out, "sum")
                ops.segment_csr(src, w.indptr, out, "mean")
                ops.gather_csr(out, w.indptr, back)
            run()
            kind = "reference"
        except Exception:  # library built against another torch: fall back to the port
            run = None
    if run is None:
        import ts_oracle

        def run():
            ts_oracle.segment_csr(src, w.indptr, out, "sum")
            ts_oracle.segment_csr(src, w.indptr, out, "mean")
            ts_oracle.gather_csr(out, w.indptr, back)
        run()
    reps = 5
    t0 = time.perf_counter()
    for _ in range(reps):
        run()
    dt = (time.perf_counter() - t0) / reps
    nbytes = 2 * wl.bytes_segment(w.E, w.N, w.K, 4) + wl.bytes_gather(w.E, w.N, w.K, 4)
    return {"value": round(gbs(nbytes, dt), 3), "unit": "GB/s", "cores": 1, "kind": kind,
            "host_cores_available": os.cpu_count(),
            "sample": f"full C2 workload (E={w.E}, N={w.N}, K={w.K}, fp32), {reps} passes of "
                      f"segment_csr sum + mean + gather_csr, {dt * 1e3:.1f} ms per pass"}


def cpu_baselines_other(wl):
    """The reference's CPU kernels (oracle/_ref, else the C oracle) on the scatter / segment_coo configurations, one
    thread: C1 in full (the configuration BASELINE.json names "on CPU reference"), C4 with one value per entry
    in full, C3 on a slice of 1/16 of its segments (the full input is 4.6 GB)."""
    import torch
    torch.set_num_threads(1)
    ref_path = os.path.join(ROOT, "oracle", "_ref", "libts_ref_cpu.so")
    ops, kind = None, "port"
    if os.path.exists(ref_path):
        try:
            torch.ops.load_library(ref_path)
            ops, kind = torch.ops.ts_ref, "reference"
        except Exception:
            ops = None
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
    w3 = wl.c3_segment_coo(scale=1.0 / 16)
    src = torch.rand((w3.E, w3.K), generator=g) * 2 - 1
    dt = timed(lambda: segment_coo(src, w3.index, w3.N, "max"), 3)
    out["C3"] = {"value": round(gbs(wl.bytes_segment(w3.E, w3.N, w3.K, 4, True, coo=True), dt), 3), "unit": "GB/s",
                 "cores": 1, "kind": kind, "host_cores_available": os.cpu_count(),
                 "sample": f"1/16 of C3 (segment_coo max + arg, E={w3.E}, N={w3.N}, K={w3.K}, fp32), 3 passes, "
                           f"{dt * 1e3:.1f} ms per pass"}
    return out


def measured_traffic():
    """HBM bytes per launch of the headline kernel as the tracked counter profile states them (a line
    `traffic_bytes_per_launch: <number>` in profiles/csr_reduce_pmc_traffic.txt), or None."""
    import re
    try:
        text = open(os.path.join(ROOT, "profiles", "csr_reduce_pmc_traffic.txt")).read()
    except OSError:
        return None
    m = re.search(r"traffic_bytes_per_launch:\s*([0-9.eE+]+)", text)
    return float(m.group(1)) if m else None


def probe_ceilings():
    """Plain streams through libts_probe.so (pytorch_scatter_amd/csrc/probe.hip): read, write, copy and reads mixed
    with writes 3:1 and 26:1, over GiB-sized buffers, HIP events around 10 launches each."""
    import ctypes
    import torch
    lib = ctypes.CDLL(os.path.join(ROOT, "pytorch_scatter_amd", "libts_probe.so"))
    lib.ts_probe_stream.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    dev = torch.device("cuda:0")
    a = torch.empty(6 << 30, dtype=torch.uint8, device=dev)
    b = torch.empty(4 << 30, dtype=torch.uint8, device=dev)
    a.fill_(1)
    b.fill_(2)
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for name, mode, wbytes in (("read only (non-temporal 16-byte loads)", 0, 4 << 30), ("write only", 1, 4 << 30),
                               ("copy 1:1", 2, 3 << 30), ("read 3 : write 1", 4, 2 << 30),
                               ("read 26 : write 1", 27, 224 << 20)):
        rd = 0 if mode == 1 else (wbytes if mode == 0 else (mode - 1) * wbytes)
        wr = 0 if mode == 0 else wbytes
        t = event_time(lambda: lib.ts_probe_stream(mode, a.data_ptr(), b.data_ptr(), wbytes, stream), 10, warm=2)
        rows.append({"stream": name, "read_GB": round(rd / 1e9, 2), "written_GB": round(wr / 1e9, 2),
                     "us": round(t * 1e6, 1), "GBps": round((rd + wr) / t / 1e9, 1),
                     "pct_of_peak": round(100 * (rd + wr) / t / 1e9 / PEAK_GBS, 1)})
    t = event_time(lambda: b[:3 << 30].copy_(a[:3 << 30]), 10, warm=2)
    rows.append({"stream": "torch copy_ 1:1", "read_GB": 3.22, "written_GB": 3.22, "us": round(t * 1e6, 1),
                 "GBps": round(2 * (3 << 30) / t / 1e9, 1), "pct_of_peak": round(100 * 2 * (3 << 30) / t / 1e9 / PEAK_GBS, 1)})
    for r in rows:
        print(f"{r['stream']:42s} read {r['read_GB']:6.2f} GB  written {r['written_GB']:6.2f} GB  {r['us']:9.1f} us  "
              f"{r['GBps']:7.1f} GB/s  {r['pct_of_peak']:5.1f} % of 8 TB/s", file=sys.stderr)
    print(json.dumps({"probe": "ceilings", "rows": rows}))


def probe_atomics():
    """Rate of device-scope 64-bit atomics (libts_probe.so): scattered addresses (one transaction per lane) and
    neighbouring addresses shared by all workgroups (a table written back by every workgroup at once)."""
    import ctypes
    import torch
    lib = ctypes.CDLL(os.path.join(ROOT, "pytorch_scatter_amd", "libts_probe.so"))
    lib.ts_probe_atomics.restype = ctypes.c_longlong
    lib.ts_probe_atomics.argtypes = [ctypes.c_void_p, ctypes.c_uint, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    dev = torch.device("cuda:0")
    table = torch.zeros(1 << 20, dtype=torch.int64, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for name, slots, iters, pattern in (("scattered, 100 k slots, 1 M atomics", 100_000, 4, 0),
                                        ("scattered, 100 k slots, 4 M atomics", 100_000, 16, 0),
                                        ("scattered, 1 M slots, 4 M atomics", 1_000_000, 16, 0),
                                        ("4096 neighbouring slots from each of 256 workgroups", 4096, 1, 1),
                                        ("8192 neighbouring slots from each of 256 workgroups", 8192, 1, 1)):
        n = lib.ts_probe_atomics(table.data_ptr(), slots, iters, pattern, stream)
        t = event_time(lambda: lib.ts_probe_atomics(table.data_ptr(), slots, iters, pattern, stream), 10, warm=2)
        rows.append({"pattern": name, "atomics": n, "us": round(t * 1e6, 1), "G_atomics_per_s": round(n / t / 1e9, 1)})
    for r in rows:
        print(f"{r['pattern']:56s} {r['atomics']:9d} atomics {r['us']:8.1f} us {r['G_atomics_per_s']:7.1f} G/s", file=sys.stderr)
    print(json.dumps({"probe": "atomics", "rows": rows}))


def sweep_thresholds():
    """scatter sum / max through the operators at sizes just either side of every size threshold of the dispatcher
    (pytorch_scatter_amd/csrc/scatter.h, scatter_binned.h, scatter_k1.h): neighbours that differ by more than 1.5x in time
    per entry are flagged. Index: Zipf(1.2) over N rows, shuffled."""
    import numpy as np
    import torch
    import pytorch_scatter_amd as ts
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(0)

    def zipf_index(E, N):
        p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
        return torch.from_numpy(rng.choice(N, size=E, p=p / p.sum()).astype(np.int64)).to(dev)

    # (what, K, N, sizes in entries around the threshold); N a list: 2 M entries, output rows around the threshold
    M = 1 << 20
    cases = [
        ("sum: LDS table from 2^16 elements (K = 16)", "sum", 16, 1000, [M // 256 - 512, M // 256 + 512]),
        ("sum: LDS table from 2^18 elements for rows of 33-64 columns (K = 64)", "sum", 64, 100_000,
         [M // 256 - 256, M // 256 + 256]),
        ("sum: LDS table from 2^19 elements for rows above 64 columns (K = 128)", "sum", 128, 100_000,
         [M // 256 - 256, M // 256 + 256]),
        ("sum: sample of the index from 2^23 elements (K = 8)", "sum", 8, 1_000_000, [M - 65536, M + 65536]),
        ("sum: buckets of output rows from 64 MB (K = 32)", "sum", 32, 100_000, [M // 2 - 16384, M // 2 + 16384]),
        ("max: LDS table from 2^20 elements (contended index)", "max", 8, 1000, [M // 8 - 4096, M // 8 + 4096]),
        ("max: one value per entry, slabs from 2^14 entries", "max", 1, 100_000, [M // 64 - 1024, M // 64 + 1024]),
        ("max: buckets of output rows from 24 MB (K = 32, keys of 25 MB)", "max", 32, 100_000,
         [3 * M // 16 - 8192, 3 * M // 16 + 8192]),
        ("max: buckets of output rows from 64 MB (K = 32, keys of 2.5 MB)", "max", 32, 10_000,
         [M // 2 - 16384, M // 2 + 16384]),
        ("max: parts of 4 / 8 / 16 entries by the number of wavefronts (K = 32)", "max", 32, 100_000,
         [M // 8 - 8192, M // 8 + 8192]),
        ("max: sample of the index from 2^23 elements (K = 8)", "max", 8, 1_000_000, [M - 65536, M + 65536]),
        ("sum: rows in slices of columns above 16384 buckets (K = 128)", "sum", 128, [M - 8192, M + 8192], None),
        ("max: rows in slices of columns above 16384 buckets (K = 128)", "max", 128, [M - 8192, M + 8192], None),
    ]
    rows, flagged = [], 0
    with torch.no_grad():
        for what, reduce, K, N, sizes in cases:
            per_entry = []
            points = [(E, N) for E in sizes] if sizes is not None else [(2 * M, n) for n in N]
            for E, N in points:
                index = zipf_index(E, N)
                src = torch.randn((E, K), device=dev)
                fn = ts.scatter_sum if reduce == "sum" else ts.scatter_max
                t = event_time(lambda: fn(src, index, 0, None, N), 10)
                per_entry.append(t / E)
                rows.append({"threshold": what, "E": E, "K": K, "N": N, "us": round(t * 1e6, 1),
                             "ns_per_entry": round(t / E * 1e9, 4)})
                del src, index
            ratio = max(per_entry) / min(per_entry)
            rows[-1]["ratio_across_threshold"] = round(ratio, 2)
            rows[-1]["cliff"] = ratio > 1.5
            flagged += ratio > 1.5
    for r in rows:
        print(r, file=sys.stderr)
    print(json.dumps({"probe": "thresholds", "cliffs": flagged, "rows": rows}))


def sweep_orders():
    """scatter sum / max through the operators for the same shape under a sorted, a shuffled and a Zipf(1.2) index,
    fp32 and bf16: the thresholds of the dispatcher are sizes, and a kernel picked by size can be the wrong one for
    the order of the index or for the element type (found that way: the accumulator table for narrow rows was
    twice as slow as the run kernel under a sorted index, and 30-300x slower for 16-bit floats under any other).
    Flags: a sorted index more than 1.5x slower than the same index shuffled; bf16 more than 8x slower than fp32."""
    import numpy as np
    import torch
    import pytorch_scatter_amd as ts
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(0)
    rows, flagged = [], 0
    with torch.no_grad():
        for E, N in ((4_000_000, 400_000), (4_000_000, 4_000), (500_000, 50_000)):
            uni = rng.integers(0, N, size=E)
            p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
            zipf = rng.choice(N, size=E, p=p / p.sum())
            orders = {"sorted": np.sort(uni), "shuffled": uni, "zipf": zipf}
            index = {k: torch.from_numpy(v.astype(np.int64)).to(dev) for k, v in orders.items()}
            for K in (1, 8, 32):
                t = {}
                for dtype in (torch.float32, torch.bfloat16):
                    src = torch.randn((E, K), device=dev).to(dtype)
                    for order, idx in index.items():
                        for reduce, fn in (("sum", ts.scatter_sum), ("max", ts.scatter_max)):
                            t[dtype, order, reduce] = event_time(lambda: fn(src, idx, 0, None, N), 5)
                    del src
                for (dtype, order, reduce), v in t.items():
                    slow_sorted = order == "sorted" and v > 1.5 * t[dtype, "shuffled", reduce]
                    slow_16 = dtype == torch.bfloat16 and v > 8 * t[torch.float32, order, reduce]
                    rows.append({"E": E, "N": N, "K": K, "dtype": str(dtype)[6:], "order": order, "reduce": reduce,
                                 "us": round(v * 1e6, 1), "flag": bool(slow_sorted or slow_16)})
                    flagged += bool(slow_sorted or slow_16)
    for r in rows:
        print(r, file=sys.stderr)
    print(json.dumps({"probe": "orders", "flagged": flagged, "rows": rows}))


def probe():
    """Launch sequence for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE -- python3 bench.py --probe`:
    1. torch copy of 1 GiB (plain loads/stores, known size: calibrates the counters);
    2. segment_csr sum with one entry per segment over 1 GiB of fp32 [4Mi, 64]: a copy through the
       reduction kernel itself (same non-temporal loads), known size;
    3. C2 segment_csr sum x3, C5 segment_csr mean x2, C5 gather_csr x2."""
    import torch
    import pytorch_scatter_amd as ts
    from pytorch_scatter_amd import workloads as wl
    dev = torch.device("cuda:0")
    a = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    b = torch.empty_like(a)
    b.copy_(a)
    n = 1 << 22
    x = torch.ones((n, 64), dtype=torch.float32, device=dev)
    ident = torch.arange(n + 1, device=dev)
    y = torch.empty_like(x)
    with torch.no_grad():
        ts.segment_csr(x, ident, y, "sum")
        del a, b, x, y
        w2 = wl.c2_segment_csr()
        src = wl.edge_values(w2, dev)
        out = torch.empty((w2.N, w2.K), dtype=torch.float32, device=dev)
        for _ in range(3):
            ts.segment_csr(src, w2.indptr.to(dev), out, "sum")
        del src, out
        w5 = wl.c5_gnn()
        src = wl.edge_values(w5, dev)
        out = torch.empty((w5.N, w5.K), dtype=torch.bfloat16, device=dev)
        ip = w5.indptr.to(dev)
        for _ in range(2):
            ts.segment_csr(src, ip, out, "mean")
        for _ in range(2):
            ts.gather_csr(out, ip, src)
    torch.cuda.synchronize()
    print(json.dumps({"probe": "done", "copy_bytes": 1 << 30, "identity_rows": n, "C2": [w2.N, w2.E, w2.K],
                      "C5": [w5.N, w5.E, w5.K]}))


def probe_scatter():
    """Launch sequence for `rocprofv3 --pmc TCC_HIT_sum TCC_MISS_sum TCC_ATOMIC_sum -- python3 bench.py
    --probe-scatter`: C1 scatter sum x3, C4 scatter max with K = 1 and K = 32 x2 each (K = 32 also as a sum and
    through an index sorted once, x2 each), scatter sum and max over the sorted index of C3 with K = 64 x2 each."""
    import torch
    import pytorch_scatter_amd as ts
    from pytorch_scatter_amd import workloads as wl
    dev = torch.device("cuda:0")
    done = {}
    with torch.no_grad():
        w1 = wl.c1_scatter_sum()
        src, index = wl.scatter_values(w1, dev), w1.index.to(dev)
        for _ in range(3):
            ts.scatter_sum(src, index, 0, None, w1.N)
        done["C1"] = [w1.N, w1.E, w1.K]
        for K in (1, 32):
            w4 = wl.c4_scatter_minmax(K)
            src, index = wl.scatter_values(w4, dev), w4.index.to(dev)
            for _ in range(2):
                ts.scatter_max(src, index, 0, None, w4.N)
            done[f"C4-K{K}"] = [w4.N, w4.E, w4.K]
            if K == 32:  # the same scatter as a sum, and through an index sorted once
                for _ in range(2):
                    ts.scatter_sum(src, index, 0, None, w4.N)
                plan = ts.SortedIndex(index, w4.N)
                for _ in range(2):
                    ts.scatter_sorted(src, plan, 0, "max")
        w3 = wl.c3_segment_coo()
        index = w3.index.to(dev)
        src = torch.randn((w3.E, 64), device=dev)
        for _ in range(2):
            ts.scatter_sum(src, index, 0, None, w3.N)
        for _ in range(2):
            ts.scatter_max(src, index, 0, None, w3.N)
        done["X-sorted-K64"] = [w3.N, w3.E, 64]
    torch.cuda.synchronize()
    print(json.dumps({"probe": "scatter done", **done}))


def main():
    args = parse_args()
    if args.probe_ceilings:
        return probe_ceilings()
    if args.probe_atomics:
        return probe_atomics()
    if args.sweep_thresholds:
        return sweep_thresholds()
    if args.sweep_orders:
        return sweep_orders()
    if args.probe:
        return probe()
    if args.probe_scatter:
        return probe_scatter()
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

    # ---------------- headline: C2 through the registered operators
    w2 = wl.c2_segment_csr()
    src = wl.edge_values(w2, dev)
    indptr = w2.indptr.to(dev)
    out = torch.empty((w2.N, w2.K), dtype=torch.float32, device=dev)
    back = torch.empty_like(src)
    step_bytes = 2 * wl.bytes_segment(w2.E, w2.N, w2.K, 4) + wl.bytes_gather(w2.E, w2.N, w2.K, 4)

    def step():
        ts.segment_csr(src, indptr, out, "sum")
        ts.segment_csr(src, indptr, out, "mean")
        ts.gather_csr(out, indptr, back)

    with torch.no_grad():
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
        # dominant kernel: the CSR reduction (segment_csr sum), HIP events on the launch stream
        t_kernel = event_time(lambda: ts.segment_csr(src, indptr, out, "sum"), max(args.steps, 20))
    kernel_bytes = wl.bytes_segment(w2.E, w2.N, w2.K, 4)
    # HBM bytes per launch of this kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, calibrated against
    # copies of known size: read from the tracked profile, null if that file does not state it
    traffic = measured_traffic()
    roofline = {"bound": "hbm", "kernel": "ts::csr_reduce_kernel<float, 4, SUM>",
                "achieved": round(gbs(kernel_bytes, t_kernel), 1), "peak": PEAK_GBS, "unit": "GB/s",
                "frac": round(gbs(kernel_bytes, t_kernel) / PEAK_GBS, 4), "traffic": traffic,
                "algorithmic_bytes_per_launch": kernel_bytes, "us_per_launch": round(t_kernel * 1e6, 2)}
    del src, back, out
    torch.cuda.empty_cache()

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

    cpu = None if args.no_cpu else cpu_baseline(wl, w2)
    cpu_other = None if args.no_cpu else cpu_baselines_other(wl)

    line = {
        "metric": "effective HBM GB/s, segment_csr sum + mean + gather_csr (BASELINE config C2), 1 MI355X",
        "value": round(gbs(step_bytes, dt), 1),
        "unit": "GB/s",
        "pct_of_8TBps_peak": round(100 * gbs(step_bytes, dt) / PEAK_GBS, 1),
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "C2: segment_csr sum+mean, gather_csr; 100000 segments, degrees "
                               "clip(Zipf(2.0),1,512), src fp32 [E,64], numpy default_rng(0)",
                   "N": w2.N, "E": w2.E, "K": w2.K, "algorithmic_bytes_per_step": step_bytes,
                   "api": "torch.ops.torch_scatter.* (eager, out= preallocated)"},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "cpu_baselines_other_configs": cpu_other,
        "configs": table,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
