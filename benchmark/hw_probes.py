#!/usr/bin/env python3
"""Hardware probes and dispatcher sweeps on one MI355X (benchmark tooling, not part of the operator library).

    python3 -m benchmark.hw_probes --ceilings          plain read / write / copy / mixed streams (libts_probe.so)
    python3 -m benchmark.hw_probes --ceiling-matrix    mixed streams 26:1 and 1:26 over store kind x write burst x
                                                       workgroups per CU x loads in flight x specialised workgroups
    python3 -m benchmark.hw_probes --atomics           rate of device-scope 64-bit atomics
    python3 -m benchmark.hw_probes --counters          launch sequence for rocprofv3 --pmc (segment / gather kernels)
    python3 -m benchmark.hw_probes --counters-scatter  launch sequence for rocprofv3 --pmc (scatter kernels)
    python3 -m benchmark.hw_probes --sweep-thresholds  scatter sum / max either side of every dispatcher threshold
    python3 -m benchmark.hw_probes --sweep-orders      one shape under a sorted / shuffled / skewed index

The streaming and atomic kernels live in benchmark/probe/probe.hip (make -C benchmark/probe).
"""
import argparse
import ctypes
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_GBS = 8000.0  # MI355X HBM3E
PROBE_LIB = os.path.join(ROOT, "benchmark", "probe", "libts_probe.so")


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


def probe_lib():
    if not os.path.exists(PROBE_LIB):
        raise SystemExit("benchmark/probe/libts_probe.so is missing: run `make -C benchmark/probe`")
    return ctypes.CDLL(PROBE_LIB)


def probe_ceilings():
    """Plain streams through libts_probe.so (benchmark/probe/probe.hip): read, write, copy and reads mixed
    with writes 3:1 and 26:1, over GiB-sized buffers, HIP events around 10 launches each."""
    import torch
    lib = probe_lib()
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


def ceiling_matrix():
    """The mixed streams a segment reduction (26 bytes read per byte written) and an expansion (26 written per byte
    read) put on the memory system, over: store kind (plain / non-temporal) x contiguous burst per workgroup on the
    light side (256 B ... 64 KB) x workgroups per CU (2 / 4 / 8 of 256 lanes) x 16-byte loads in flight per lane
    (4 / 8 / 16) x workgroups that both read and write against read-only and write-only workgroups side by side.
    ~6.4 GB moved per launch, 1 warm-up + 3 timed launches per cell; the best cells per mix are printed last."""
    import torch
    lib = probe_lib()
    lib.ts_probe_matrix.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t] + \
        [ctypes.c_int] * 8 + [ctypes.c_void_p]
    dev = torch.device("cuda:0")
    heavy = 6 << 30
    ratio = 26
    a = torch.empty(heavy, dtype=torch.uint8, device=dev)
    b = torch.empty(heavy, dtype=torch.uint8, device=dev)
    a.fill_(1)
    b.fill_(2)
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for heavy_read in (1, 0):
        for burst in (256, 1024, 4096, 16384, 65536):
            units = heavy // (ratio * burst)
            moved = units * burst * (ratio + 1)
            for nt_store in (0, 1):
                for wg_per_cu in (2, 4, 8):
                    for depth in (4, 8, 16):
                        for split in (0, 1):
                            for nt_load in ((1,) if not (burst == 4096 and depth == 8) else (1, 0)):
                                grid = 256 * wg_per_cu
                                fn = lambda: lib.ts_probe_matrix(a.data_ptr(), b.data_ptr(), units, burst, ratio, heavy_read,
                                                                 depth, nt_load, nt_store, split, grid, 0, stream)
                                assert fn() == 0
                                t = event_time(fn, 3, warm=1)
                                rows.append({"mix": "read 26 : write 1" if heavy_read else "read 1 : write 26",
                                             "burst_B": burst, "store": "nt" if nt_store else "plain",
                                             "load": "nt" if nt_load else "plain", "wg_per_cu": wg_per_cu,
                                             "loads_in_flight": depth, "specialised_wgs": bool(split),
                                             "us": round(t * 1e6, 1), "GBps": round(moved / t / 1e9, 1),
                                             "pct_of_peak": round(100 * moved / t / 1e9 / PEAK_GBS, 1)})
    for r in rows:
        print(f"{r['mix']:18s} burst {r['burst_B']:6d} B  store {r['store']:5s} load {r['load']:5s} "
              f"{r['wg_per_cu']} wg/CU  {r['loads_in_flight']:2d} in flight  "
              f"{'specialised' if r['specialised_wgs'] else 'mixed      '}  {r['us']:8.1f} us  {r['GBps']:7.1f} GB/s  "
              f"{r['pct_of_peak']:5.1f} %", file=sys.stderr)
    best = {}
    for mix in ("read 26 : write 1", "read 1 : write 26"):
        cells = sorted((r for r in rows if r["mix"] == mix), key=lambda r: -r["GBps"])
        best[mix] = cells[:5]
        print(f"best cells, {mix}:", file=sys.stderr)
        for r in cells[:5]:
            print("   ", r, file=sys.stderr)
    print(json.dumps({"probe": "ceiling matrix", "cells": len(rows), "best": best, "rows": rows}))


def probe_atomics():
    """Rate of device-scope 64-bit atomics (libts_probe.so): scattered addresses (one transaction per lane) and
    neighbouring addresses shared by all workgroups (a table written back by every workgroup at once)."""
    import torch
    lib = probe_lib()
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
        ("sum: single values in buckets from 2^21 entries (K = 1; sample of the index)", "sum", 1, 1_000_000,
         [2 * M - 65536, 2 * M + 65536]),
        ("sum: single values, tables in slabs from 2^19 entries (K = 1)", "sum", 1, 100_000,
         [M // 2 - 16384, M // 2 + 16384]),
        ("sum: rows of two values in buckets from 2^21 entries (K = 2; sample of the index)", "sum", 2, 1_000_000,
         [2 * M - 65536, 2 * M + 65536]),
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


def counters():
    """Launch sequence for the memory-side request counters, one rocprofv3 run per counter group:
        rocprofv3 --pmc TCC_EA0_RDREQ_sum TCC_EA0_RDREQ_32B_sum TCC_EA0_RDREQ_64B_sum TCC_EA0_RDREQ_128B_sum -- \
            python3 -m benchmark.hw_probes --counters
        rocprofv3 --pmc TCC_EA0_WRREQ_sum TCC_EA0_WRREQ_64B_sum -- python3 -m benchmark.hw_probes --counters
    1. torch copy of 1 GiB (plain loads / stores, known size: checks how the counters read);
    2. segment_csr sum with one entry per segment over 1 GiB of fp32 [4Mi, 64]: a copy through the
       reduction kernel itself (same non-temporal loads), known size;
    3. C2 segment_csr sum x3, C3 segment_coo max x2, C5 segment_csr mean x2, C5 gather_csr x2, C5 fused mean
       backward x2."""
    import torch
    import pytorch_scatter_amd as ts
    from pytorch_scatter_amd import capi
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
        w3 = wl.c3_segment_coo()
        src = wl.edge_values(w3, dev, uniform=True)
        idx = w3.index.to(dev)
        for _ in range(2):
            ts.segment_max_coo(src, idx, None, w3.N)
        del src, idx
        w5 = wl.c5_gnn()
        src = wl.edge_values(w5, dev)
        out = torch.empty((w5.N, w5.K), dtype=torch.bfloat16, device=dev)
        ip = w5.indptr.to(dev)
        for _ in range(2):
            ts.segment_csr(src, ip, out, "mean")
        for _ in range(2):
            ts.gather_csr(out, ip, src)
        for _ in range(2):
            capi.segment_mean_csr_backward(out, ip, src, 1, w5.N, w5.E, w5.K, 0)
    torch.cuda.synchronize()
    print(json.dumps({"probe": "done", "copy_bytes": 1 << 30, "identity_rows": n, "C2": [w2.N, w2.E, w2.K],
                      "C3": [w3.N, w3.E, w3.K], "C5": [w5.N, w5.E, w5.K]}))


def counters_scatter():
    """Launch sequence for `rocprofv3 --pmc TCC_HIT_sum TCC_MISS_sum TCC_ATOMIC_sum -- python3 -m benchmark.hw_probes
    --counters-scatter`: C1 scatter sum x3, C4 scatter max with K = 1 and K = 32 x2 each (K = 32 also as a sum and
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


def lane_moves():
    """The kernels whose fixed-pattern cross-lane steps run in the vector ALU (csrc/dpp.h): HIP-event times of ten
    calls each on stderr, and, under `rocprofv3 --pmc SQ_INSTS_VALU SQ_INSTS_SALU SQ_INSTS_LDS SQ_WAVE_CYCLES
    SQ_BUSY_CYCLES -- python3 -m benchmark.hw_probes --lane-moves`, their instruction counts per dispatch. Run
    against a library built with -DTS_DPP_OFF (make -B EXTRA=-DTS_DPP_OFF, then make torch) it gives the same
    kernels with every such step as a shuffle through LDS."""
    import torch
    import pytorch_scatter_amd as ts
    from pytorch_scatter_amd import workloads as wl
    dev = torch.device("cuda:0")
    w3 = wl.c3_segment_coo()
    index, indptr = w3.index.to(dev), w3.indptr.to(dev)
    src8, g8 = torch.randn((w3.E, 8), device=dev), torch.randn((w3.E, 8), device=dev)
    src1, out1 = torch.randn((w3.E, 1), device=dev), torch.empty((w3.N, 1), device=dev)
    src64 = torch.randn((w3.E, 64), device=dev)
    x = src8.clone().requires_grad_(True)
    y = ts.scatter_softmax(x, index, 0, w3.N)
    cases = {
        "scatter_softmax forward, sorted index, K=8": lambda: ts.scatter_softmax(src8, index, 0, w3.N),
        "scatter_softmax backward, sorted index, K=8": lambda: torch.autograd.grad(y, x, g8, retain_graph=True),
        "segment_csr sum, K=1": lambda: ts.segment_csr(src1, indptr, out1, "sum"),
        "segment_csr max, K=1": lambda: ts.segment_max_csr(src1, indptr),
        "gather_csr, K=1": lambda: ts.gather_csr(out1, indptr, src1),
        "scatter sum, sorted index, K=64": lambda: ts.scatter_sum(src64, index, 0, None, w3.N),
        "scatter sum, sorted index, K=8": lambda: ts.scatter_sum(src8, index, 0, None, w3.N),
    }
    w4 = wl.c4_scatter_minmax(32)
    s4, i4 = wl.scatter_values(w4, dev), w4.index.to(dev)
    cases["C4 scatter max, K=32"] = lambda: ts.scatter_max(s4, i4, 0, None, w4.N)
    rows = []
    for name, fn in cases.items():
        if "backward" in name:
            t = event_time(fn, 10)
        else:
            with torch.no_grad():
                t = event_time(fn, 10)
        rows.append({"case": name, "us": round(t * 1e6, 1)})
        print(f"{name:48s} {t * 1e6:9.1f} us", file=sys.stderr)
    print(json.dumps({"probe": "lane moves", "rows": rows}))


def value_buckets():
    """Sums and means of one float per entry under an index in random order, at the sizes of the two large row
    structures of the benchmark tables: this library against torch's scatter_add_ (HIP-event times on stderr); under
    `rocprofv3 --kernel-trace --stats` the passes of the value buckets (count, scan, place, add) one by one."""
    import torch
    import pytorch_scatter_amd as ts
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    rows = []
    with torch.no_grad():
        for name, N, E in (("StocF-1465-like", 1_465_137, 21_005_389), ("ldoor-like", 952_203, 46_522_475)):
            index = torch.randint(0, N, (E,), generator=g).to(dev)
            src = torch.randn((E, 1), device=dev)
            out = torch.zeros((N, 1), device=dev)
            idx2 = index.view(-1, 1)
            t_sum = event_time(lambda: ts.scatter_sum(src, index, 0, None, N), 10)
            t_mean = event_time(lambda: ts.scatter_mean(src, index, 0, None, N), 10)
            t_torch = event_time(lambda: out.zero_().scatter_add_(0, idx2, src), 10)
            want = torch.zeros((N, 1), dtype=torch.float64, device=dev).index_add_(0, index, src.double())
            got = ts.scatter_sum(src, index, 0, None, N)
            ok = bool(torch.allclose(got.double(), want, rtol=1e-5, atol=1e-4))
            rows.append({"structure": name, "N": N, "E": E, "sum_us": round(t_sum * 1e6, 1), "mean_us": round(t_mean * 1e6, 1),
                         "torch_scatter_add_us": round(t_torch * 1e6, 1), "sum_matches_fp64": ok})
            print(f"{name:18s} N {N:8d} E {E:9d}  sum {t_sum * 1e6:8.1f} us  mean {t_mean * 1e6:8.1f} us  "
                  f"torch scatter_add_ {t_torch * 1e6:8.1f} us  sum matches fp64 index_add_: {ok}", file=sys.stderr)
            del index, src, out, idx2, want, got
    print(json.dumps({"probe": "value buckets", "rows": rows}))


def main():
    ap = argparse.ArgumentParser()
    for flag in ("--ceilings", "--ceiling-matrix", "--atomics", "--counters", "--counters-scatter",
                 "--sweep-thresholds", "--sweep-orders", "--lane-moves", "--value-buckets"):
        ap.add_argument(flag, action="store_true")
    args = ap.parse_args()
    if args.ceilings:
        return probe_ceilings()
    if args.ceiling_matrix:
        return ceiling_matrix()
    if args.atomics:
        return probe_atomics()
    if args.counters:
        return counters()
    if args.counters_scatter:
        return counters_scatter()
    if args.sweep_thresholds:
        return sweep_thresholds()
    if args.sweep_orders:
        return sweep_orders()
    if args.lane_moves:
        return lane_moves()
    if args.value_buckets:
        return value_buckets()
    ap.print_help()


if __name__ == "__main__":
    main()
