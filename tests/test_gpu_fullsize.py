"""Parity at the full sizes of the measurement configurations (C1..C5).

C1, C2 (both readings), C3, C4 (one and 32 values per entry) are compared with
the CPU oracle on the same inputs at full size (seconds on one host core):
min / max values and every arg bit for bit, sums and means within rtol 1e-5 of
the result plus 1e-5 of the largest sum of magnitudes of a row. C5 (48 GB
live) is compared with the oracle on a 1/8 slice with random bf16 features
(mean, fused backward, gather) and, at full size, as a sum of random edges
against fp64 index_add_ on the device. Next to that, size-independent
properties and cross-checks between independent algorithms:

* gather then reduce: max over copies of a row is that row, first position wins;
* packed-key atomic scatter (unsorted, contended, with exact ties) against the
  merge-path CSR reduction of the same data after a stable sort -- two
  unrelated kernels that must agree bit for bit, args mapped back through the
  permutation;
* arg invariants (src[arg] == out, empty rows -> 0 / E), checksums of sums,
  torch library routines (index_add_, repeat_interleave, index_select) where
  they are affordable.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture(scope="module")
def env():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import pytorch_scatter_amd as ts
    from pytorch_scatter_amd import workloads as wl
    return ts, wl


def test_c1_scatter_sum(env):
    ts, wl = env
    w = wl.c1_scatter_sum()
    src = wl.scatter_values(w, DEV)
    index = w.index.to(DEV)
    got = ts.scatter_sum(src, index, 0, None, w.N)
    want = torch.zeros(w.N, w.K, device=DEV, dtype=torch.float64).index_add_(0, index, src.double())
    scale = torch.zeros(w.N, w.K, device=DEV, dtype=torch.float64).index_add_(0, index, src.double().abs()).max()
    assert bool(((got.double() - want).abs() <= 1e-5 * want.abs() + 1e-5 * scale).all())
    mean = ts.scatter_mean(src, index, 0, None, w.N)
    cnt = torch.bincount(index, minlength=w.N).clamp(min=1).unsqueeze(1)
    assert bool(((mean.double() - want / cnt).abs() <= 1e-5 * (want / cnt).abs() + 1e-5 * scale).all())


@pytest.mark.parametrize("mean16", [False, True])
def test_c2_segment_csr_and_gather(env, mean16):
    ts, wl = env
    w = wl.c2_segment_csr(mean16=mean16)
    src = wl.edge_values(w, DEV)
    indptr, index = w.indptr.to(DEV), w.index.to(DEV)
    deg = (indptr[1:] - indptr[:-1])
    want = torch.zeros(w.N, w.K, device=DEV, dtype=torch.float64).index_add_(0, index, src.double())
    scale = torch.zeros(w.N, w.K, device=DEV, dtype=torch.float64).index_add_(0, index, src.double().abs()).max()
    got = ts.segment_csr(src, indptr, None, "sum")
    assert bool(((got.double() - want).abs() <= 1e-5 * want.abs() + 1e-5 * scale).all())
    # bit-reproducible: a second run gives the same bits
    assert torch.equal(got, ts.segment_csr(src, indptr, None, "sum"))
    mean = ts.segment_csr(src, indptr, None, "mean")
    assert torch.equal(mean, got / deg.clamp(min=1).unsqueeze(1).float())   # mean = T(sum) / T(count)
    back = ts.gather_csr(got, indptr)
    assert torch.equal(back, torch.repeat_interleave(got, deg, dim=0))
    assert torch.equal(back, ts.gather_coo(got, index))
    # same reduction through the sorted-index entry point
    assert torch.equal(got, ts.segment_coo(src, index, None, w.N, "sum"))


def test_c3_segment_coo_max_against_scatter_max(env):
    ts, wl = env
    w = wl.c3_segment_coo()
    src = wl.edge_values(w, DEV, uniform=True)
    # exact ties inside segments: copy every 16th row onto its successor
    src[1::16] = src[0:-1:16][: src[1::16].shape[0]]
    index = w.index.to(DEV)
    out, arg = ts.segment_max_coo(src, index, None, w.N)
    deg = (w.indptr[1:] - w.indptr[:-1]).to(DEV)
    empty = deg == 0
    assert int(empty.sum()) > 0
    assert bool((out[empty] == 0).all()) and bool((arg[empty] == w.E).all())
    # arg invariants on the non-empty rows
    full = ~empty
    a = arg[full]
    assert bool((a < w.E).all())
    assert torch.equal(torch.gather(src, 0, a), out[full])
    assert torch.equal(index[a[:, 0]], torch.nonzero(full).squeeze(1))
    # the packed-key atomic scatter is a different algorithm: same values, same args (first index on ties)
    out2, arg2 = ts.scatter_max(src, index, 0, None, w.N)
    assert torch.equal(out, out2)
    assert torch.equal(arg, arg2)
    del out2, arg2
    # and the CSR entry point
    out3, arg3 = ts.segment_max_csr(src, w.indptr.to(DEV))
    assert torch.equal(out, out3) and torch.equal(arg, arg3)


@pytest.mark.parametrize("K", [1, 4, 8, 16])
def test_c3_graph_narrow_rows(env, K):
    """The 9 M-entry graph of C3 with 1 to 16 values per entry: the LDS-staged reduction, the
    one-lane-per-16-bytes expansion and the run-combining scatter against each other and torch."""
    ts, wl = env
    w = wl.c3_segment_coo()
    g = torch.Generator(device=DEV).manual_seed(K)
    src = torch.randint(-8, 9, (w.E, K), generator=g, device=DEV).float()   # many exact ties, exact sums
    indptr, index = w.indptr.to(DEV), w.index.to(DEV)
    deg = indptr[1:] - indptr[:-1]
    want = torch.zeros(w.N, K, device=DEV).index_add_(0, index, src)
    got = ts.segment_csr(src, indptr, None, "sum")
    assert torch.equal(got, want)                                          # small integers: exact in fp32
    assert torch.equal(ts.segment_coo(src, index, None, w.N, "sum"), want)
    assert torch.equal(ts.scatter_sum(src, index, 0, None, w.N), want)     # sorted index: runs combined in the wavefront
    out, arg = ts.segment_max_csr(src, indptr)
    out2, arg2 = ts.scatter_max(src, index, 0, None, w.N)
    assert torch.equal(out, out2) and torch.equal(arg, arg2)
    full = deg > 0
    a = arg[full]
    assert bool((a < w.E).all()) and torch.equal(torch.gather(src, 0, a), out[full])
    assert bool((arg[~full] == w.E).all()) and bool((out[~full] == 0).all())
    # first position wins: no earlier entry of the row holds the same value
    first = indptr[:-1][full].unsqueeze(1)
    probe = torch.minimum(a - 1, a).clamp(min=0)
    earlier_same = (torch.gather(src, 0, probe) == out[full]) & (a - 1 >= first)
    assert not bool(earlier_same.any())
    back = ts.gather_csr(got, indptr)
    assert torch.equal(back, torch.repeat_interleave(got, deg, dim=0))
    assert torch.equal(back, ts.gather_coo(got, index))


@pytest.mark.parametrize("K", [1, 32])
@pytest.mark.parametrize("reduce", ["max", "min"])
def test_c4_contended_scatter_against_sorted_reduction(env, K, reduce):
    ts, wl = env
    w = wl.c4_scatter_minmax(K)
    src = wl.scatter_values(w, DEV)
    index = w.index.to(DEV)
    # the workload really has exact ties inside nodes
    assert bool((src[w.tie_dst.to(DEV)[:1000]] == src[w.tie_src.to(DEV)[:1000]]).float().mean() > 0.8)
    fn = ts.scatter_max if reduce == "max" else ts.scatter_min
    out, arg = fn(src, index, 0, None, w.N)
    # independent path: stable sort by node, merge-path CSR reduction, map args back
    sorted_index, perm = torch.sort(index, stable=True)
    counts = torch.bincount(index, minlength=w.N)
    indptr = torch.zeros(w.N + 1, dtype=torch.long, device=DEV)
    indptr[1:] = torch.cumsum(counts, 0)
    seg = ts.segment_max_csr if reduce == "max" else ts.segment_min_csr
    want, warg = seg(src[perm], indptr)
    warg = torch.where(warg < w.E, perm[warg.clamp(max=w.E - 1)], warg)
    assert torch.equal(out, want)
    assert torch.equal(arg, warg)
    # empty nodes
    empty = counts == 0
    assert bool((out[empty] == 0).all()) and bool((arg[empty] == w.E).all())


def test_c5_gather_reduce_round_trips(env):
    ts, wl = env
    w = wl.c5_gnn()
    assert w.E * w.K > 2 ** 31  # 64-bit offsets are exercised
    indptr, index = w.indptr.to(DEV), w.index.to(DEV)
    deg = indptr[1:] - indptr[:-1]
    g = torch.Generator(device=DEV).manual_seed(1)
    x = torch.randn((w.N, w.K), generator=g, device=DEV).to(torch.bfloat16)
    edges = ts.gather_csr(x, indptr)                       # node -> edge
    assert edges.shape == (w.E, w.K)
    sample = torch.randint(0, w.E, (2_000_000,), generator=g, device=DEV)
    assert torch.equal(edges[sample], x[index[sample]])
    hub = int(torch.argmax(deg))
    lo, hi = int(indptr[hub]), int(indptr[hub + 1])
    assert bool((edges[lo:hi] == x[hub]).all())
    assert torch.equal(edges[:4096], ts.gather_coo(x, index[:4096].contiguous()))
    # max over identical copies returns the row, arg = first edge of the row
    out, arg = ts.segment_max_csr(edges, indptr)
    assert torch.equal(out, x)
    assert torch.equal(arg, indptr[:-1].unsqueeze(1).expand(w.N, w.K))
    # mean over identical copies: fp32 sum of deg copies is exact, then two bf16 roundings
    mean = ts.segment_csr(edges, indptr, None, "mean")
    want = ((x.float() * deg.unsqueeze(1)).to(torch.bfloat16).float()
            / deg.to(torch.bfloat16).float().unsqueeze(1)).to(torch.bfloat16)
    assert torch.equal(mean, want)
    # mean backward: grad_in[e] = g[row(e)] / bf16(deg(row(e)))
    edges.requires_grad_()
    ts.segment_csr(edges, indptr, None, "mean").backward(x)
    wantg = (x.float() / deg.to(torch.bfloat16).float().unsqueeze(1)).to(torch.bfloat16)
    assert torch.equal(edges.grad[sample], wantg[index[sample]])
    assert torch.equal(edges.grad[lo:hi], wantg[hub].expand(hi - lo, w.K))


# ---- against the CPU oracle at full size ----------------------------------------------------------------------
def _close(got, want, scale, rtol):
    err = (got.double().cpu() - want.double()).abs()
    return bool((err <= rtol * want.double().abs() + rtol * scale).all()), float(err.max())


def _row_scale(oracle, src, index, N):
    """Largest sum of magnitudes of an output row (sums of N(0,1) cancel towards 0: the absolute part of the bound)."""
    a, _ = oracle.scatter(src.abs(), index.view(-1, 1).expand_as(src), 0, None, N, "sum")
    return float(a.max())


def test_c1_against_oracle(env, oracle):
    ts, wl = env
    w = wl.c1_scatter_sum()
    src = wl.scatter_values(w, DEV)
    src_cpu = src.cpu()
    idx = w.index.view(-1, 1).expand_as(src_cpu)
    scale = _row_scale(oracle, src_cpu, w.index, w.N)
    want, _ = oracle.scatter(src_cpu, idx, 0, None, w.N, "sum")
    ok, err = _close(ts.scatter_sum(src, w.index.to(DEV), 0, None, w.N), want, scale, 1e-5)   # fp32: rtol 1e-5
    assert ok, err
    want = oracle.op_scatter(src_cpu, w.index, 0, None, w.N, "mean")
    ok, err = _close(ts.scatter_mean(src, w.index.to(DEV), 0, None, w.N), want, scale, 1e-5)
    assert ok, err
    for reduce in ("min", "max"):
        want, warg = oracle.scatter(src_cpu, idx, 0, None, w.N, reduce)
        got, arg = getattr(ts, "scatter_" + reduce)(src, w.index.to(DEV), 0, None, w.N)
        assert torch.equal(got.cpu(), want) and torch.equal(arg.cpu(), warg)


@pytest.mark.parametrize("mean16", [False, True])
def test_c2_against_oracle(env, oracle, mean16):
    ts, wl = env
    w = wl.c2_segment_csr(mean16=mean16)
    src = wl.edge_values(w, DEV)
    src_cpu = src.cpu()
    indptr = w.indptr.to(DEV)
    scale = float(oracle.segment_csr(src_cpu.abs(), w.indptr, None, "sum")[0].max())
    for reduce in ("sum", "mean"):
        want, _ = oracle.segment_csr(src_cpu, w.indptr, None, reduce)
        ok, err = _close(ts.segment_csr(src, indptr, None, reduce), want, scale, 1e-5)         # fp32: rtol 1e-5
        assert ok, (reduce, err)
    for reduce in ("min", "max"):
        want, warg = oracle.segment_csr(src_cpu, w.indptr, None, reduce)
        got, arg = getattr(ts, f"segment_{reduce}_csr")(src, indptr)
        assert torch.equal(got.cpu(), want) and torch.equal(arg.cpu(), warg), reduce
    want, _ = oracle.segment_csr(src_cpu, w.indptr, None, "sum")
    assert torch.equal(ts.gather_csr(want.to(DEV), indptr).cpu(), oracle.gather_csr(want, w.indptr))
    assert torch.equal(ts.gather_coo(want.to(DEV), w.index.to(DEV)).cpu(), oracle.gather_coo(want, w.index))


def test_c3_against_oracle(env, oracle):
    ts, wl = env
    w = wl.c3_segment_coo()
    src = wl.edge_values(w, DEV, uniform=True)
    src[1::16] = src[0:-1:16][: src[1::16].shape[0]]   # exact ties inside segments
    src_cpu = src.cpu()
    want, warg = oracle.segment_coo(src_cpu, w.index, None, w.N, "max")
    got, arg = ts.segment_max_coo(src, w.index.to(DEV), None, w.N)
    assert torch.equal(got.cpu(), want)
    assert torch.equal(arg.cpu(), warg)


@pytest.mark.parametrize("K", [1, 32])
@pytest.mark.parametrize("reduce", ["max", "min"])
def test_c4_against_oracle(env, oracle, K, reduce):
    ts, wl = env
    w = wl.c4_scatter_minmax(K)
    src = wl.scatter_values(w, DEV)
    src_cpu = src.cpu()
    want, warg = oracle.scatter(src_cpu, w.index.view(-1, 1).expand_as(src_cpu), 0, None, w.N, reduce)
    got, arg = getattr(ts, "scatter_" + reduce)(src, w.index.to(DEV), 0, None, w.N)
    assert torch.equal(got.cpu(), want)
    assert torch.equal(arg.cpu(), warg)


def test_c5_slice_against_oracle(env, oracle):
    """1/8 of C5 (the same generator with the node count scaled: same degree law, same cap rule), random bf16
    features: mean within rtol 1e-2 of the result plus 1e-2 of the row's sum of magnitudes over its length
    (bf16: the fp32 partial sums here and the oracle's sequential fp32 sum round to neighbouring bf16 values),
    fused backward and gather bit for bit."""
    ts, wl = env
    w = wl.c5_gnn(scale=1.0 / 8)
    src = wl.edge_values(w, DEV)
    src_cpu = src.cpu()
    indptr = w.indptr.to(DEV)
    want, _ = oracle.segment_csr(src_cpu, w.indptr, None, "mean")
    got = ts.segment_csr(src, indptr, None, "mean").cpu()
    deg = (w.indptr[1:] - w.indptr[:-1]).clamp(min=1).unsqueeze(1).double()
    mags = oracle.segment_csr(src_cpu.float().abs(), w.indptr, None, "sum")[0].double() / deg
    err = (got.double() - want.double()).abs()
    assert bool((err <= 1e-2 * want.double().abs() + 1e-2 * mags).all()), float(err.max())
    exact = torch.equal(got, want)   # informational: most rows agree bit for bit
    g = torch.Generator(device=DEV).manual_seed(2)
    grad = torch.randn((w.N, w.K), generator=g, device=DEV).to(torch.bfloat16)
    x = src.clone().requires_grad_()
    ts.segment_csr(x, indptr, None, "mean").backward(grad)
    assert torch.equal(x.grad.cpu(), oracle.segment_mean_csr_backward(grad.cpu(), w.indptr, (w.E, w.K)))
    assert torch.equal(ts.gather_csr(grad, indptr).cpu(), oracle.gather_csr(grad.cpu(), w.indptr))
    del exact


def test_c5_full_size_sum_of_random_edges(env):
    """segment_csr sum of random bf16 edges at the full size of C5 (the 50 876-edge hub row passes through 27 tiles
    of carries) against a chunked fp64 index_add_ on the device: within one bf16 rounding of the exact sum
    (2^-8 relative) plus the fp32 accumulation error (1e-5 of the row's sum of magnitudes)."""
    ts, wl = env
    w = wl.c5_gnn()
    src = wl.edge_values(w, DEV)
    indptr, index = w.indptr.to(DEV), w.index.to(DEV)
    got = ts.segment_csr(src, indptr, None, "sum")
    want = torch.zeros((w.N, w.K), dtype=torch.float64, device=DEV)
    mags = torch.zeros((w.N, w.K), dtype=torch.float64, device=DEV)
    step = 1 << 22
    for s0 in range(0, w.E, step):
        chunk = src[s0:s0 + step].double()
        want.index_add_(0, index[s0:s0 + step], chunk)
        mags.index_add_(0, index[s0:s0 + step], chunk.abs())
        del chunk
    err = (got.double() - want).abs()
    bound = 2.0 ** -8 * want.abs() + 1e-5 * mags
    bad = err > bound
    assert not bool(bad.any()), (int(bad.sum()), float(err.max()))
    hub = int(torch.argmax(indptr[1:] - indptr[:-1]))
    assert int(indptr[hub + 1] - indptr[hub]) > 40_000 and not bool(bad[hub].any())
    # the mean of the same edges: T(sum) / T(count), bit for bit from the sum above
    mean = ts.segment_csr(src, indptr, None, "mean")
    cnt = (indptr[1:] - indptr[:-1]).clamp(min=1).to(torch.bfloat16).float().unsqueeze(1)
    assert torch.equal(mean, (got.float() / cnt).to(torch.bfloat16))
