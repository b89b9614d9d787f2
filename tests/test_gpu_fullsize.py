"""Parity at the full sizes of the measurement configurations (C1..C5), where
the CPU oracle would take minutes: size-independent properties and
cross-checks between independent algorithms.

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
