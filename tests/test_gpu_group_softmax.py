"""The fused softmax / log-softmax / logsumexp / std over groups (ts_group_softmax,
ts_group_logsumexp, ts_group_std and their backward calls through the C ABI,
torch.ops.torch_scatter.scatter_softmax / scatter_logsumexp / scatter_std through
the Python API) against the CPU oracle on the same seeded inputs.

Bars. fp32 / fp64 compare with the oracle's result in the same type:
rtol 1e-5 / 1e-12 (the two differ in the exp of the math library and in the
order of the group sum). 16-bit floats compare with the oracle evaluated in
fp64 on the same 16-bit inputs, within the roundings the reference's own
sequence commits in the element type: the shifted value z = src - max is
rounded to the element type before exp, so the bound grows with |z|."""
from itertools import product

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
EPS_T = {torch.float32: 1e-5, torch.float64: 1e-12, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}
DTYPES = [torch.float32, torch.float64, torch.bfloat16, torch.float16]
SHAPES = [
    # B, E, K, N
    (1, 5000, 1, 300), (2, 3000, 4, 50), (1, 2000, 8, 100), (1, 1500, 3, 40), (1, 900, 64, 20),
    (1, 700, 130, 9), (3, 400, 16, 7), (1, 1, 1, 1), (1, 257, 2, 300),
    # 2^16 terms and more, rows of up to 128 columns: the group sums go through the accumulator table
    (1, 70_000, 1, 3000), (2, 6000, 8, 500), (1, 1200, 64, 90), (1, 600, 128, 40),
]


@pytest.fixture(scope="module")
def capi():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from pytorch_scatter_amd import capi
    capi.lib()
    return capi


@pytest.fixture(scope="module")
def ts():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import pytorch_scatter_amd
    return pytorch_scatter_amd


def make_index(kind, rng, E, N):
    idx = rng.integers(0, N, size=E)
    if kind == "sorted":
        idx = np.sort(idx)
    elif kind == "hub":
        idx[E // 4: 3 * E // 4] = idx[0]
    return torch.from_numpy(idx)


def bucket_lanes(K, dtype):
    """lanes that hold a row in the bucket kernels: 16 bytes each when the row is a whole number of them, else one column"""
    full = 16 // torch.empty((), dtype=dtype).element_size()
    return K // full if K % full == 0 else K


def forward_bound(dtype, want64, z64, log_space, exact=True):
    e = EPS_T[dtype]
    if dtype in (torch.float32, torch.float64) and exact:
        return e * want64.abs() + e * (1.0 if log_space else 1e-30)
    if log_space:
        return e * (4.0 + want64.abs() + z64.abs())
    # fp16 results below 2^-14 are subnormal: absolute spacing 2^-24, for e and for the quotient
    return e * (4.0 + z64.abs()) * want64.abs() + (2.0 ** -23 if dtype == torch.float16 else 1e-30)


def check_against_oracle(capi, oracle, src, grad, index1, shape, dtype):
    B, E, K, N = shape
    index = index1.view(1, E, 1).expand(B, E, K)
    # fp32 / fp64 against the oracle's sequence in the same type -- for groups of up to a few thousand entries: the
    # fp32 sum of a group of 35 000 terms in entry order is itself 1e-5 away from the exact one, so the large
    # shapes are checked against the oracle in fp64, like the 16-bit types
    exact = dtype in (torch.float32, torch.float64) and E <= 10_000
    ref_src = src if exact else src.double()
    inside = (index >= 0) & (index < N)
    safe = index.clamp(0, N - 1)
    if bool(inside.all()):
        group_max = oracle.scatter(ref_src, index, 1, None, N, "max")[0]
    else:  # entries outside [0, N) belong to no group: keep them out of the reference, expect 0 for them
        low = torch.finfo(ref_src.dtype).min
        group_max = oracle.scatter(torch.where(inside, ref_src, torch.full_like(ref_src, low)), safe, 1, None, N, "max")[0]
    z64 = (ref_src - group_max.gather(1, safe)).double()
    for log_space in (False, True):
        out = torch.empty((B, E, K), dtype=dtype, device=DEV)
        capi.group_softmax(src.to(DEV), index1.to(DEV), out, B, E, K, N, 0, 1, log_space)
        torch.cuda.synchronize()
        if bool(inside.all()):
            want = (oracle.scatter_log_softmax(ref_src, index, 1, 1e-12, N) if log_space
                    else oracle.scatter_softmax(ref_src, index, 1, N)).double()
        else:
            keep = inside[0, :, 0]
            part = (oracle.scatter_log_softmax(ref_src[:, keep], index[:, keep], 1, 1e-12, N) if log_space
                    else oracle.scatter_softmax(ref_src[:, keep], index[:, keep], 1, N)).double()
            want = torch.zeros((B, E, K), dtype=torch.float64)
            want[:, keep] = part
        err = (out.cpu().double() - want).abs()
        bound = forward_bound(dtype, want, z64, log_space, exact)
        assert bool((err <= bound).all()), (log_space, float((err - bound).max()))
        assert float(out.cpu().double()[~inside].abs().max() if bool((~inside).any()) else 0.0) == 0.0

        grad_in = torch.empty((B, E, K), dtype=dtype, device=DEV)
        capi.group_softmax_backward(out, grad.to(DEV), index1.to(DEV), grad_in, B, E, K, N, 0, 1, log_space)
        torch.cuda.synchronize()
        y64, g64 = out.cpu().double(), grad.double()
        keep = inside[0, :, 0]
        want_g = torch.zeros((B, E, K), dtype=torch.float64)
        want_g[:, keep] = oracle.scatter_softmax_backward(y64[:, keep], g64[:, keep], index[:, keep], 1, N, log_space)
        terms = (g64.abs() if log_space else (y64 * g64).abs())
        spread = oracle.scatter(terms * inside, safe, 1, None, N, "sum")[0].gather(1, safe)
        scale = g64.abs() + y64.exp() * spread if log_space else y64.abs() * (g64.abs() + spread)
        e = EPS_T[dtype]
        gerr = (grad_in.cpu().double() - want_g).abs()
        gbound = 8 * e * scale + (2.0 ** -23 if dtype == torch.float16 else 1e-30)  # fp16 subnormals
        assert bool((gerr[:, keep] <= gbound[:, keep]).all()), ("backward", log_space, float((gerr - gbound).max()))
        assert float(grad_in.cpu().double()[~inside].abs().max() if bool((~inside).any()) else 0.0) == 0.0


@pytest.mark.parametrize("shape,kind,dtype", product(SHAPES + [(1, 300_000, 8, 2000)], ["random", "sorted", "hub"], DTYPES))
@pytest.mark.parametrize("route", ["passes", "buckets"])
def test_forward_and_backward_capi(capi, oracle, monkeypatch, shape, kind, dtype, route):
    """route = buckets: the forward call finds key and sum of every group through buckets of groups (group_binned.h)
    at any size, then the elementwise finish; a hub group fills several chunks of its bucket."""
    B, E, K, N = shape
    if route == "buckets":
        if bucket_lanes(K, dtype) > 32:
            pytest.skip("rows held by more than 32 lanes stay with the three passes")
        monkeypatch.setenv("TS_GROUP_BINS", "2")
        assert capi.group_bins_workspace_bytes(B, E, K, N, dtype) > 0
    elif E > 100_000:
        pytest.skip("a shape for the buckets")
    else:
        monkeypatch.setenv("TS_GROUP_BINS", "0")
    rng = np.random.default_rng(E * 13 + K)
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K)) * 3).to(dtype)
    grad = torch.from_numpy(rng.standard_normal(size=(B, E, K))).to(dtype)
    check_against_oracle(capi, oracle, src, grad, make_index(kind, rng, E, N), shape, dtype)


# The one-pass kernels for an index that is in order (group_fused.h) take over from 16 / 32 MB of input; the
# environment switches them on at any size and sets their tile, so that small inputs reach every part of them:
# runs inside a tile, runs that cross one border or fill whole tiles, short / medium / long runs, entries outside
# [0, N) at either end, an index that is not in order (the tiles notice and the three passes redo the work).
FUSED_SHAPES = [
    # B, E, K, N
    (1, 5000, 1, 600), (1, 5000, 1, 3), (2, 3000, 4, 50), (1, 2000, 8, 300), (1, 2000, 8, 2), (1, 1500, 3, 40),
    (1, 900, 32, 20), (3, 400, 16, 7), (1, 257, 2, 300), (1, 4099, 8, 1), (1, 2, 4, 5),
]


def fused_index(kind, rng, E, N):
    if kind == "skewed":  # a few long runs among many short ones
        idx = np.sort(np.concatenate([rng.integers(0, N, size=E - E // 2), np.full(E // 2, N // 2)]))
    elif kind == "outside":  # sorted, with entries below 0 in front and from N on at the end
        idx = np.sort(rng.integers(-max(N // 8, 1), N + max(N // 8, 1), size=E))
    elif kind == "one_descent":
        idx = np.sort(rng.integers(0, N, size=E))
        idx[E // 2:] = np.sort(rng.integers(0, N, size=E - E // 2))
    else:
        idx = np.sort(rng.integers(0, N, size=E))
    return torch.from_numpy(idx)


@pytest.mark.parametrize("shape,kind,dtype",
                         product(FUSED_SHAPES, ["sorted", "skewed", "outside", "one_descent"], DTYPES))
@pytest.mark.parametrize("tile,bins", [(256, "0"), (0, "0"), (256, "2")])
def test_one_pass_kernels_capi(capi, oracle, monkeypatch, shape, kind, dtype, tile, bins):
    """bins = 2: the passes behind the tiles are those through buckets of groups, which run only when the tiles
    have found the index out of order."""
    B, E, K, N = shape
    monkeypatch.setenv("TS_GROUP_FUSED", "2")
    monkeypatch.setenv("TS_GROUP_BINS", bins)
    if tile:
        monkeypatch.setenv("TS_GROUP_TILE", str(tile))
    rng = np.random.default_rng(E * 7 + K + N)
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K)) * 3).to(dtype)
    grad = torch.from_numpy(rng.standard_normal(size=(B, E, K))).to(dtype)
    check_against_oracle(capi, oracle, src, grad, fused_index(kind, rng, E, N), shape, dtype)

@pytest.mark.parametrize("shape,kind,dtype",
                         product(FUSED_SHAPES + [(1, 40_000, 8, 3000), (1, 1200, 64, 30), (2, 700, 48, 9), (1, 1500, 128, 40),
                                                (2, 600, 192, 9)],
                                 ["sorted", "skewed", "outside", "one_descent"], DTYPES))
@pytest.mark.parametrize("tile", [256, 0])
def test_std_and_logsumexp_one_pass_tiles_capi(capi, oracle, monkeypatch, shape, kind, dtype, tile):
    """scatter_std / scatter_logsumexp forward through the one-pass tiles for an index in order
    (group_fused_reduce.h), switched on at any size: runs inside a tile, runs that cross one border or fill whole
    tiles (their partials merged), entries outside [0, N), empty groups, rows of more than 256 bytes (column slices),
    and an index with one descent (the tiles notice, the passes through buckets of groups write every result again)."""
    B, E, K, N = shape
    if bucket_lanes(K, dtype) > 32:
        pytest.skip("rows held by more than 32 lanes: no buckets behind the tiles, the three passes keep the call")
    monkeypatch.setenv("TS_GROUP_FUSED", "2")
    monkeypatch.setenv("TS_GROUP_BINS", "2")
    if tile:
        monkeypatch.setenv("TS_GROUP_TILE", str(tile))
    exact = dtype in (torch.float32, torch.float64)
    if kind == "skewed" and not exact:
        pytest.skip("a 16-bit group sum over hundreds of entries is not meaningful")
    rng = np.random.default_rng(E * 23 + K + N)
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K)) * 3 + 1).to(dtype)
    index1 = fused_index(kind, rng, E, N)
    keep = (index1 >= 0) & (index1 < N)
    index = index1.view(1, E, 1).expand(B, E, K)
    src_k, index_k = src[:, keep], index[:, keep]
    e = EPS_T[dtype]
    want_cnt = np.bincount(index1[keep].numpy(), minlength=N)
    cnt_n = torch.from_numpy(want_cnt).double().view(1, N, 1).clamp(1).expand(B, N, K)
    abs64 = oracle.scatter(src_k.double().abs(), index_k, 1, None, N, "sum")[0]
    sum64 = oracle.scatter(src_k.double(), index_k, 1, None, N, "sum")[0]
    for unbiased in (True, False):
        total = torch.full((B, N, K), 7, dtype=dtype, device=DEV)
        count = torch.full((B, N), -7, dtype=torch.int32, device=DEV)
        out = torch.full((B, N, K), 7, dtype=dtype, device=DEV)
        capi.group_std_forward(src.to(DEV), index1.to(DEV), total, count, out, B, E, K, N, 0, 1, unbiased)
        torch.cuda.synchronize()
        for b in range(B):
            assert count.cpu().view(B, N)[b].tolist() == want_cnt.tolist()
        assert bool(((total.cpu().double() - sum64).abs() <= e * sum64.abs() + min(e, 4e-6) * abs64 + 1e-30).all())
        want = oracle.scatter_std(src_k if exact else src_k.double(), index_k, 1, None, N, unbiased).double()
        err = (out.cpu().double() - want).abs()
        if exact:
            bound = e * want + (1e-6 if dtype == torch.float32 else 1e-12)
        else:
            bound = 8.0 * e * want + 2.0 * e * (abs64 / cnt_n) * (1.0 + cnt_n.sqrt())
        assert bool((err <= bound).all()), (unbiased, float((err - bound).max()))
    out = torch.full((B, N, K), 7, dtype=dtype, device=DEV)
    capi.group_logsumexp(src.to(DEV), index1.to(DEV), out, B, E, K, N, 0, 1)
    torch.cuda.synchronize()
    want = oracle.scatter_logsumexp(src_k if exact else src_k.double(), index_k, 1, None, N).double()
    err = (out.cpu().double() - want).abs()
    bound = e * (1.0 + want.abs()) if exact else e * (30.0 + want.abs())
    assert bool((err <= bound).all()), float((err - bound).max())



def test_one_pass_kernels_leave_their_verdict(capi, monkeypatch):
    """The word behind the workspace of the three passes says whether the tiles found the index in order: 1 after
    one descent (the three passes then ran), 0 for a sorted index (they returned at once)."""
    monkeypatch.setenv("TS_GROUP_FUSED", "2")
    monkeypatch.setenv("TS_GROUP_TILE", "256")
    rng = np.random.default_rng(3)
    B, E, K, N = 1, 3000, 4, 200
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K))).float().to(DEV)
    for kind, verdict in (("one_descent", 1), ("sorted", 0), ("one_descent", 1)):
        index = fused_index(kind, rng, E, N).to(DEV)
        out = torch.empty_like(src)
        ws = capi.group_softmax(src, index, out, B, E, K, N, 0, 1, False)
        torch.cuda.synchronize()
        front = capi.lib().ts_group_softmax_workspace_bytes(capi._i(B), capi._i(N), capi._i(K), capi.DTYPE[torch.float32])
        assert int(ws[front - 256:front - 252].cpu().view(torch.int32)[0]) == verdict, kind


def test_one_pass_kernels_take_few_large_groups(capi, oracle, monkeypatch):
    """Few groups of many entries: the tiles' records do not fit the workspace of the three passes (2 x N x K words) and
    live in the scratch behind it (ts_group_workspace_bytes). The verdict word says that the tiles took the call."""
    monkeypatch.setenv("TS_GROUP_FUSED", "2")
    monkeypatch.setenv("TS_GROUP_BINS", "0")
    monkeypatch.setenv("TS_GROUP_TILE", "256")
    rng = np.random.default_rng(8)
    B, E, K, N = 1, 60_000, 4, 6
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K)) * 2).float()
    grad = torch.from_numpy(rng.standard_normal(size=(B, E, K))).float()
    index1 = torch.from_numpy(np.sort(rng.integers(0, N, size=E)))
    L = capi.lib()
    front = L.ts_group_softmax_workspace_bytes(capi._i(B), capi._i(N), capi._i(K), capi.DTYPE[torch.float32])
    assert L.ts_group_workspace_bytes(capi._i(B), capi._i(E), capi._i(K), capi._i(N), capi.DTYPE[torch.float32]) > front
    out = torch.empty((B, E, K), device=DEV)
    ws = capi.group_softmax(src.to(DEV), index1.to(DEV), out, B, E, K, N, 0, 1, False)
    torch.cuda.synchronize()
    assert int(ws[front - 256:front - 252].cpu().view(torch.int32)[0]) == 0
    check_against_oracle(capi, oracle, src, grad, index1, (B, E, K, N), torch.float32)


def test_one_pass_kernels_special_values(capi, oracle, monkeypatch):
    """The cases of test_special_values_capi in order, in tiles of 256 entries with the groups repeated so that
    runs of -inf, a NaN and an empty group meet tile borders."""
    monkeypatch.setenv("TS_GROUP_FUSED", "2")
    monkeypatch.setenv("TS_GROUP_TILE", "256")
    vals = [[0.2, 0.2], [0.0, -2.1, 3.2], [7.0], [], [-1.0, float("-inf")], [float("-inf")] * 2,
            [1.0, float("nan"), 2.0], []]
    reps = 90
    src = torch.tensor([v for _ in range(reps) for grp in vals for v in grp])
    index = torch.tensor([r * len(vals) + g for r in range(reps) for g, grp in enumerate(vals) for _ in grp])
    E, N = src.numel(), reps * len(vals)
    for log_space in (False, True):
        out = torch.empty(E, device=DEV)
        capi.group_softmax(src.to(DEV), index.to(DEV), out, 1, E, 1, N, 0, 1, log_space)
        torch.cuda.synchronize()
        want = (oracle.scatter_log_softmax(src, index, 0, 1e-12, N) if log_space
                else oracle.scatter_softmax(src, index, 0, dim_size=N))
        assert torch.allclose(out.cpu(), want, rtol=1e-5, atol=1e-7, equal_nan=True), log_space


@pytest.mark.parametrize("dtype,K", [(torch.float32, 8), (torch.bfloat16, 16), (torch.float32, 1)])
def test_one_pass_kernels_take_large_sorted_inputs(capi, monkeypatch, dtype, K):
    """At its default settings the library sends a sorted index of this size through the one-pass kernels;
    the three passes (switched on by the environment) give the reference result."""
    E, N = (1 << 21) + 77, 250_000
    if K == 1:
        E *= 4
    g = torch.Generator().manual_seed(5)
    index = torch.sort(torch.randint(0, N, (E,), generator=g)).values.to(DEV)
    src = (torch.randn((1, E, K), generator=g) * 3).to(dtype).to(DEV)
    grad = torch.randn((1, E, K), generator=g).to(dtype).to(DEV)
    res = {}
    for mode in ("0", "1"):
        monkeypatch.setenv("TS_GROUP_FUSED", mode)
        for log_space in (False, True):
            out, gin = torch.empty_like(src), torch.empty_like(src)
            capi.group_softmax(src, index, out, 1, E, K, N, 0, 1, log_space)
            capi.group_softmax_backward(out, grad, index, gin, 1, E, K, N, 0, 1, log_space)
            res[mode, log_space] = (out.double(), gin.double())
    torch.cuda.synchronize()
    e = EPS_T[dtype]
    for log_space in (False, True):
        a, b = res["0", log_space], res["1", log_space]
        assert bool(((a[0] - b[0]).abs() <= 16 * e * (1.0 + a[0].abs())).all())
        assert bool(((a[1] - b[1]).abs() <= 64 * e * (1.0 + a[1].abs())).all())

@pytest.mark.parametrize("kind", ["sorted", "random", "hubs"])
@pytest.mark.parametrize("dtype,K", [(torch.float32, 8), (torch.float32, 1), (torch.bfloat16, 16), (torch.float64, 3)])
def test_operators_at_sizes_that_take_the_buckets(ts, dtype, K, kind):
    """scatter_std, scatter_logsumexp and scatter_softmax through the operators at the library's default settings, at a
    size from which the route through buckets of groups applies (group_binned.h), against a double-precision
    evaluation with torch's own index_add_ / scatter_reduce_ on the CPU (on the device a double-precision index_add_
    is a compare-and-swap loop, which a hub group of 600 k entries stalls for minutes): sorted, random and a power-law
    index whose hub groups fill many chunks."""
    E, N = 1_200_000, 150_000
    if K == 1:
        E *= 2
    g = torch.Generator().manual_seed(7)
    if kind == "hubs":
        w = torch.arange(1, N + 1, dtype=torch.float64) ** -1.3
        index = torch.multinomial(w, E, replacement=True, generator=g)
    else:
        index = torch.randint(0, N, (E,), generator=g)
        if kind == "sorted":
            index = index.sort().values
    src_cpu = (torch.randn((E, K), generator=g) * 2 + 0.5).to(dtype)
    src, x = src_cpu.to(DEV), src_cpu.double()
    index_dev = index.to(DEV)
    idx2 = index.view(E, 1).expand(E, K)
    e = EPS_T[dtype]
    cnt = torch.bincount(index, minlength=N).double().view(N, 1)
    total = torch.zeros((N, K), dtype=torch.float64, device='cpu').index_add_(0, index, x)
    mean = total / cnt.clamp(min=1)
    # std (unbiased)
    m2 = torch.zeros((N, K), dtype=torch.float64, device='cpu').index_add_(0, index, (x - mean[index]) ** 2)
    want = (m2 / ((cnt - 1).clamp(min=1) + 1e-6)).sqrt()
    got = ts.scatter_std(src, index_dev, 0, None, N).double().cpu()
    mean_abs = torch.zeros((N, K), dtype=torch.float64, device='cpu').index_add_(0, index, x.abs()) / cnt.clamp(min=1)
    if dtype in (torch.float32, torch.float64):
        bound = 4 * e * want + 4 * e * mean_abs + 1e-30
    else:
        bound = 8.0 * e * want + 2.0 * e * mean_abs * (1.0 + cnt.sqrt())
    assert bool(((got - want).abs() <= bound).all()), float(((got - want).abs() - bound).max())
    # logsumexp and softmax
    gmax = torch.full((N, K), float("-inf"), dtype=torch.float64, device='cpu').scatter_reduce_(0, idx2, x, "amax")
    z = x - gmax[index]
    gsum = torch.zeros((N, K), dtype=torch.float64, device='cpu').index_add_(0, index, z.exp())
    want_lse = torch.where(cnt > 0, gsum.log() + gmax, torch.zeros_like(gsum))
    got_lse = ts.scatter_logsumexp(src, index_dev, 0, None, N).double().cpu()
    lse_bound = e * (1.0 + want_lse.abs()) * (4 if dtype in (torch.float32, torch.float64) else 30)
    assert bool(((got_lse - want_lse).abs() <= lse_bound).all()), float(((got_lse - want_lse).abs() - lse_bound).max())
    want_sm = z.exp() / gsum[index]
    got_sm = ts.scatter_softmax(src, index_dev, 0, N).double().cpu()
    sm_bound = e * (4.0 + z.abs()) * want_sm * (4 if dtype in (torch.float32, torch.float64) else 1) + 1e-30
    assert bool(((got_sm - want_sm).abs() <= sm_bound).all()), float(((got_sm - want_sm).abs() - sm_bound).max())
    # the gradient of std through the operator (one line per entry in the backward pass)
    xs = src.clone().requires_grad_(True)
    y = ts.scatter_std(xs, index_dev, 0, None, N)
    go = torch.randn((N, K), generator=g).to(dtype)
    (gi,) = torch.autograd.grad(y, xs, go.to(DEV))
    gi, y = gi.cpu(), y.detach().cpu()
    div = (cnt - 1).clamp(min=1) + 1e-6
    want_g = (go.double() / (y.detach().double() * div))[index] * (x - mean[index])
    live = (cnt[index] > 1).expand(E, K) & torch.isfinite(want_g)
    scale = (go.double().abs() / y.detach().double().clamp_min(1e-300))[index]
    gb = 16 * e * (want_g.abs() + scale * mean_abs[index] / cnt[index].clamp(min=1)) + (2.0 ** -24 if dtype == torch.float16 else 1e-30)
    assert bool(((gi.double() - want_g).abs()[live] <= gb[live]).all())


@pytest.mark.parametrize("bins", ["0", "2"])
def test_special_values_capi(capi, oracle, monkeypatch, bins):
    """-inf entries, a group of only -inf, NaN in a group, entries outside [0, N), an empty group; through the three
    passes (bins = 0) and through buckets of groups (bins = 2), softmax and logsumexp. A hub variant repeats the
    values so that the groups of the first bucket fill several chunks (slabs merged with -inf and NaN partials)."""
    monkeypatch.setenv("TS_GROUP_BINS", bins)
    src = torch.tensor([0.2, 0, 0.2, -2.1, 3.2, 7, -1, float("-inf"), float("-inf"), float("-inf"),
                        1.0, float("nan"), 2.0, 5.0])
    index = torch.tensor([0, 1, 0, 1, 1, 2, 4, 4, 5, 5, 6, 6, 6, 9])
    E, N = src.numel(), 8
    keep = index < N
    for log_space in (False, True):
        out = torch.empty(E, device=DEV)
        capi.group_softmax(src.to(DEV), index.to(DEV), out, 1, E, 1, N, 0, 1, log_space)
        torch.cuda.synchronize()
        fn = oracle.scatter_log_softmax if log_space else oracle.scatter_softmax
        want = fn(src[keep], index[keep], 0, dim_size=N) if not log_space else fn(src[keep], index[keep], 0, 1e-12, N)
        got = out.cpu()
        assert torch.allclose(got[keep], want, rtol=1e-5, atol=1e-7, equal_nan=True), (log_space, got, want)
        assert float(got[~keep].abs().max()) == 0.0
    for reps in (1, 6000):  # 6000: 78 000 single values in 8 groups, the groups of three entries in three chunks each
        s, i = src[keep].repeat(reps), index[keep].repeat(reps)
        out = torch.full((N,), 7.0, device=DEV)
        capi.group_logsumexp(s.to(DEV), i.to(DEV), out, 1, s.numel(), 1, N, 0, 1)
        torch.cuda.synchronize()
        want = oracle.scatter_logsumexp(s.double(), i, 0, None, N)
        assert torch.allclose(out.cpu().double(), want, rtol=1e-5, atol=1e-6, equal_nan=True), (reps, out, want)
        for log_space in (False, True):
            o = torch.empty(s.numel(), device=DEV)
            capi.group_softmax(s.to(DEV), i.to(DEV), o, 1, s.numel(), 1, N, 0, 1, log_space)
            torch.cuda.synchronize()
            w = (oracle.scatter_log_softmax(s.double(), i, 0, 1e-12, N) if log_space
                 else oracle.scatter_softmax(s.double(), i, 0, dim_size=N))
            assert torch.allclose(o.cpu().double(), w, rtol=1e-5, atol=1e-6, equal_nan=True), (reps, log_space)


def test_workspace_and_argument_checks(capi):
    import ctypes
    L = capi.lib()
    x = torch.zeros(8, device=DEV)
    idx = torch.zeros(8, dtype=torch.long, device=DEV)
    ws = torch.empty(16, dtype=torch.uint8, device=DEV)
    args = (capi._p(x), capi._p(idx), capi._p(x), capi._i(1), capi._i(8), capi._i(1), capi._i(4), capi._i(0),
            capi._i(1))
    rc = L.ts_group_softmax(*args, capi.DTYPE[torch.float32], 0, ctypes.c_double(0.0), capi._p(ws),
                            ctypes.c_size_t(16), None)
    assert rc == 3  # TS_ERR_WORKSPACE
    rc = L.ts_group_softmax(*args, capi.DTYPE[torch.int32], 0, ctypes.c_double(0.0), capi._p(ws),
                            ctypes.c_size_t(16), None)
    assert rc == 2  # TS_ERR_UNSUPPORTED: floating types only


# ------------------------------------------------------------------ operator level
def per_group(lib, src, index, dim, n):
    out = torch.zeros_like(src)
    for g in range(n):
        sel = (index == g).nonzero().flatten()
        if sel.numel() > 0:
            out = out.index_copy(dim, sel, lib(src.index_select(dim, sel), dim))
    return out


@pytest.mark.parametrize("dim,shape,log_space", product([0, 1, 2, -1], [(40, 30, 20)], [False, True]))
def test_operator_dims_and_autograd(ts, dim, shape, log_space):
    g = torch.Generator().manual_seed(5)
    d = dim if dim >= 0 else len(shape) + dim
    src_cpu = torch.randn(shape, generator=g, dtype=torch.double) * 2
    index = torch.randint(0, 6, (shape[d],), generator=g)
    grad = torch.randn(shape, generator=g, dtype=torch.double)
    lib = torch.log_softmax if log_space else torch.softmax
    ref = src_cpu.clone().requires_grad_(True)
    want = per_group(lib, ref, index, d, 6)
    want.backward(grad)
    fn = ts.scatter_log_softmax if log_space else ts.scatter_softmax
    src = src_cpu.to(DEV).requires_grad_(True)
    shape1 = [1] * len(shape)
    shape1[d] = shape[d]
    for idx in (index.to(DEV), index.view(shape1).expand(shape).to(DEV)):
        if idx.dim() == 1 and d != 0:
            idx = idx.view(shape1[:d + 1])  # leading dims broadcast, trailing dims implied
        src.grad = None
        out = fn(src, idx, dim)
        out.backward(grad.to(DEV))
        assert torch.allclose(out.detach().cpu(), want.detach(), rtol=1e-9, atol=1e-9)
        assert torch.allclose(src.grad.cpu(), ref.grad, rtol=1e-8, atol=1e-9)


def test_operator_reference_cases_script_and_fallback(ts, oracle):
    # test/composite/test_softmax.py:6-54
    src = torch.tensor([0.2, 0, 0.2, -2.1, 3.2, 7, -1, float("-inf")], device=DEV, requires_grad=True)
    index = torch.tensor([0, 1, 0, 1, 1, 2, 4, 4], device=DEV)
    for fn, ofn in ((ts.scatter_softmax, oracle.scatter_softmax), (ts.scatter_log_softmax, oracle.scatter_log_softmax)):
        out = fn(src, index)
        assert torch.allclose(out.detach().cpu(), ofn(src.detach().cpu(), index.cpu()), equal_nan=True)
        out.backward(torch.randn_like(out))
        jit = torch.jit.script(fn)
        assert jit(src, index).tolist() == out.tolist()
    # an index that differs between the columns of a row: composed from the scatter operators
    g = torch.Generator().manual_seed(1)
    x = torch.randn(50, 6, generator=g)
    idx = torch.randint(0, 5, (50, 6), generator=g)
    got = ts.scatter_softmax(x.to(DEV), idx.to(DEV), 0)
    assert torch.allclose(got.cpu(), oracle.scatter_softmax(x, idx, 0), rtol=1e-5, atol=1e-7)
    got = ts.scatter_log_softmax(x.to(DEV), idx.to(DEV), 0, dim_size=7)
    assert torch.allclose(got.cpu(), oracle.scatter_log_softmax(x, idx, 0, 1e-12, 7), rtol=1e-5, atol=1e-6)
    # per-row index on the last dimension (B > 1, K = 1) is the fused path
    x = torch.randn(7, 90, generator=g)
    idx = torch.randint(0, 9, (7, 90), generator=g)
    got = ts.scatter_softmax(x.to(DEV), idx.to(DEV), -1)
    assert torch.allclose(got.cpu(), oracle.scatter_softmax(x, idx, -1), rtol=1e-5, atol=1e-7)
    # zero-size input, integer input
    assert ts.scatter_softmax(torch.empty(0, 4, device=DEV), torch.empty(0, dtype=torch.long, device=DEV), 0).shape == (0, 4)
    with pytest.raises(ValueError):
        ts.scatter_softmax(torch.ones(4, dtype=torch.long, device=DEV), torch.zeros(4, dtype=torch.long, device=DEV))


# ------------------------------------------------------------------ logsumexp
# one shape whose hub group fills more than 32 chunks of its bucket (the slabs merged by wavefronts side by side)
BIN_SHAPES = SHAPES + [(1, 300_000, 8, 2000)]


@pytest.mark.parametrize("shape,kind,dtype", product(BIN_SHAPES, ["random", "sorted", "hub"], DTYPES))
@pytest.mark.parametrize("route", ["passes", "buckets"])
def test_logsumexp_forward_and_backward_capi(capi, oracle, monkeypatch, shape, kind, dtype, route):
    """route = buckets: the call goes through buckets of groups (group_binned.h) at any size; a hub group fills
    several chunks of its bucket, whose slabs are merged."""
    B, E, K, N = shape
    if route == "buckets":
        if bucket_lanes(K, dtype) > 32:
            pytest.skip("rows held by more than 32 lanes stay with the three passes")
        monkeypatch.setenv("TS_GROUP_BINS", "2")
        assert capi.group_bins_workspace_bytes(B, E, K, N + 3, dtype) > 0
    elif E > 100_000:
        pytest.skip("a shape for the buckets")
    else:
        monkeypatch.setenv("TS_GROUP_BINS", "0")
    N = N + 3  # the last groups stay empty
    rng = np.random.default_rng(E * 17 + K)
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K)) * 3).to(dtype)
    index1 = make_index(kind, rng, E, N - 3)
    index = index1.view(1, E, 1).expand(B, E, K)
    exact = dtype in (torch.float32, torch.float64) and E <= 100_000
    ref_src = src if exact else src.double()
    out = torch.full((B, N, K), 7, dtype=dtype, device=DEV)
    capi.group_logsumexp(src.to(DEV), index1.to(DEV), out, B, E, K, N, 0, 1)
    torch.cuda.synchronize()
    want = oracle.scatter_logsumexp(ref_src, index, 1, None, N).double()
    e = EPS_T[dtype]
    err = (out.cpu().double() - want).abs()
    # 16-bit floats: z is rounded before the exp (relative error of a term up to eps_T * |z|, |z| <~ 25 here)
    bound = e * (1.0 + want.abs()) if exact else e * (30.0 + want.abs())
    assert bool((err <= bound).all()), float((err - bound).max())
    assert float(out[:, N - 3:, :].abs().max()) == 0.0

    grad = torch.from_numpy(rng.standard_normal(size=(B, N, K))).to(dtype)
    y64 = out.cpu().double()
    want_g = oracle.scatter_logsumexp_backward(src.double(), y64, grad.double(), index, 1)
    gbound = 8 * e * want_g.abs() * (1 + (src.double() - y64.gather(1, index)).abs()) + \
        (2.0 ** -23 if dtype == torch.float16 else 1e-30)
    for with_workspace in (True, False):  # a group's result and gradient laid side by side first, or gathered
        grad_in = torch.empty((B, E, K), dtype=dtype, device=DEV)
        capi.group_logsumexp_backward(src.to(DEV), index1.to(DEV), out, grad.to(DEV), grad_in, B, E, K, N, 0, 1,
                                      with_workspace)
        torch.cuda.synchronize()
        gerr = (grad_in.cpu().double() - want_g).abs()
        assert bool((gerr <= gbound).all()), ("backward", with_workspace, float((gerr - gbound).max()))


def test_logsumexp_operator(ts, oracle):
    # test/composite/test_logsumexp.py:5-45
    inputs = torch.tensor([0.5, 0.5, 0.0, -2.1, 3.2, 7.0, -1.0, -100.0], device=DEV, requires_grad=True)
    index = torch.tensor([0, 0, 1, 1, 1, 2, 4, 4], device=DEV)
    outputs = ts.scatter_logsumexp(inputs, index)
    for part, got in zip(inputs.split([2, 3, 1, 0, 2]), outputs.unbind()):
        if part.numel() > 0:
            assert torch.allclose(got, torch.logsumexp(part, dim=0), rtol=1e-6)
        else:
            assert got.item() == 0.0
    outputs.backward(torch.randn_like(outputs))
    jit = torch.jit.script(ts.scatter_logsumexp)
    assert jit(inputs, index).tolist() == outputs.tolist()
    out = torch.tensor([-10.0, -10.0], device=DEV)
    ts.scatter_logsumexp(src=torch.tensor([-1.0, -50.0], device=DEV), index=torch.tensor([0, 0], device=DEV), out=out)
    assert out.cpu().allclose(torch.tensor([-0.9999, -10.0]), atol=1e-4)
    # special values: NaN entries drop out, a group of only -inf gives 0
    x = torch.tensor([1.0, float("nan"), 2.0, float("-inf"), float("-inf"), 3.0])
    idx = torch.tensor([0, 0, 0, 1, 1, 3])
    got = ts.scatter_logsumexp(x.to(DEV), idx.to(DEV), dim_size=5)
    assert torch.allclose(got.cpu(), oracle.scatter_logsumexp(x, idx, -1, None, 5), rtol=1e-6)
    # dims, autograd against the per-group library routine
    g = torch.Generator().manual_seed(2)
    src_cpu = torch.randn(12, 40, 6, generator=g, dtype=torch.double)
    idx = torch.randint(0, 5, (40,), generator=g)
    ref = src_cpu.clone().requires_grad_(True)
    want = torch.stack([torch.logsumexp(ref.index_select(1, (idx == n).nonzero().flatten()), 1) for n in range(5)], 1)
    grad = torch.randn(12, 5, 6, generator=g, dtype=torch.double)
    want.backward(grad)
    src = src_cpu.to(DEV).requires_grad_(True)
    got = ts.scatter_logsumexp(src, idx.view(1, 40).to(DEV), 1, dim_size=5)
    got.backward(grad.to(DEV))
    assert torch.allclose(got.detach().cpu(), want.detach(), rtol=1e-9, atol=1e-9)
    assert torch.allclose(src.grad.cpu(), ref.grad, rtol=1e-8, atol=1e-10)
    # an index that differs between the columns of a row: composed from the scatter operators
    x = torch.randn(50, 6, generator=g)
    idx2 = torch.randint(0, 5, (50, 6), generator=g)
    got = ts.scatter_logsumexp(x.to(DEV), idx2.to(DEV), 0)
    assert torch.allclose(got.cpu(), oracle.scatter_logsumexp(x, idx2, 0), rtol=1e-5, atol=1e-6)
    with pytest.raises(ValueError):
        ts.scatter_logsumexp(torch.ones(4, dtype=torch.long, device=DEV), torch.zeros(4, dtype=torch.long, device=DEV))


# ------------------------------------------------------------------ std
STD_SHAPES = [
    # B, E, K, N
    (1, 5000, 1, 600), (2, 3000, 4, 300), (1, 2000, 8, 250), (1, 1500, 3, 200), (1, 900, 64, 100),
    (1, 700, 130, 80), (3, 400, 16, 50), (1, 1, 1, 1), (1, 257, 2, 300),
    # 2^16 terms and more, rows of up to 128 columns: the group sums go through the accumulator table
    (1, 70_000, 1, 3000), (2, 6000, 8, 500), (1, 1200, 64, 90), (1, 600, 128, 40),
]


@pytest.mark.parametrize("shape,kind,dtype,unbiased",
                         product(STD_SHAPES, ["random", "sorted", "hub"], DTYPES, [True, False]))
def test_std_forward_and_backward_capi(capi, oracle, shape, kind, dtype, unbiased):
    """fp32 / fp64 against the oracle's sequence in the same type. 16-bit floats against the
    oracle in fp64 on the same inputs, within the roundings the reference's sequence commits in
    the element type (deviation, square, sum, quotient, root: a few ulp of the result); no hub
    groups there, whose sum in a 16-bit type the reference itself cannot hold."""
    B, E, K, N = shape
    exact = dtype in (torch.float32, torch.float64)
    if kind == "hub" and not exact:
        pytest.skip("a 16-bit group sum over hundreds of entries is not meaningful")
    rng = np.random.default_rng(E * 17 + K)
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K)) * 3 + 1).to(dtype)
    grad = torch.from_numpy(rng.standard_normal(size=(B, N, K))).to(dtype)
    index1 = make_index(kind, rng, E, N)
    index = index1.view(1, E, 1).expand(B, E, K)
    src_d, idx_d = src.to(DEV), index1.to(DEV)
    total = torch.empty((B, N, K), dtype=dtype, device=DEV)
    capi.scatter(src_d, idx_d, total, None, B, E, K, N, 0, 1, 0, capi.SUM, False)
    count = torch.empty((B, N), dtype=torch.int32, device=DEV)
    capi.scatter_count(idx_d, count, B, E, N, 0, 1)
    out = torch.empty((B, N, K), dtype=dtype, device=DEV)
    capi.group_std(src_d, idx_d, total, count, out, B, E, K, N, 0, 1, unbiased)
    torch.cuda.synchronize()
    assert count.cpu().view(B, N)[0].tolist() == np.bincount(index1.numpy(), minlength=N).tolist()

    ref_src = src if exact else src.double()
    want = oracle.scatter_std(ref_src, index, 1, None, N, unbiased).double()
    e = EPS_T[dtype]
    err = (out.cpu().double() - want).abs()
    cnt_n = count.cpu().double().view(B, N, 1).clamp(1).expand(B, N, K)
    mean_abs = oracle.scatter(src.double().abs(), index, 1, None, N, "sum")[0] / cnt_n
    if exact:
        bound = e * want + (1e-6 if dtype == torch.float32 else 1e-12)
    else:  # the mean carries the roundings of a sum in the element type; an offset of the mean adds to the std
        bound = 8.0 * e * want + 2.0 * e * mean_abs * (1.0 + cnt_n.sqrt())
    assert bool((err <= bound).all()), float((err - bound).max())

    std64, want_g = oracle.scatter_std_backward(src.double(), grad.double(), index, 1, N, unbiased)
    for with_workspace in (True, False):  # mean and grad / (std * divisor) laid side by side first, or gathered
        grad_in = torch.empty((B, E, K), dtype=dtype, device=DEV)
        capi.group_std_backward(src_d, idx_d, total, count, out, grad.to(DEV), grad_in, B, E, K, N, 0, 1, unbiased,
                                with_workspace)
        torch.cuda.synchronize()
        check_std_gradient(grad_in.cpu().double(), want_g, std64, grad, index, cnt_n, mean_abs, exact, e, dtype)


def check_std_gradient(got_g, want_g, std64, grad, index, cnt_n, mean_abs, exact, e, dtype):
    # a group whose std is 0 (one entry, or equal entries): NaN on both sides
    dead = (std64 == 0).gather(1, index)
    assert bool(torch.isnan(got_g[dead]).all()) and bool(torch.isnan(want_g[dead]).all())
    live = ~dead & ~torch.isnan(want_g)
    # the deviation src - mean cancels: its error is that of the mean, relative to the group's spread
    scale = (grad.double().abs() / std64.clamp_min(1e-300)).gather(1, index)
    cnt = cnt_n.gather(1, index)
    gbound = (8 if exact else 16) * e * (want_g.abs() + scale * mean_abs.gather(1, index) / cnt)
    if dtype == torch.float16:
        gbound = gbound + 2.0 ** -24  # gradients below 2^-14 are subnormal in fp16: absolute spacing 2^-24
    gerr = (got_g - want_g).abs()
    assert bool((gerr[live] <= gbound[live]).all()), float((gerr[live] - gbound[live]).max())


@pytest.mark.parametrize("shape,kind,dtype,unbiased",
                         product(STD_SHAPES + [(1, 300_000, 8, 2000)], ["random", "sorted", "hub"], DTYPES, [True, False]))
def test_std_forward_through_buckets_capi(capi, oracle, monkeypatch, shape, kind, dtype, unbiased):
    """ts_group_std_forward: group sums, counts and standard deviation from one gather of src through buckets of
    groups (group_binned.h), at any size. Bars as in test_std_forward_and_backward_capi; the count is exact, the group
    sum is the double-precision sum rounded once."""
    B, E, K, N = shape
    exact = dtype in (torch.float32, torch.float64)
    if kind == "hub" and not exact:
        pytest.skip("a 16-bit group sum over hundreds of entries is not meaningful")
    if bucket_lanes(K, dtype) > 32:
        pytest.skip("rows held by more than 32 lanes stay with the three passes")
    monkeypatch.setenv("TS_GROUP_BINS", "2")
    rng = np.random.default_rng(E * 19 + K)
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K)) * 3 + 1).to(dtype)
    index1 = make_index(kind, rng, E, N)
    if E > 10:
        index1[3] = -1   # outside [0, N): belongs to no group
        index1[E - 2] = N
    index = index1.view(1, E, 1).expand(B, E, K)
    keep = (index1 >= 0) & (index1 < N)
    total = torch.full((B, N, K), 7, dtype=dtype, device=DEV)
    count = torch.full((B, N), -7, dtype=torch.int32, device=DEV)
    out = torch.full((B, N, K), 7, dtype=dtype, device=DEV)
    used = capi.group_std_forward(src.to(DEV), index1.to(DEV), total, count, out, B, E, K, N, 0, 1, unbiased)
    torch.cuda.synchronize()
    assert used > 8 * B * E
    want_cnt = np.bincount(index1[keep].numpy(), minlength=N)
    for b in range(B):
        assert count.cpu().view(B, N)[b].tolist() == want_cnt.tolist()
    src_k, index_k = src[:, keep], index[:, keep]
    sum64 = oracle.scatter(src_k.double(), index_k, 1, None, N, "sum")[0]
    abs64 = oracle.scatter(src_k.double().abs(), index_k, 1, None, N, "sum")[0]
    e = EPS_T[dtype]
    # the group sum: lanes add their few entries in fp32 (fp64 for doubles) and meet in double precision; rounded once
    assert bool(((total.cpu().double() - sum64).abs() <= e * sum64.abs() + min(e, 4e-6) * abs64 + 1e-30).all())
    ref_src = src_k if exact and E <= 100_000 else src_k.double()
    want = oracle.scatter_std(ref_src, index_k, 1, None, N, unbiased).double()
    err = (out.cpu().double() - want).abs()
    cnt_n = torch.from_numpy(want_cnt).double().view(1, N, 1).clamp(1).expand(B, N, K)
    mean_abs = abs64 / cnt_n
    if exact:
        bound = e * want + (1e-6 if dtype == torch.float32 else 1e-12)
    else:
        bound = 8.0 * e * want + 2.0 * e * mean_abs * (1.0 + cnt_n.sqrt())
    assert bool((err <= bound).all()), float((err - bound).max())


def test_bucket_route_declines(capi, monkeypatch):
    """Where the buckets of groups do not apply the size query says 0 and ts_group_std_forward refuses."""
    assert capi.group_bins_workspace_bytes(1, 1000, 8, 100, torch.float32) == 0        # small
    assert capi.group_bins_workspace_bytes(1, 1 << 22, 8, 1 << 20, torch.float32) > 0
    assert capi.group_bins_workspace_bytes(1, 1 << 22, 8, 1 << 20, torch.int32) == 0   # floating types only
    assert capi.group_bins_workspace_bytes(1, 1 << 20, 256, 1 << 10, torch.float32) == 0  # 64 lanes per row
    monkeypatch.setenv("TS_GROUP_BINS", "0")
    assert capi.group_bins_workspace_bytes(1, 1 << 22, 8, 1 << 20, torch.float32) == 0
    src = torch.zeros((1000, 8), device=DEV)
    idx = torch.zeros(1000, dtype=torch.long, device=DEV)
    total, out = torch.empty((10, 8), device=DEV), torch.empty((10, 8), device=DEV)
    count = torch.empty(10, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError):
        capi.group_std_forward(src, idx, total, count, out, 1, 1000, 8, 10, 0, 1)


@pytest.mark.parametrize("dim,unbiased", product([0, 1, 2, -1], [True, False]))
def test_std_operator_dims_and_autograd(ts, oracle, dim, unbiased):
    shape = (40, 30, 20)
    g = torch.Generator().manual_seed(11)
    d = dim if dim >= 0 else len(shape) + dim
    src_cpu = torch.randn(shape, generator=g, dtype=torch.double) * 2 + 0.5
    index = torch.randint(0, 6, (shape[d],), generator=g)
    shape_g = list(shape)
    shape_g[d] = 8  # two groups without entries
    grad = torch.randn(shape_g, generator=g, dtype=torch.double)
    want, want_g = oracle.scatter_std_backward(src_cpu, grad, index, d, 8, unbiased)
    # torch's own std per group, where the group has more than one entry
    for grp in range(6):
        sel = (index == grp).nonzero().flatten()
        if sel.numel() > 1:
            lib = src_cpu.index_select(d, sel).std(d, unbiased=unbiased)
            assert torch.allclose(want.select(d, grp), lib, rtol=1e-5)
    src = src_cpu.to(DEV).requires_grad_(True)
    shape1 = [1] * len(shape)
    shape1[d] = shape[d]
    for idx in (index.to(DEV), index.view(shape1).expand(shape).to(DEV)):
        if idx.dim() == 1 and d != 0:
            idx = idx.view(shape1[:d + 1])
        src.grad = None
        out = ts.scatter_std(src, idx, dim, dim_size=8, unbiased=unbiased)
        out.backward(grad.to(DEV))
        assert torch.allclose(out.detach().cpu(), want, rtol=1e-9, atol=1e-12)
        assert float(out.detach().select(d, 7).abs().max()) == 0.0
        assert torch.allclose(src.grad.cpu(), want_g, rtol=1e-7, atol=1e-9, equal_nan=True)


def test_std_operator_reference_case_script_and_fallback(ts, oracle):
    # test/composite/test_std.py:5-23
    src = torch.tensor([[2.0, 0, 1, 4, 3], [0, 2, 1, 3, 4]], device=DEV, requires_grad=True)
    index = torch.tensor([[0, 0, 0, 0, 0], [1, 1, 1, 1, 1]], device=DEV)
    out = ts.scatter_std(src, index, dim=-1, unbiased=True)
    std = src.std(dim=-1, unbiased=True)[0]
    assert torch.allclose(out, torch.tensor([[std, 0], [0, std]], device=DEV))
    out.backward(torch.randn_like(out))
    jit = torch.jit.script(ts.scatter_std)
    assert jit(src, index, dim=-1, unbiased=True).tolist() == out.tolist()
    g = torch.Generator().manual_seed(2)
    # an index that differs between the columns of a row, and `out` given: composed as upstream
    x = torch.randn(60, 5, generator=g)
    idx = torch.randint(0, 4, (60, 5), generator=g)
    got = ts.scatter_std(x.to(DEV), idx.to(DEV), 0)
    assert torch.allclose(got.cpu(), oracle.scatter_std(x, idx, 0), rtol=1e-5, atol=1e-6)
    idx1 = torch.randint(0, 4, (60,), generator=g)
    base = torch.rand(6, 5, generator=g)
    got = ts.scatter_std(x.to(DEV), idx1.to(DEV), 0, out=base.clone().to(DEV), unbiased=False)
    assert torch.allclose(got.cpu(), oracle.scatter_std(x, idx1, 0, base.clone(), None, False), rtol=1e-5, atol=1e-6)
    # fused and composed agree (fp32, 1-D index along dim 0; last dim with a per-row index)
    fused = ts.scatter_std(x.to(DEV), idx1.to(DEV), 0, dim_size=6)
    assert torch.allclose(fused.cpu(), oracle.scatter_std(x, idx1, 0, None, 6), rtol=1e-5, atol=1e-6)
    x = torch.randn(7, 90, generator=g)
    idx = torch.randint(0, 9, (7, 90), generator=g)
    got = ts.scatter_std(x.to(DEV), idx.to(DEV), -1)
    assert torch.allclose(got.cpu(), oracle.scatter_std(x, idx, -1), rtol=1e-5, atol=1e-6)
    # integer input goes through the composed sequence as upstream (count + 1e-6 promotes to float)
    xi = torch.randint(0, 9, (50,), generator=g)
    ii = torch.randint(0, 5, (50,), generator=g)
    got = ts.scatter_std(xi.to(DEV), ii.to(DEV), 0)
    assert torch.allclose(got.cpu(), oracle.scatter_std(xi, ii, 0), rtol=1e-5, atol=1e-6)
    # zero-size input
    assert ts.scatter_std(torch.empty(0, 4, device=DEV), torch.empty(0, dtype=torch.long, device=DEV), 0,
                          dim_size=3).shape == (3, 4)


@pytest.mark.parametrize("kind", ["sorted", "random"])
def test_group_operators_under_graph_replay(ts, kind):
    """scatter_std, scatter_logsumexp and scatter_softmax at a size that takes the one-pass tiles (sorted) or the
    buckets of groups (random), captured in a graph and replayed three times with fresh inputs and eager work in
    between: every replay equals the eager call on the same inputs (the passes clear their own counters with kernels,
    the verdict word of the tiles is rewritten by every call)."""
    E, N, K = 700_000, 90_000, 8
    g = torch.Generator().manual_seed(13)
    index = torch.randint(0, N, (E,), generator=g)
    if kind == "sorted":
        index = index.sort().values
    index = index.to(DEV)
    static_src = torch.zeros((E, K), device=DEV)

    def step():
        return (ts.scatter_std(static_src, index, 0, None, N), ts.scatter_logsumexp(static_src, index, 0, None, N),
                ts.scatter_softmax(static_src, index, 0, N))

    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                step()  # warm-up on a side stream
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            outs = step()
        for rep in range(3):
            static_src.copy_(torch.randn((E, K), generator=g).to(DEV))
            graph.replay()
            torch.cuda.synchronize()
            got = [o.clone() for o in outs]
            eager = step()
            torch.cuda.synchronize()
            for a, b in zip(got, eager):
                assert torch.allclose(a, b, rtol=1e-5, atol=1e-6), (rep, float((a - b).abs().max()))
