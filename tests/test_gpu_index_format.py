"""Index formats and the sorted scatter on the GPU: ts_index_to_indptr,
ts_indptr_to_index, ts_sort_index and ts_segment_csr_permuted through the C ABI,
SortedIndex / scatter_sorted through the Python API.

Bars: permutations, row pointers, min / max values and arg positions are bit-exact
against the CPU oracle (its plain-loop restatement at small sizes, numpy's stable
argsort -- which the CPU suite pins to the same loops -- at large ones); sum / mean
within rtol 1e-5 (fp32) / 1e-2 (16-bit floats) of the oracle's scatter, integers exact.
"""
from itertools import product

import numpy as np
import pytest
import torch

from helpers import random_values

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
RTOL = {torch.float32: 1e-5, torch.float64: 1e-12, torch.bfloat16: 1e-2, torch.float16: 1e-2}
ALL_DTYPES = [torch.float32, torch.float64, torch.float16, torch.bfloat16, torch.int32, torch.int64, torch.int16,
              torch.int8, torch.uint8]


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
    if kind == "hub":
        idx = rng.integers(0, N, size=E)
        idx[E // 4: 3 * E // 4] = N // 2
    elif kind == "sorted":
        idx = np.sort(rng.integers(0, N, size=E))
    elif kind == "gaps":  # most rows empty
        idx = rng.integers(0, max(N // 16, 1), size=E) * 16 % N
    else:
        idx = rng.integers(0, N, size=E)
    return torch.from_numpy(idx.astype(np.int64))


def sort_on_gpu(capi, index, N):
    E = index.numel()
    perm = torch.empty(E, dtype=torch.int32, device=DEV)
    indptr = torch.empty(N + 1, dtype=torch.long, device=DEV)
    capi.sort_index(index.to(DEV), perm, indptr, E, N)
    torch.cuda.synchronize()
    return perm, indptr


@pytest.mark.parametrize("E,N,kind", [(0, 0, "random"), (0, 7, "random"), (1, 1, "random"), (300, 17, "random"),
                                      (4000, 3, "hub"), (3000, 5000, "gaps"), (2500, 40, "sorted")])
def test_sort_and_formats_against_oracle_loops(capi, oracle, E, N, kind):
    rng = np.random.default_rng(E * 3 + N)
    index = make_index(kind, rng, E, N) if E > 0 else torch.zeros(0, dtype=torch.long)
    perm, indptr = sort_on_gpu(capi, index, N)
    want_perm, want_ptr = oracle.sort_index(index, N)
    assert torch.equal(perm.cpu().long(), want_perm)
    assert torch.equal(indptr.cpu(), want_ptr)
    srt = index[want_perm]
    ptr2 = torch.empty(N + 1, dtype=torch.long, device=DEV)
    capi.index_to_indptr(srt.to(DEV), ptr2, 1, E, N, E)
    torch.cuda.synchronize()
    assert torch.equal(ptr2.cpu(), oracle.index_to_indptr(srt, N))
    back = torch.full((E,), -1, dtype=torch.long, device=DEV)
    capi.indptr_to_index(ptr2, back, 1, N, E, N + 1)
    torch.cuda.synchronize()
    assert torch.equal(back.cpu(), oracle.indptr_to_index(want_ptr)) and torch.equal(back.cpu(), srt)


@pytest.mark.parametrize("E,N,kind", [(1 << 20, 1000, "hub"), (3_000_001, 2_000_000, "random"),
                                      (2_000_000, 70_000, "gaps"), (1 << 21, 1, "random")])
def test_sort_large_against_numpy(capi, E, N, kind):
    rng = np.random.default_rng(N)
    index = make_index(kind, rng, E, N)
    perm, indptr = sort_on_gpu(capi, index, N)
    assert torch.equal(perm.cpu().long(), torch.from_numpy(np.argsort(index.numpy(), kind="stable")))
    want_ptr = np.zeros(N + 1, dtype=np.int64)
    want_ptr[1:] = np.cumsum(np.bincount(index.numpy(), minlength=N))
    assert torch.equal(indptr.cpu(), torch.from_numpy(want_ptr))
    # batched round trip of the formats: two batch rows that hold the same number of entries
    srt = np.sort(index.numpy())
    both = torch.from_numpy(np.stack([srt, np.sort((srt * 7 + 1) % N)])).to(DEV)
    ptr = torch.empty((2, N + 1), dtype=torch.long, device=DEV)
    capi.index_to_indptr(both, ptr, 2, E, N, E)
    back = torch.empty((2, E), dtype=torch.long, device=DEV)
    capi.indptr_to_index(ptr, back, 2, N, E, N + 1)
    torch.cuda.synchronize()
    assert torch.equal(back, both)
    assert torch.equal(ptr[0].cpu(), torch.from_numpy(want_ptr))


def test_sort_marks_entries_outside_the_range(capi):
    index = torch.tensor([3, -1, 0, 9, 2, 3, 4], dtype=torch.long)
    perm, indptr = sort_on_gpu(capi, index, 4)
    assert indptr.tolist() == [0, 1, 1, 2, 4]  # indptr[N] = 4 < E = 7
    assert perm.tolist()[:4] == [2, 4, 0, 5] and sorted(perm.tolist()[4:]) == [1, 3, 6]


SHAPES = [
    # B, E, K, N
    (1, 5000, 1, 300), (2, 3000, 4, 50), (1, 2000, 8, 100), (1, 1500, 3, 40), (1, 900, 64, 20),
    (1, 700, 130, 9), (3, 400, 16, 7), (1, 1, 1, 1), (1, 257, 2, 300), (1, 40000, 32, 1500),
]


@pytest.mark.parametrize("shape,kind,dtype", product(SHAPES, ["random", "hub", "gaps"], ALL_DTYPES))
def test_permuted_reduce_against_oracle_scatter(capi, oracle, shape, kind, dtype):
    B, E, K, N = shape
    rng = np.random.default_rng(E * 5 + K)
    index1 = make_index(kind, rng, E, N)
    perm, indptr = sort_on_gpu(capi, index1, N)
    index = index1.view(1, E, 1).expand(B, E, K)
    for reduce in ("sum", "mean", "min", "max"):
        small = dtype in (torch.int8, torch.uint8) and reduce in ("sum", "mean")
        src = random_values(rng, (B, E, K), dtype, ties=True)
        if small:  # keep 8-bit sums inside the type
            src = (src.abs() > 6).to(dtype)
            if kind != "random":  # more than 127 entries per slot: the reference's 8-bit count wraps
                continue
        want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
        if reduce == "mean":  # the division belongs to the op layer (floor division for integers)
            want = oracle.op_scatter(src, index1, 1, None, N, "mean")
        out = torch.empty((B, N, K), dtype=dtype, device=DEV)
        arg = torch.empty((B, N, K), dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
        code = capi.REDUCE[reduce]
        if reduce == "mean" and not dtype.is_floating_point:
            capi.segment_csr_permuted(src.to(DEV), perm, indptr, out, arg, B, N, E, K, 0, 0, capi.SUM)
            cnt = (indptr[1:] - indptr[:-1]).clamp(min=1).view(1, N, 1)
            out = torch.div(out, cnt, rounding_mode="floor").to(dtype)
        else:
            capi.segment_csr_permuted(src.to(DEV), perm, indptr, out, arg, B, N, E, K, 0, 0, code)
        torch.cuda.synchronize()
        if reduce in ("min", "max"):
            assert torch.equal(out.cpu(), want), reduce
            assert torch.equal(arg.cpu(), want_arg), reduce
        elif dtype.is_floating_point:
            scale = float(oracle.scatter(src.double().abs(), index, 1, None, N, "sum")[0].max())
            err = (out.cpu().double() - want.double()).abs()
            bound = RTOL[dtype] * want.double().abs() + RTOL[dtype] * scale
            assert bool((err <= bound).all()), (reduce, float((err - bound).max()))
        else:
            assert torch.equal(out.cpu(), want), reduce


def test_permuted_reduce_argument_checks(capi):
    import ctypes
    L = capi.lib()
    x = torch.zeros((8, 4), device=DEV)
    perm = torch.arange(8, dtype=torch.int32, device=DEV)
    ptr = torch.tensor([0, 8], device=DEV)
    out = torch.zeros((1, 4), device=DEV)
    ws = torch.empty(1, dtype=torch.uint8, device=DEV)
    args = (capi._p(x), capi._p(perm), capi._p(ptr), capi._p(out), None, capi._i(1), capi._i(1), capi._i(8), capi._i(4),
            capi._i(0), capi._i(0), capi.DTYPE[torch.float32])
    assert L.ts_segment_csr_permuted(*args, capi.MUL, capi._p(ws), ctypes.c_size_t(1), None) == 2  # unsupported
    assert L.ts_segment_csr_permuted(*args, capi.MAX, capi._p(ws), ctypes.c_size_t(1), None) == 1  # arg_out missing
    assert L.ts_segment_csr_permuted(*args, capi.SUM, None, ctypes.c_size_t(0), None) == 3         # workspace


# ------------------------------------------------------------------ operator level
@pytest.mark.parametrize("dim,reduce,dtype", product([0, 1, -1], ["sum", "mean", "min", "max"],
                                                     [torch.float32, torch.float64, torch.bfloat16, torch.int64]))
def test_scatter_sorted_matches_scatter(ts, dim, reduce, dtype):
    shape = (60, 50, 24)
    g = torch.Generator().manual_seed(13)
    d = dim if dim >= 0 else len(shape) + dim
    N = 11
    index = torch.randint(0, N - 1, (shape[d],), generator=g).to(DEV)  # slot N-1 stays empty
    src = torch.randint(-9, 10, shape, generator=g).to(dtype).to(DEV)
    plan = ts.SortedIndex(index, N)
    assert torch.equal(index[plan.perm.long()], plan.sorted_index())
    if reduce in ("min", "max"):
        out, arg = ts.scatter_sorted(src, plan, dim, reduce)
        want, want_arg = (ts.scatter_min if reduce == "min" else ts.scatter_max)(src, index, dim, None, N)
        assert torch.equal(out, want) and torch.equal(arg, want_arg)
    else:
        out = ts.scatter_sorted(src, plan, dim, reduce)
        want = ts.scatter(src, index, dim, None, N, reduce)
        assert torch.equal(out, want)  # small integers: every sum is exact in every type
    again = ts.scatter_sorted(src, plan, dim, reduce)
    assert torch.equal(out, again[0] if reduce in ("min", "max") else again)


@pytest.mark.parametrize("reduce", ["sum", "mean", "min", "max"])
def test_scatter_sorted_autograd(ts, reduce):
    g = torch.Generator().manual_seed(17)
    N = 40
    index = torch.randint(0, N, (500,), generator=g).to(DEV)
    x = torch.randn((3, 500, 6), generator=g, dtype=torch.double).to(DEV)
    grad = torch.randn((3, N, 6), generator=g, dtype=torch.double).to(DEV)
    plan = ts.SortedIndex(index, N)
    a = x.clone().requires_grad_(True)
    b = x.clone().requires_grad_(True)
    got = ts.scatter_sorted(a, plan, 1, reduce)
    want = ts.scatter(b, index, 1, None, N, reduce)
    got = got[0] if reduce in ("min", "max") else got
    got.backward(grad)
    want.backward(grad)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    assert torch.allclose(a.grad, b.grad, rtol=1e-12, atol=1e-12)


def test_scatter_sorted_is_bit_reproducible_and_close_to_scatter(ts):
    g = torch.Generator().manual_seed(19)
    E, N, K = 400_000, 5000, 32
    index = torch.randint(0, N, (E,), generator=g)
    index[: E // 3] = 7  # a hub
    index = index[torch.randperm(E, generator=g)].to(DEV)
    src = torch.randn((E, K), generator=g).to(DEV)
    plan = ts.SortedIndex(index, N)
    first = ts.scatter_sorted(src, plan, 0, "sum")
    for _ in range(3):
        assert torch.equal(first, ts.scatter_sorted(src, plan, 0, "sum"))
    want = ts.scatter_sum(src.double(), index, 0, None, N)
    scale = float(ts.scatter_sum(src.abs().double(), index, 0, None, N).max())
    assert float((first.double() - want).abs().max()) <= 1e-5 * scale


def test_formats_and_plan_operator_checks(ts):
    index = torch.tensor([0, 0, 2, 2, 2, 5], device=DEV)
    ptr = ts.index_to_indptr(index, 7)
    assert ptr.tolist() == [0, 2, 2, 5, 5, 5, 6, 6]
    assert torch.equal(ts.indptr_to_index(ptr), index)
    assert torch.equal(ts.indptr_to_index(ptr, 6), index)
    both = torch.stack([index, torch.tensor([1, 1, 1, 3, 6, 6], device=DEV)])
    ptr2 = ts.index_to_indptr(both, 7)
    assert ptr2.shape == (2, 8) and torch.equal(ts.indptr_to_index(ptr2), both)
    assert ts.indptr_to_index(torch.zeros(4, dtype=torch.long, device=DEV)).shape == (0,)
    with pytest.raises(RuntimeError, match="out of range"):
        ts.SortedIndex(torch.tensor([0, 3, 9], device=DEV), 5)
    with pytest.raises(ValueError):
        ts.SortedIndex(both)
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        ts.index_to_indptr(index.cpu(), 7)
    plan = ts.SortedIndex(index)
    assert plan.dim_size == 6
    with pytest.raises(ValueError):
        ts.scatter_sorted(torch.ones(6, device=DEV), plan, 0, "mul")
    with pytest.raises(RuntimeError, match="Input mismatch"):
        ts.scatter_sorted(torch.ones(5, device=DEV), plan, 0, "sum")
    # a plan over no entries
    empty = ts.SortedIndex(torch.zeros(0, dtype=torch.long, device=DEV), 3)
    assert ts.scatter_sorted(torch.ones((0, 2), device=DEV), empty, 0, "sum").tolist() == [[0, 0]] * 3


@pytest.mark.parametrize("K,dtype", [(4, torch.float32), (32, torch.float32), (2, torch.float64), (64, torch.bfloat16),
                                     (8, torch.int32)])
def test_hub_row_through_many_tiles(capi, oracle, K, dtype):
    """A row of 200 000 entries passes through about a hundred tiles: the walk over their partial results is
    shared by the workgroup that ends the row. Small-integer values: every sum is exact and ties are
    everywhere, so values and positions must match the oracle bit for bit, with and without a permutation."""
    rng = np.random.default_rng(K)
    N, E = 50, 300_000
    deg = np.full(N, (E - 200_000) // (N - 1), dtype=np.int64)
    deg[17] = 200_000
    deg[-1] += E - deg.sum()
    indptr = torch.zeros(N + 1, dtype=torch.long)
    indptr[1:] = torch.from_numpy(np.cumsum(deg))
    src = torch.from_numpy(rng.integers(-3, 4, size=(E, K)).astype(np.float64)).to(dtype)
    order = torch.from_numpy(rng.permutation(E))
    index = torch.repeat_interleave(torch.arange(N), torch.from_numpy(deg))
    shuffled_index = torch.empty(E, dtype=torch.long)
    shuffled_index[order] = index          # entry order[i] of the shuffled input is sorted entry i ...
    shuffled_src = torch.empty_like(src)
    shuffled_src[order] = src              # ... up to the order inside a row, which the stable sort fixes
    perm, ptr_d = sort_on_gpu(capi, shuffled_index, N)
    assert torch.equal(ptr_d.cpu(), indptr)
    for reduce in ("sum", "min", "max"):
        code = capi.REDUCE[reduce]
        want, want_arg = oracle.segment_csr(src, indptr, None, reduce)
        out = torch.empty((N, K), dtype=dtype, device=DEV)
        arg = torch.empty((N, K), dtype=torch.long, device=DEV) if reduce != "sum" else None
        capi.segment_csr(src.to(DEV), indptr.to(DEV), out, arg, 1, N, E, K, 0, code)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), want), reduce
        if arg is not None:
            assert torch.equal(arg.cpu(), want_arg), reduce
        want2, want_arg2 = oracle.scatter(shuffled_src.view(1, E, K), shuffled_index.view(1, E, 1).expand(1, E, K), 1,
                                          None, N, reduce)
        out2 = torch.empty((N, K), dtype=dtype, device=DEV)
        arg2 = torch.empty((N, K), dtype=torch.long, device=DEV) if reduce != "sum" else None
        capi.segment_csr_permuted(shuffled_src.to(DEV), perm, ptr_d, out2, arg2, 1, N, E, K, 0, 0, code)
        torch.cuda.synchronize()
        # sums against the segmented oracle: scatter's oracle adds 16-bit floats in the element type
        assert torch.equal(out2.cpu(), want if reduce == "sum" else want2[0]), reduce
        if arg2 is not None:
            assert torch.equal(arg2.cpu(), want_arg2[0]), reduce


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.int32, torch.uint8])
def test_permuted_minmax_with_a_large_output(capi, oracle, dtype):
    """From 8 M output elements on, the reduction writes the positions in src's order itself (no pass over
    arg_out afterwards), including scatter's rule for slots that never beat the initial value (uint8 zeros
    under max). Values and positions bit-exact against the oracle's scatter."""
    rng = np.random.default_rng(23)
    B, E, K, N = 1, 150_000, 128, 70_000
    index1 = make_index("gaps", rng, E, N)
    index1[: E // 5] = 31  # a row through many tiles
    index1 = index1[torch.from_numpy(rng.permutation(E))]
    perm, indptr = sort_on_gpu(capi, index1, N)
    src = random_values(rng, (B, E, K), dtype, ties=True)
    index = index1.view(1, E, 1).expand(B, E, K)
    for reduce in ("min", "max"):
        want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
        out = torch.empty((B, N, K), dtype=dtype, device=DEV)
        arg = torch.empty((B, N, K), dtype=torch.long, device=DEV)
        capi.segment_csr_permuted(src.to(DEV), perm, indptr, out, arg, B, N, E, K, 0, 0, capi.REDUCE[reduce])
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), want), reduce
        assert torch.equal(arg.cpu(), want_arg), reduce


def test_sorted_and_binned_scatter_under_graph_replay(ts, oracle, monkeypatch):
    """scatter_sorted (a hub row that the whole workgroup walks back over; carry flags in the workspace are
    cleared by their readers) and scatter_max with its workspace path, captured once and replayed three times
    with fresh inputs and eager work in between; every replay is checked."""
    monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    g = torch.Generator().manual_seed(29)
    E, N, K = 200_000, 300, 32
    index = torch.randint(0, N, (E,), generator=g)
    index[: E // 2] = 5  # 100 000 entries: about fifty tiles
    index = index[torch.randperm(E, generator=g)]
    d_index = index.to(DEV)
    plan = ts.SortedIndex(d_index, N)
    static_src = torch.zeros(E, K, device=DEV)
    for _ in range(2):  # warm-up outside the capture
        ts.scatter_sorted(static_src, plan, 0, "sum")
        ts.scatter_sorted(static_src, plan, 0, "max")
        ts.scatter_max(static_src, d_index, 0, None, N)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s_sum = ts.scatter_sorted(static_src, plan, 0, "sum")
        s_max, s_arg = ts.scatter_sorted(static_src, plan, 0, "max")
        b_max, b_arg = ts.scatter_max(static_src, d_index, 0, None, N)
    full = index.view(E, 1).expand(E, K)
    for rep in range(3):
        src = torch.randint(-20, 21, (E, K), generator=g).float()
        static_src.copy_(src.to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        want_sum = oracle.scatter(src, full, 0, None, N, "sum")[0]
        want_max, want_arg = oracle.scatter(src, full, 0, None, N, "max")
        assert torch.equal(s_sum.cpu(), want_sum), rep  # small integers: exact
        assert torch.equal(s_max.cpu(), want_max) and torch.equal(s_arg.cpu(), want_arg), rep
        assert torch.equal(b_max.cpu(), want_max) and torch.equal(b_arg.cpu(), want_arg), rep
        eager = ts.scatter_sorted(static_src, plan, 0, "sum")
        assert torch.equal(eager, s_sum)


def test_index_reuse_front_end(ts):
    """Off: scatter runs the atomic kernels. On: the first call with an index still does, the second sorts the
    index once and from then on scatter runs as a segmented reduction over permuted rows (bit-identical
    results call after call, positions equal to scatter_max's); an in-place change of the index, another
    dim_size, `out=`, narrow rows and a 2-D index are not taken from the cache."""
    from pytorch_scatter_amd import index_reuse
    g = torch.Generator().manual_seed(31)
    E, N, K = 50_000, 700, 32
    index = torch.randint(0, N, (E,), generator=g).to(DEV)
    src = torch.randint(-9, 10, (E, K), generator=g).float().to(DEV)
    assert not ts.index_reuse_enabled()
    base_sum = ts.scatter_sum(src, index, 0, None, N)
    base_max, base_arg = ts.scatter_max(src, index, 0, None, N)
    assert len(index_reuse._cache) == 0
    ts.enable_index_reuse(max_plans=3)
    try:
        first = ts.scatter_sum(src, index, 0, None, N)          # first sighting: remembered, no plan yet
        (entry,) = index_reuse._cache.values()
        assert entry[2] is None
        second = ts.scatter_sum(src, index, 0, None, N)         # second sighting: sorted once
        assert entry[2] is not None
        plan = entry[2]
        assert torch.equal(first, base_sum) and torch.equal(second, base_sum)  # small integers: exact sums
        got_max, got_arg = ts.scatter_max(src, index, 0, None, N)
        assert entry[2] is plan and torch.equal(got_max, base_max) and torch.equal(got_arg, base_arg)
        x = src.clone().requires_grad_(True)
        ts.scatter_mean(x, index, 0, None, N).sum().backward()
        y = src.clone().requires_grad_(True)
        torch.ops.torch_scatter.scatter_mean(y, index, 0, None, N).sum().backward()
        assert torch.allclose(x.grad, y.grad)
        # dim_size is part of the key; so is the version counter of the index
        assert ts.scatter_sum(src, index, 0, None, N + 5).shape[0] == N + 5
        assert len(index_reuse._cache) == 2
        index[0] = (index[0] + 1) % N
        moved = ts.scatter_sum(src, index, 0, None, N)
        assert torch.equal(moved, torch.ops.torch_scatter.scatter_sum(src, index, 0, None, N))
        assert torch.equal(ts.scatter_sum(src, index, 0, None, N), moved)  # plan of the changed index
        assert len(index_reuse._cache) == 3
        # not eligible: out given, rows under 64 bytes, an index of the shape of src
        before = len(index_reuse._cache)
        ts.scatter_sum(src, index, 0, torch.zeros(N, K, device=DEV))
        ts.scatter_sum(src[:, :4].contiguous(), index, 0, None, N)
        ts.scatter_sum(src, index.view(E, 1).expand(E, K), 0, None, N)
        assert len(index_reuse._cache) == before
        # least recently used out
        for i in range(4):
            ts.scatter_sum(src, torch.randint(0, N, (E,), generator=g).to(DEV), 0, None, N)
        assert len(index_reuse._cache) == 3
        # scripted wrappers keep going to the operator
        assert torch.equal(torch.jit.script(ts.scatter_sum)(src, index, 0, None, N), moved)
    finally:
        ts.disable_index_reuse()
    assert len(index_reuse._cache) == 0 and not ts.index_reuse_enabled()
