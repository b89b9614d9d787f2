"""Parity of the HIP kernels, called through the C ABI (libts_hip.so), against
the CPU oracle on the same seeded inputs.

Bars: bit-exact for min/max values, every arg index and every gather output;
for sum/mean |got - want| <= rtol * |want| + atol with rtol = 1e-5 (fp32) /
1e-2 (bf16, fp16), atol = rtol * max over rows of sum(|src|) (sums of N(0,1)
values cancel towards zero, so a purely relative bound is ill-posed).
"""
from itertools import product

import numpy as np
import pytest
import torch

from helpers import random_values

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
RTOL = {torch.float32: 1e-5, torch.float64: 1e-12, torch.bfloat16: 1e-2, torch.float16: 1e-2}


@pytest.fixture(scope="module")
def capi():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from pytorch_scatter_amd import capi
    capi.lib()
    return capi


def _bits(t):
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])


HALF_ULP = {torch.bfloat16: 2.0 ** -9, torch.float16: 2.0 ** -12}


def assert_sum16_no_worse_than_reference(oracle, out, src, index, index1, N, dim, exact, prev, what=""):
    """Accuracy of a 16-bit scatter sum, stated against the reference's own arithmetic. The reference adds entry
    by entry in the element type (csrc/cpu/scatter_cpu.cpp:74-76; atomicAdd on bf16 / half in scatter_cuda.cu:30-33):
    one rounding of the running total per entry. The kernels here add in fp32 inside a wavefront, a table or a
    bucket and round once per partial sum that leaves it, so a row meets at most as many roundings as it has
    entries, and a hub row far fewer. Checked two ways against the exact (fp64) sum:
      * in aggregate: the RMS error is not above that of the oracle run in the 16-bit type (the reference's
        arithmetic on the same input);
      * element by element: at most 4 * min(n, 100) half-ulp roundings of a running total of the size
        max(|exact|, sqrt(sum of squares)) (n: entries of the row), i.e. never more than 400 such units: twice the
        200 that the kernels reach on these inputs (the reference's own arithmetic reaches 480)."""
    dtype = src.dtype
    u = HALF_ULP[dtype]
    want = exact + (prev.double() if prev is not None else 0)
    ref16 = oracle.scatter(src, index, dim, prev.clone() if prev is not None else None,
                           None if prev is not None else N, "sum")[0].double()
    sq = oracle.scatter(src.double() ** 2, index, dim, None, N, "sum")[0]
    if prev is not None:
        sq = sq + prev.double() ** 2
    scale = torch.maximum(want.abs(), sq.sqrt())
    shape = [1] * want.dim()
    shape[dim] = N
    n_row = torch.bincount(index1, minlength=N).double().clamp(min=1, max=100).view(shape)
    err = (out.cpu().double() - want).abs()
    bound = u * 4 * n_row * scale + 1e-30
    assert bool((err <= bound).all()), (what, "element", float((err / bound).max()))
    rms, rms_ref = float(err.pow(2).mean().sqrt()), float((ref16 - want).abs().pow(2).mean().sqrt())
    assert rms <= 1.05 * rms_ref + u * float(scale.mean()), (what, "rms", rms, rms_ref)


def assert_exact(got, want, what=""):
    got = got.cpu()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if got.dtype.is_floating_point:
        # +0.0 / -0.0 carry different bits but are the same value under the reference's compares
        same = (_bits(got) == _bits(want)) | ((got == 0) & (want == 0))
        assert bool(same.all()), (what, int((~same).sum()))
    else:
        assert torch.equal(got, want), (what, int((got != want).sum()))


def assert_close(got, want, scale, dtype, what=""):
    got = got.cpu().double()
    want = want.double()
    rtol = RTOL[dtype]
    err = (got - want).abs()
    bound = rtol * want.abs() + rtol * scale
    assert bool((err <= bound).all()), (what, float((err - bound).max()))


def degrees(kind, rng, n):
    if kind == "short":
        d = rng.integers(0, 6, size=n)
    elif kind == "zipf":
        d = np.minimum(rng.zipf(1.8, size=n), 5000)
        d[rng.random(n) < 0.1] = 0
    elif kind == "hub":  # rows that span many tiles, next to empty rows at both ends
        d = rng.integers(0, 4, size=n)
        d[:3] = 0
        d[-3:] = 0
        d[n // 3] = 9000
        d[n // 2] = 2049
        d[n // 2 + 1] = 700
    elif kind == "uniform":
        d = np.full(n, 7)
    elif kind == "long":  # every row passes through dozens of tiles; two empty rows in between
        d = rng.integers(20000, 40000, size=n)
        d[n // 2] = 0
        d[n // 2 + 1] = 0
    else:
        raise ValueError(kind)
    return d.astype(np.int64)


def make_csr(kind, seed, n):
    rng = np.random.default_rng(seed)
    deg = degrees(kind, rng, n)
    indptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(deg, out=indptr[1:])
    index = np.repeat(np.arange(n, dtype=np.int64), deg)
    return rng, torch.from_numpy(indptr), torch.from_numpy(index)


def values(rng, shape, dtype, reduce):
    if reduce in ("min", "max") or not dtype.is_floating_point:
        return random_values(rng, shape, dtype, ties=True)
    return torch.from_numpy(rng.standard_normal(size=shape)).to(dtype)


CSR_CASES = [
    # kind, rows, K
    ("short", 300, 1), ("short", 1000, 4), ("zipf", 2000, 16), ("zipf", 3000, 64),
    ("hub", 900, 64), ("hub", 500, 128), ("uniform", 257, 3), ("zipf", 700, 200),
    ("hub", 300, 520), ("short", 5, 8), ("hub", 40, 1),
    ("long", 12, 8), ("long", 12, 64), ("long", 9, 1), ("hub", 120, 1100),
]


@pytest.mark.parametrize("case,reduce,dtype", product(
    CSR_CASES, ["sum", "mean", "min", "max"], [torch.float32, torch.bfloat16]))
def test_segment_csr(capi, oracle, case, reduce, dtype):
    kind, n, K = case
    rng, indptr, index = make_csr(kind, CSR_CASES.index(case), n)
    E = index.numel()
    src = values(rng, (E, K), dtype, reduce)
    want, want_arg = oracle.segment_csr(src, indptr, None, reduce)
    out = torch.full((n, K), 7, dtype=dtype, device=DEV)
    arg = torch.full((n, K), -1, dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
    capi.segment_csr(src.to(DEV), indptr.to(DEV), out, arg, 1, n, E, K, 0, capi.REDUCE[reduce])
    torch.cuda.synchronize()
    if reduce in ("min", "max"):
        assert_exact(out, want, "values")
        assert_exact(arg, want_arg, "arg")
    else:
        scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max()) if E else 0.0
        assert_close(out, want, scale, dtype, "values")


@pytest.mark.parametrize("case", [("long", 12, 64), ("hub", 900, 64), ("long", 9, 1), ("zipf", 3000, 64)])
def test_segment_csr_is_bit_reproducible(capi, case):
    """Rows that cross tiles are combined in an order fixed by the tiling (carries collected by the tile in
    which the row ends, or by the second kernel), never by arrival: repeated launches give identical bits."""
    kind, n, K = case
    rng, indptr, index = make_csr(kind, 31, n)
    E = index.numel()
    src = torch.from_numpy(rng.standard_normal(size=(E, K))).float().to(DEV)
    dptr = indptr.to(DEV)
    first = None
    for rep in range(6):
        out = torch.empty((n, K), device=DEV)
        capi.segment_csr(src, dptr, out, None, 1, n, E, K, 0, capi.SUM)
        torch.cuda.synchronize()
        if first is None:
            first = out.clone()
        assert torch.equal(_bits(out), _bits(first)), rep


@pytest.mark.parametrize("dtype,reduce", product(
    [torch.float16, torch.float64, torch.int32, torch.int64, torch.int16, torch.int8, torch.uint8],
    ["sum", "mean", "min", "max"]))
def test_segment_csr_other_dtypes(capi, oracle, dtype, reduce):
    rng, indptr, index = make_csr("hub", 5, 400)
    E = index.numel()
    K = 24
    src = random_values(rng, (E, K), dtype, ties=True)
    if reduce in ("sum", "mean") and dtype in (torch.int8, torch.uint8, torch.int16, torch.float16):
        src = src.clamp(-1, 1) if dtype != torch.uint8 else src.clamp(0, 1)
    if dtype == torch.uint8 and reduce == "mean":
        pytest.skip("8-bit counts wrap to 0 on long rows: undefined upstream")
    if dtype == torch.uint8 and reduce == "max":
        src = src + 1  # a row that never beats the initial value 0 keeps a stale arg upstream: unpinned
    want, want_arg = oracle.segment_csr(src, indptr, None, reduce)
    out = torch.zeros((400, K), dtype=dtype, device=DEV)
    arg = torch.zeros((400, K), dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
    capi.segment_csr(src.to(DEV), indptr.to(DEV), out, arg, 1, 400, E, K, 0, capi.REDUCE[reduce])
    torch.cuda.synchronize()
    if reduce in ("min", "max") or not dtype.is_floating_point:
        if dtype == torch.int8 and reduce == "mean":
            pytest.skip("8-bit counts wrap on long rows: undefined upstream")
        assert_exact(out, want, "values")
        if arg is not None:
            assert_exact(arg, want_arg, "arg")
    else:
        scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max())
        assert_close(out, want, scale, dtype)


NARROW_CASES = [
    # kind, rows, K: rows of at most 32 bytes take the LDS-staged kernel
    ("zipf", 3000, 1), ("zipf", 2500, 2), ("hub", 900, 3), ("hub", 700, 5), ("zipf", 2000, 8),
    ("uniform", 5000, 1), ("hub", 300, 8), ("short", 6000, 2), ("hub", 1200, 4),
]


@pytest.mark.parametrize("case,reduce,dtype", product(
    NARROW_CASES, ["sum", "mean", "min", "max"],
    [torch.float32, torch.bfloat16, torch.float64, torch.int32, torch.int8]))
def test_segment_csr_narrow_rows(capi, oracle, case, reduce, dtype):
    """Narrow rows, every element type width, with the entries starting at an address
    that is not 16-byte aligned (second pass) and long rows that cross many tiles."""
    kind, n, K = case
    rng, indptr, index = make_csr(kind, 100 + NARROW_CASES.index(case), n)
    E = index.numel()
    src = values(rng, (E, K), dtype, reduce)
    if dtype == torch.int8 and reduce in ("sum", "mean"):
        if kind != "short":
            pytest.skip("8-bit sums and counts wrap on long rows: undefined upstream")
        src = src.clamp(-1, 1)
    want, want_arg = oracle.segment_csr(src, indptr, None, reduce)
    for offset in (0, 1):
        flat = torch.empty(E * K + 8, dtype=dtype, device=DEV)
        dsrc = flat[offset:offset + E * K].view(E, K)
        dsrc.copy_(src)
        out = torch.full((n, K), 7, dtype=dtype, device=DEV)
        arg = torch.full((n, K), -1, dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
        capi.segment_csr(dsrc, indptr.to(DEV), out, arg, 1, n, E, K, 0, capi.REDUCE[reduce])
        torch.cuda.synchronize()
        if reduce in ("min", "max") or not dtype.is_floating_point:
            assert_exact(out, want, f"values offset={offset}")
            if arg is not None:
                assert_exact(arg, want_arg, f"arg offset={offset}")
        else:
            scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max()) if E else 0.0
            assert_close(out, want, scale, dtype, f"values offset={offset}")


@pytest.mark.parametrize("reduce,dtype", product(["sum", "max"], [torch.float32, torch.bfloat16]))
def test_segment_csr_wide_rows_unaligned(capi, oracle, reduce, dtype):
    """Buffers off the 16-byte grid take one element per lane, a different tile size and
    more partial results: the workspace size reported for the shape has to cover that plan too."""
    kind, n, K = "hub", 900, 64
    rng, indptr, index = make_csr(kind, 77, n)
    E = index.numel()
    src = values(rng, (E, K), dtype, reduce)
    want, want_arg = oracle.segment_csr(src, indptr, None, reduce)
    flat = torch.empty(E * K + 8, dtype=dtype, device=DEV)
    dsrc = flat[1:1 + E * K].view(E, K)
    dsrc.copy_(src)
    oflat = torch.full((n * K + 8,), 7, dtype=dtype, device=DEV)
    out = oflat[1:1 + n * K].view(n, K)
    arg = torch.full((n, K), -1, dtype=torch.long, device=DEV) if reduce == "max" else None
    capi.segment_csr(dsrc, indptr.to(DEV), out, arg, 1, n, E, K, 0, capi.REDUCE[reduce])
    torch.cuda.synchronize()
    if reduce == "max":
        assert_exact(out, want, "values")
        assert_exact(arg, want_arg, "arg")
    else:
        scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max())
        assert_close(out, want, scale, dtype, "values")
    assert bool((oflat[:1] == 7).all()) and bool((oflat[1 + n * K:] == 7).all())


@pytest.mark.parametrize("case,reduce", product(NARROW_CASES[:5], ["sum", "mean", "min", "max"]))
def test_segment_coo_narrow_rows(capi, oracle, case, reduce):
    kind, n, K = case
    rng, indptr, index = make_csr(kind, 200 + NARROW_CASES.index(case), n)
    E = index.numel()
    src = values(rng, (E, K), torch.float32, reduce)
    want, want2 = oracle.segment_coo(src, index, None, n, reduce)
    out = torch.full((n, K), 7, dtype=torch.float32, device=DEV)
    wa = reduce in ("min", "max")
    arg = torch.full((n, K), -1, dtype=torch.long, device=DEV) if wa else None
    count = torch.full((n,), -1, dtype=torch.float32, device=DEV) if reduce == "mean" else None
    capi.segment_coo(src.to(DEV), index.to(DEV), out, arg, count, 1, n, E, K, 0, capi.REDUCE[reduce], False)
    torch.cuda.synchronize()
    if wa:
        assert_exact(out, want)
        assert_exact(arg, want2, "arg")
    else:
        scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max()) if E else 0.0
        assert_close(out, want, scale, torch.float32)
        if reduce == "mean":
            assert_exact(count, want2, "count")


@pytest.mark.parametrize("reduce", ["sum", "mean", "min", "max"])
def test_segment_csr_batched(capi, oracle, reduce):
    rng = np.random.default_rng(21)
    B, n, K = 3, 50, 8
    E = 400
    ptrs = []
    for _ in range(B):
        deg = rng.multinomial(E, np.ones(n) / n)
        ptrs.append(np.concatenate([[0], np.cumsum(deg)]))
    indptr = torch.from_numpy(np.stack(ptrs).astype(np.int64))
    src = values(rng, (B, E, K), torch.float32, reduce)
    for ip, stride in ((indptr, n + 1), (indptr[:1], 0)):
        want, want_arg = oracle.segment_csr(src, ip, None, reduce)
        out = torch.empty((B, n, K), dtype=torch.float32, device=DEV)
        arg = torch.empty((B, n, K), dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
        capi.segment_csr(src.to(DEV), ip.contiguous().to(DEV), out, arg, B, n, E, K, stride, capi.REDUCE[reduce])
        torch.cuda.synchronize()
        if reduce in ("min", "max"):
            assert_exact(out, want)
            assert_exact(arg, want_arg)
        else:
            assert_close(out, want, float(src.abs().sum(1).max()), torch.float32)


@pytest.mark.parametrize("case,dtype", product(CSR_CASES, [torch.float32, torch.bfloat16, torch.int64, torch.uint8]))
def test_gather_csr(capi, oracle, case, dtype):
    kind, n, K = case
    rng, indptr, index = make_csr(kind, CSR_CASES.index(case), n)
    E = index.numel()
    src = random_values(rng, (n, K), dtype, ties=False)
    want = oracle.gather_csr(src, indptr)
    out = torch.full((E, K), 3, dtype=dtype, device=DEV)
    capi.gather_csr(src.to(DEV), indptr.to(DEV), out, 1, n, E, K, 0)
    torch.cuda.synchronize()
    assert_exact(out, want)


@pytest.mark.parametrize("case,dtype", product(CSR_CASES[:8], [torch.float32, torch.bfloat16, torch.float64]))
def test_segment_mean_csr_backward(capi, oracle, case, dtype):
    kind, n, K = case
    rng, indptr, index = make_csr(kind, CSR_CASES.index(case), n)
    E = index.numel()
    g = torch.from_numpy(rng.standard_normal(size=(n, K))).to(dtype)
    want = oracle.segment_mean_csr_backward(g, indptr, (E, K))
    out = torch.empty((E, K), dtype=dtype, device=DEV)
    capi.segment_mean_csr_backward(g.to(DEV), indptr.to(DEV), out, 1, n, E, K, 0)
    torch.cuda.synchronize()
    assert_exact(out, want)  # one correctly rounded division per element: bit-exact


@pytest.mark.parametrize("case,dtype", product(
    NARROW_CASES + [("zipf", 1500, 16), ("hub", 400, 12)],
    [torch.float32, torch.bfloat16, torch.float64, torch.int64, torch.uint8]))
def test_gather_csr_and_mean_backward_narrow_rows(capi, oracle, case, dtype):
    """Narrow rows take the one-lane-per-16-bytes kernel; also with `out` off the 16-byte grid
    and with a batch whose slices are not multiples of 16 bytes."""
    kind, n, K = case
    rng, indptr, index = make_csr(kind, 300 + n + K, n)
    E = index.numel()
    src = random_values(rng, (n, K), dtype, ties=False)
    want = oracle.gather_csr(src, indptr)
    for offset in (0, 1):
        flat = torch.full((E * K + 8,), 3, dtype=dtype, device=DEV)
        out = flat[offset:offset + E * K].view(E, K)
        capi.gather_csr(src.to(DEV), indptr.to(DEV), out, 1, n, E, K, 0)
        torch.cuda.synchronize()
        assert_exact(out, want, f"offset={offset}")
        assert bool((flat[:offset] == 3).all()) and bool((flat[offset + E * K:] == 3).all())
    B = 3
    srcb = random_values(rng, (B, n, K), dtype, ties=False)
    wantb = oracle.gather_csr(srcb, indptr.view(1, -1).expand(B, -1))
    outb = torch.full((B, E, K), 3, dtype=dtype, device=DEV)
    capi.gather_csr(srcb.to(DEV), indptr.to(DEV), outb, B, n, E, K, 0)
    torch.cuda.synchronize()
    assert_exact(outb, wantb, "batched")
    if dtype.is_floating_point:
        g = torch.from_numpy(rng.standard_normal(size=(n, K))).to(dtype)
        wantg = oracle.segment_mean_csr_backward(g, indptr, (E, K))
        outg = torch.empty((E, K), dtype=dtype, device=DEV)
        capi.segment_mean_csr_backward(g.to(DEV), indptr.to(DEV), outg, 1, n, E, K, 0)
        torch.cuda.synchronize()
        assert_exact(outg, wantg, "mean backward")


@pytest.mark.parametrize("case,reduce,dtype", product(
    CSR_CASES[:9] + CSR_CASES[11:14], ["sum", "mean", "min", "max"], [torch.float32, torch.bfloat16]))
def test_segment_coo(capi, oracle, case, reduce, dtype):
    kind, n, K = case
    rng, indptr, index = make_csr(kind, CSR_CASES.index(case), n)
    E = index.numel()
    src = values(rng, (E, K), dtype, reduce)
    want, want2 = oracle.segment_coo(src, index, None, n, reduce)
    out = torch.full((n, K), 7, dtype=dtype, device=DEV)
    arg = torch.full((n, K), -1, dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
    cnt = torch.full((n,), -1, dtype=dtype, device=DEV) if reduce == "mean" else None
    capi.segment_coo(src.to(DEV), index.to(DEV), out, arg, cnt, 1, n, E, K, 0, capi.REDUCE[reduce], False)
    torch.cuda.synchronize()
    if reduce in ("min", "max"):
        assert_exact(out, want)
        assert_exact(arg, want2)
    else:
        scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max()) if E else 0.0
        assert_close(out, want, scale, dtype)
        if reduce == "mean":
            assert_exact(cnt, want2)


@pytest.mark.parametrize("K,E,reduce,dtype", [
    (16, 400_000, "sum", torch.float32), (16, 400_000, "max", torch.float32), (16, 400_000, "mean", torch.float32),
    (1, 2_400_000, "sum", torch.float32), (1, 2_400_000, "min", torch.float32), (4, 700_000, "max", torch.float32),
    (16, 600_000, "max", torch.bfloat16), (3, 900_000, "sum", torch.int32), (2, 1_300_000, "max", torch.int64)])
def test_segment_csr_one_row_through_hundreds_of_tiles(capi, oracle, K, E, reduce, dtype):
    """Narrow rows, one segment that holds nearly all entries and so passes through more than 512 tiles of the
    first kernel: its chain of partial results is combined by all wavefronts of a workgroup of the second kernel.
    A few short segments either side of it, and a second long one behind it that stays with one wavefront."""
    rng = np.random.default_rng(K + E)
    deg = np.concatenate([rng.integers(0, 5, size=40), [E], rng.integers(0, 5, size=30), [E // 40],
                          rng.integers(0, 3, size=20)])
    n = deg.size
    indptr = torch.from_numpy(np.concatenate([[0], np.cumsum(deg)]).astype(np.int64))
    total = int(indptr[-1])
    src = values(rng, (total, K), dtype, reduce)
    want, want2 = oracle.segment_csr(src, indptr, None, reduce)
    out = torch.full((n, K), 7, dtype=dtype, device=DEV)
    arg = torch.full((n, K), -1, dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
    capi.segment_csr(src.to(DEV), indptr.to(DEV), out, arg, 1, n, total, K, 0, capi.REDUCE[reduce])
    torch.cuda.synchronize()
    if reduce in ("min", "max") or not dtype.is_floating_point:
        assert_exact(out, want)
        if arg is not None:
            assert_exact(arg, want2)
    else:
        scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max())
        assert_close(out, want, scale, dtype)


GAP_KINDS = ["one_row", "empty_tail", "empty_head", "two_hubs", "every_3000th"]


def gap_index(kind, rng, E, N):
    """Sorted indices that leave long ranges of output rows without entries."""
    if kind == "one_row":
        return np.full(E, N // 2)
    if kind == "empty_tail":
        return np.sort(rng.integers(0, max(N // 100, 1), size=E))
    if kind == "empty_head":
        return np.sort(rng.integers(N - max(N // 100, 1), N, size=E))
    if kind == "two_hubs":
        return np.sort(np.where(rng.random(E) < 0.5, 17, N - 9))
    return np.sort(rng.integers(0, N // 3000 + 1, size=E) * 3000 % N)


@pytest.mark.parametrize("kind,shape,reduce", product(
    GAP_KINDS, [(1, 5000, 3, 50_000), (2, 700, 8, 9000), (1, 300, 1, 300_000), (3, 9, 2, 70_000)], ["sum", "max"]))
def test_segment_coo_long_ranges_of_empty_rows(capi, oracle, kind, shape, reduce):
    """Row pointers of a sorted index whose entries leave thousands of neighbouring rows empty: the rows between
    two entries are written by the lane that owns the later entry when they are few, by its wavefront or
    workgroup when they are many (gap_rows in device_utils.h). Results as the oracle's, batches included."""
    B, E, K, N = shape
    rng = np.random.default_rng(E + N)
    idx = np.stack([gap_index(kind, rng, E, N) for _ in range(B)])
    index = torch.from_numpy(idx)
    src = values(rng, (B, E, K), torch.float32, reduce)
    want, want2 = oracle.segment_coo(src, index, None, N, reduce)
    out = torch.full((B, N, K), 7, dtype=torch.float32, device=DEV)
    arg = torch.full((B, N, K), -1, dtype=torch.long, device=DEV) if reduce == "max" else None
    capi.segment_coo(src.to(DEV), index.to(DEV), out, arg, None, B, N, E, K, E, capi.REDUCE[reduce], False)
    torch.cuda.synchronize()
    if reduce == "max":
        assert_exact(out, want)
        assert_exact(arg, want2)
    else:
        assert torch.allclose(out.cpu(), want, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("kind", GAP_KINDS)
def test_sort_index_long_ranges_of_empty_rows(capi, kind):
    """The row pointers that ts_sort_index writes next to its permutation, for indices that leave long ranges of
    rows empty: ptr[r] = number of entries below row r."""
    E, N = 6000, 200_000
    rng = np.random.default_rng(5)
    idx = rng.permutation(gap_index(kind, rng, E, N))
    perm = torch.empty(E, dtype=torch.int32, device=DEV)
    ptr = torch.full((N + 1,), -5, dtype=torch.long, device=DEV)
    capi.sort_index(torch.from_numpy(idx).to(DEV), perm, ptr, E, N)
    torch.cuda.synchronize()
    want = np.concatenate([[0], np.cumsum(np.bincount(idx, minlength=N))])
    assert np.array_equal(ptr.cpu().numpy(), want)
    assert np.array_equal(np.sort(idx, kind="stable"), idx[perm.cpu().numpy()])


@pytest.mark.parametrize("reduce,dtype,K", product(["sum", "mean", "min", "max"], [torch.float32, torch.bfloat16],
                                                   [16, 2]))
def test_segment_coo_out_given(capi, oracle, reduce, dtype, K):
    kind, n = "hub", 500
    rng, indptr, index = make_csr(kind, 33, n)
    E = index.numel()
    src = values(rng, (E, K), dtype, reduce)
    prev = random_values(rng, (n, K), dtype, ties=True)
    prev[0] = 1  # the oracle seeds the first run from row 0: keep both readings equal
    deg = indptr[1:] - indptr[:-1]
    first = int(index[0])
    prev[first] = prev[0]
    want = prev.clone()
    oracle.segment_coo(src, index, want, None, reduce)
    out = prev.clone().to(DEV)
    arg = torch.full((n, K), E, dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
    capi.segment_coo(src.to(DEV), index.to(DEV), out, arg, None, 1, n, E, K, 0, capi.REDUCE[reduce], True)
    torch.cuda.synchronize()
    if reduce in ("min", "max"):
        assert_exact(out, want)
        # arg: E where the previous content survived, else first position of the winner
        a = arg.cpu()
        kept = (out.cpu() == prev) & (a == E)
        won = a < E
        assert bool((kept | won).all())
        picked = torch.gather(src, 0, a.clamp(max=E - 1))
        assert torch.equal(picked[won], out.cpu()[won])
    else:
        scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max()) + float(prev.abs().max())
        assert_close(out, want, scale, dtype)
    # rows without entries keep their content
    assert_exact(out[(deg == 0).to(DEV)], prev[deg == 0])


@pytest.mark.parametrize("case,dtype", product(CSR_CASES[:9], [torch.float32, torch.bfloat16, torch.int32]))
def test_gather_coo_and_mean_backward(capi, oracle, case, dtype):
    kind, n, K = case
    rng, indptr, index = make_csr(kind, CSR_CASES.index(case), n)
    E = index.numel()
    if E == 0:
        pytest.skip("empty")
    src = random_values(rng, (n, K), dtype, ties=False)
    want = oracle.gather_coo(src, index)
    out = torch.empty((E, K), dtype=dtype, device=DEV)
    capi.gather_coo(src.to(DEV), index.to(DEV), out, 1, n, E, K, 0)
    torch.cuda.synchronize()
    assert_exact(out, want)
    if dtype.is_floating_point:
        count = (indptr[1:] - indptr[:-1]).clamp(min=1).to(dtype)
        want = oracle.segment_mean_coo_backward(src, index, count, (E, K))
        capi.segment_mean_coo_backward(src.to(DEV), index.to(DEV), count.to(DEV), out, 1, n, E, K, 0)
        torch.cuda.synchronize()
        assert_exact(out, want)


@pytest.mark.parametrize("K,dtype,B", product(
    [1, 3, 5, 7, 17, 33, 47, 129], [torch.float32, torch.bfloat16, torch.float64, torch.int8], [1, 3]))
def test_gather_coo_odd_widths(capi, oracle, K, dtype, B):
    """Row widths that are no multiple of 16 bytes take the flat kernel (a lane owns 16 consecutive bytes
    of out that may span several edges); batches whose slices leave the 16-byte grid, and out / src
    buffers off that grid, take its one-element-per-lane form. Bit-exact, and nothing outside out is touched."""
    n, E = 300, 2511
    rng = np.random.default_rng(K * 7 + B)
    index = torch.from_numpy(np.sort(rng.integers(0, n, size=(B, E)), axis=1))
    src = random_values(rng, (B, n, K), dtype, ties=False)
    want = torch.stack([oracle.gather_coo(src[b], index[b]) for b in range(B)])
    for off in (0, 1):
        sflat = torch.zeros(B * n * K + 8, dtype=dtype, device=DEV)
        dsrc = sflat[off:off + B * n * K].view(B, n, K)
        dsrc.copy_(src)
        oflat = torch.full((B * E * K + 8,), 7, dtype=dtype, device=DEV)
        out = oflat[off:off + B * E * K].view(B, E, K)
        capi.gather_coo(dsrc, index.to(DEV), out, B, n, E, K, E)
        torch.cuda.synchronize()
        assert_exact(out, want, f"off={off}")
        assert bool((oflat[:off] == 7).all()) and bool((oflat[off + B * E * K:] == 7).all())
        if dtype.is_floating_point:
            count = torch.stack([torch.bincount(index[b], minlength=n) for b in range(B)]).clamp(min=1).to(dtype)
            want_b = torch.stack([oracle.segment_mean_coo_backward(src[b], index[b], count[b], (E, K)) for b in range(B)])
            capi.segment_mean_coo_backward(dsrc, index.to(DEV), count.to(DEV), out, B, n, E, K, E)
            torch.cuda.synchronize()
            assert_exact(out, want_b, f"mean backward off={off}")


SCATTER_SHAPES = [
    # B, E, K, N
    (1, 1000, 1, 37), (1, 5000, 16, 300), (1, 3000, 32, 10), (2, 700, 5, 50), (3, 400, 8, 1),
    (1, 20000, 4, 2000), (1, 64, 130, 7),
]


@pytest.mark.parametrize("shape,reduce,dtype", product(
    SCATTER_SHAPES, ["sum", "mul", "min", "max"], [torch.float32, torch.bfloat16, torch.int32]))
def test_scatter(capi, oracle, shape, reduce, dtype):
    B, E, K, N = shape
    rng = np.random.default_rng(B * 1000 + E + K)
    src = values(rng, (B, E, K), dtype, reduce)
    if reduce == "mul":
        src = random_values(rng, (B, E, K), dtype, ties=True).clamp(-1, 1)
        if dtype.is_floating_point:
            src = torch.where(src == 0, torch.ones_like(src), src)
    index1 = torch.from_numpy(rng.integers(0, N, size=E))
    for mode in ("broadcast", "full"):
        if mode == "broadcast":
            index = index1.view(1, E, 1).expand(B, E, K)
            strides = (0, 1, 0)
            dev_index = index1.to(DEV)
        else:
            index = torch.from_numpy(rng.integers(0, N, size=(B, E, K)))
            strides = (E * K, K, 1)
            dev_index = index.to(DEV)
        want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
        out = torch.full((B, N, K), 9, dtype=dtype, device=DEV)
        arg = torch.full((B, N, K), -5, dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
        capi.scatter(src.to(DEV), dev_index, out, arg, B, E, K, N, *strides, capi.REDUCE[reduce], False)
        torch.cuda.synchronize()
        if reduce in ("min", "max") or not dtype.is_floating_point or reduce == "mul":
            assert_exact(out, want, mode)
            if arg is not None:
                assert_exact(arg, want_arg, mode + " arg")
        else:
            absum = oracle.scatter(src.abs().double(), index, 1, None, N, "sum")[0]
            if dtype == torch.float32:
                assert_close(out, want, float(absum.max()), dtype, mode)
            else:
                # bf16 atomics round after every add, in arrival order: compare with the exact sum
                exact = oracle.scatter(src.double(), index, 1, None, N, "sum")[0]
                err = (out.cpu().double() - exact).abs()
                cnt = oracle.scatter(torch.ones(B, E, K, dtype=torch.double), index, 1, None, N, "sum")[0]
                assert bool((err <= 2.0 ** -8 * cnt * absum.clamp(min=1e-30) + 1e-30).all()), mode


@pytest.mark.parametrize("shape,reduce,dtype", product(
    [(1, 30000, 1, 500), (1, 9000, 32, 300), (2, 5000, 8, 40), (1, 4000, 12, 70000)],
    ["min", "max"], [torch.float32, torch.bfloat16, torch.int32, torch.int64, torch.float64]))
def test_scatter_minmax_lds_cached_variant(capi, oracle, shape, reduce, dtype, monkeypatch):
    """The workgroup-private table variant (forced on, with a small chunk so that
    several workgroups meet on the same slots), skewed index with heavy ties. 64-bit types: the table of keys
    in front of their compare-and-swap pass."""
    monkeypatch.setenv("TS_SCATTER_LDS", "2")
    monkeypatch.setenv("TS_SCATTER_EPB", "700")
    B, E, K, N = shape
    rng = np.random.default_rng(E + K)
    src = random_values(rng, (B, E, K), dtype, ties=True)
    if dtype == torch.float64:  # the values that the keys fold or skip
        flat = src.view(-1)
        flat[::97] = float("nan")
        flat[5::89] = -0.0
        flat[7::83] = float("-inf")
        flat[11::79] = float("inf")
    elif dtype == torch.int64:  # the ends of the range map to the keys that stand for "no entry"
        flat = src.view(-1)
        flat[::97] = torch.iinfo(torch.int64).min
        flat[5::89] = torch.iinfo(torch.int64).max
    p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
    index1 = torch.from_numpy(rng.choice(N, size=E, p=p / p.sum()))
    index = index1.view(1, E, 1).expand(B, E, K)
    for out_given in (False, True):
        if out_given:
            prev = random_values(rng, (B, N, K), dtype, ties=True)
            want = prev.clone()
            _, want_arg = oracle.scatter(src, index, 1, want, None, reduce)
            out = prev.clone().to(DEV)
        else:
            want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
            out = torch.empty((B, N, K), dtype=dtype, device=DEV)
        arg = torch.empty((B, N, K), dtype=torch.long, device=DEV)
        capi.scatter(src.to(DEV), index1.to(DEV), out, arg, B, E, K, N, 0, 1, 0, capi.REDUCE[reduce], out_given)
        torch.cuda.synchronize()
        assert_exact(out, want)
        assert_exact(arg, want_arg)


@pytest.mark.parametrize("shape,reduce,dtype", list(product(
    [(1, 60000, 32, 300), (2, 40000, 16, 700), (1, 50000, 128, 90), (1, 30000, 24, 5000), (1, 20000, 64, 100000),
     (3, 9000, 512, 5), (1, 70000, 17, 40),
     (2, 30000, 64, 40000),   # 625 buckets over two batch rows: the place pass that sorts its tile in LDS
     (1, 8000, 1024, 50), (2, 5000, 768, 33)],   # rows wider than a table row: reduced in slices of columns
    ["min", "max"], [torch.float32, torch.bfloat16, torch.int32, torch.int8]))
    + [((1, 20000, 64, 600000), "max", torch.float32), ((1, 20000, 64, 600000), "min", torch.int32),  # 4688 buckets
       ((1, 20000, 128, 540000), "max", torch.float32),  # 8438 buckets
       # too many buckets of whole rows (16 875): four slices of 128 columns, 4219 buckets
       ((1, 20000, 512, 270000), "max", torch.float32), ((1, 20000, 512, 270000), "min", torch.bfloat16)])
def test_scatter_minmax_binned_variant(capi, oracle, shape, reduce, dtype, monkeypatch):
    """min / max with a workspace: entries binned by bucket of output rows and reduced in LDS (forced on at
    these sizes), skewed index with heavy ties, with and without previous content in out. Rows under 64 bytes
    (int8 at K < 64, ...) keep the path without workspace."""
    monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    B, E, K, N = shape
    rng = np.random.default_rng(E + K)
    src = random_values(rng, (B, E, K), dtype, ties=True)
    p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
    idx = rng.choice(N, size=E, p=p / p.sum())
    index1 = torch.from_numpy(idx)
    index = index1.view(1, E, 1).expand(B, E, K)
    for out_given in (False, True):
        if out_given:
            prev = random_values(rng, (B, N, K), dtype, ties=True)
            want = prev.clone()
            _, want_arg = oracle.scatter(src, index, 1, want, None, reduce)
            out = prev.clone().to(DEV)
        else:
            want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
            out = torch.empty((B, N, K), dtype=dtype, device=DEV)
        arg = torch.empty((B, N, K), dtype=torch.long, device=DEV)
        capi.scatter_with_workspace(src.to(DEV), index1.to(DEV), out, arg, B, E, K, N, 0, 1, 0, capi.REDUCE[reduce],
                                    out_given)
        torch.cuda.synchronize()
        assert_exact(out, want)
        assert_exact(arg, want_arg)
    L = capi.lib()
    need = L.ts_scatter_workspace_bytes(capi._i(B), capi._i(E), capi._i(K), capi._i(N), capi.DTYPE[dtype],
                                        capi.REDUCE[reduce])
    assert (need > 0) == (K * src.element_size() >= 64)
    assert L.ts_scatter_workspace_bytes(capi._i(B), capi._i(E), capi._i(K), capi._i(N), capi.DTYPE[dtype], capi.MUL) == 0


@pytest.mark.parametrize("shape,kind,reduce,dtype", product(
    [(1, 60000, 8, 3000), (2, 40000, 4, 700), (1, 50000, 32, 9000), (1, 9000, 64, 1000), (1, 30000, 6, 500),
     (3, 9000, 16, 50000)],
    ["zipf", "uniform", "sorted zipf", "hub in sorted"], ["min", "max"],
    [torch.float32, torch.bfloat16, torch.int32, torch.uint8]))
def test_scatter_minmax_skew_probe(capi, oracle, shape, kind, reduce, dtype, monkeypatch):
    """min / max with 256 bytes of workspace and few entries per output row: a sample of the index picks the
    table kernel (skewed, unsorted index) or the run kernel (uniform or sorted index); forced on at these sizes.
    Both must give the oracle's values and arg indices, with and without previous content in out."""
    monkeypatch.setenv("TS_SCATTER_SKEW", "2")
    B, E, K, N = shape
    rng = np.random.default_rng(E + K)
    src = random_values(rng, (B, E, K), dtype, ties=True)
    if kind == "uniform":
        idx = rng.integers(0, N, size=E)
    else:
        p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
        idx = rng.choice(N, size=E, p=p / p.sum())
        if kind == "sorted zipf":
            idx = np.sort(idx)
        elif kind == "hub in sorted":
            idx = np.sort(rng.integers(0, N, size=E))
            idx[rng.random(E) < 0.4] = N // 3
    index1 = torch.from_numpy(idx)
    index = index1.view(1, E, 1).expand(B, E, K)
    L = capi.lib()
    need = L.ts_scatter_workspace_bytes(capi._i(B), capi._i(E), capi._i(K), capi._i(N), capi.DTYPE[dtype],
                                        capi.REDUCE[reduce])
    assert need == (256 if src.element_size() == 4 else 0)   # 4-byte elements only
    for out_given in (False, True):
        if out_given:
            prev = random_values(rng, (B, N, K), dtype, ties=True)
            want = prev.clone()
            _, want_arg = oracle.scatter(src, index, 1, want, None, reduce)
            out = prev.clone().to(DEV)
        else:
            want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
            out = torch.empty((B, N, K), dtype=dtype, device=DEV)
        arg = torch.empty((B, N, K), dtype=torch.long, device=DEV)
        ws = capi.scatter_with_workspace(src.to(DEV), index1.to(DEV), out, arg, B, E, K, N, 0, 1, 0,
                                         capi.REDUCE[reduce], out_given)
        torch.cuda.synchronize()
        assert_exact(out, want)
        assert_exact(arg, want_arg)
        if need == 0:
            continue
        # the probe's decision, restated: 1024 evenly spaced entries, repeats of an output row and descents
        pos = np.arange(1024, dtype=np.int64) * ((B * E) // 1024)
        b, e = pos // E, pos % E
        dup = 1024 - np.unique(b * N + idx[e]).size
        desc = int(np.sum(((pos + 1) // E == b) & (idx[(pos + 1) % E] < idx[e])))
        flag = int(ws[:4].view(torch.int32).item())
        if not (220 < dup < 290 or 12 < desc < 20):   # away from the thresholds (256 repeats, 16 descents)
            assert flag == int(dup >= 256 and desc >= 16), (kind, dup, desc, flag)
    if need:
        assert flag == {"sorted zipf": 0, "zipf": 1}.get(kind, flag)


@pytest.mark.parametrize("shape,kind,dtype", list(product(
    [(1, 60000, 32, 300), (2, 40000, 16, 700), (1, 50000, 128, 90), (1, 20000, 64, 100000), (3, 9000, 256, 5),
     (1, 30000, 24, 500), (2, 30000, 64, 40000),
     (1, 8000, 1024, 50), (2, 5000, 96, 330)],   # reduced in slices of columns (96: no power of two of lanes)
    ["zipf", "sorted", "one descent"],
    [torch.float32, torch.float64, torch.bfloat16, torch.float16, torch.int32, torch.int64, torch.int16]))
    + [((1, 20000, 64, 600000), "zipf", torch.float32), ((1, 20000, 64, 600000), "one descent", torch.int32),  # 4688 buckets
       ((1, 20000, 128, 540000), "zipf", torch.int32),  # 8438 buckets
       ((1, 20000, 512, 270000), "zipf", torch.float32)])  # four slices of 128 columns, 4219 buckets
def test_scatter_sum_binned_variant(capi, oracle, shape, kind, dtype, monkeypatch):
    """Sum with a workspace (forced on at these sizes): a sample of the index (or, with the sample switched
    off as in the "one descent" cases, the count pass) finds out whether the index is sorted;
    if not, the entries are binned by bucket of output rows and added in LDS (double slots for floating
    types), else the usual kernels run. Exact for integers (int16 and K = 24 keep the path without
    workspace), within tolerance of the exact sum for floats, with and without previous content in out."""
    monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    if kind == "one descent":
        monkeypatch.setenv("TS_BIN_NO_SAMPLE", "1")
    B, E, K, N = shape
    rng = np.random.default_rng(E + K + len(kind))
    p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
    idx = rng.choice(N, size=E, p=p / p.sum())
    if kind != "zipf":
        idx = np.sort(idx)
    if kind == "one descent":
        idx[E // 2] = N - 1
        idx[E // 2 + 1] = 0
    index1 = torch.from_numpy(idx)
    index = index1.view(1, E, 1).expand(B, E, K)
    if dtype.is_floating_point:
        src = torch.from_numpy(rng.standard_normal(size=(B, E, K))).to(dtype)
    else:
        src = torch.from_numpy(rng.integers(-20, 20, size=(B, E, K))).to(dtype)
    for out_given in (False, True):
        prev = (torch.from_numpy(rng.standard_normal(size=(B, N, K))).to(dtype) if dtype.is_floating_point
                else torch.from_numpy(rng.integers(-20, 20, size=(B, N, K))).to(dtype))
        out = prev.clone().to(DEV) if out_given else torch.full((B, N, K), 9, dtype=dtype, device=DEV)
        capi.scatter_with_workspace(src.to(DEV), index1.to(DEV), out, None, B, E, K, N, 0, 1, 0, capi.SUM, out_given)
        torch.cuda.synchronize()
        if not dtype.is_floating_point:
            want = oracle.scatter(src, index, 1, prev.clone() if out_given else None, None if out_given else N,
                                  "sum")[0]
            assert_exact(out, want, f"{kind} out_given={out_given}")
            continue
        exact = oracle.scatter(src.double(), index, 1, None, N, "sum")[0]
        if dtype in (torch.bfloat16, torch.float16):
            assert_sum16_no_worse_than_reference(oracle, out, src, index, index1, N, 1, exact,
                                                 prev if out_given else None, f"{kind} out_given={out_given}")
            continue
        absum = oracle.scatter(src.double().abs(), index, 1, None, N, "sum")[0]
        want = exact + (prev.double() if out_given else 0)
        rtol = RTOL[dtype]
        err = (out.cpu().double() - want).abs()
        bound = rtol * want.abs() + rtol * (absum + (prev.double().abs() if out_given else 0)).clamp(min=1e-30)
        assert bool((err <= bound).all()), (kind, out_given, float((err - bound).max()))


SORTED_KINDS = ["sorted", "sorted gaps", "one descent", "beyond N", "negative first", "empty tail", "one row"]


@pytest.mark.parametrize("shape,reduce,kind,dtype", list(product(
    [(1, 60000, 32, 300), (2, 40000, 16, 700), (1, 20000, 64, 100000), (1, 8000, 1024, 50), (3, 9000, 512, 5)],
    ["sum", "min", "max"], SORTED_KINDS, [torch.float32, torch.bfloat16, torch.int32])))
def test_scatter_sorted_index_with_workspace(capi, oracle, shape, reduce, kind, dtype, monkeypatch):
    """With a workspace, the count pass of the buckets (forced on at these sizes) checks the whole index; one that
    is in order and inside [0, N) is finished by the segmented reduction (row pointers from the index, one pass
    over src, no atomics), anything else by the buckets. Both must give scatter's result: values that never beat
    the initial value of the element type (-inf, lowest()) leave 0 with position E, empty rows too; a single
    descent, an index beyond N at the end or a negative one in front sends the call down the other path."""
    monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    B, E, K, N = shape
    rng = np.random.default_rng(E + K + len(kind))
    src = random_values(rng, (B, E, K), dtype, ties=True)
    if dtype.is_floating_point:
        src[:, ::7, ::3] = float("-inf") if reduce == "max" else float("inf")
        src[:, 5::11, 1::2] = torch.finfo(dtype).min if reduce == "max" else torch.finfo(dtype).max
    elif reduce != "sum":
        src[:, ::7, ::3] = torch.iinfo(dtype).min if reduce == "max" else torch.iinfo(dtype).max
    if reduce == "sum" and dtype.is_floating_point:
        src = torch.from_numpy(rng.standard_normal(size=(B, E, K))).to(dtype)
    idx = np.sort(rng.integers(0, N, size=E))
    if kind == "sorted gaps":
        idx = np.sort(rng.choice(np.arange(0, N, 3), size=E))
    if kind == "one descent":
        idx[E // 2], idx[E // 2 + 1] = N - 1, 0
    if kind == "empty tail":  # long ranges of rows without entries: written by a wavefront or the workgroup
        idx = np.sort(rng.integers(0, max(N // 100, 1), size=E))
    if kind == "one row":
        idx = np.full(E, N // 2)
    if kind == "beyond N":
        idx[-3:] = N + 5
    if kind == "negative first":
        idx[:2] = -1
    index1 = torch.from_numpy(idx)
    valid = (index1 >= 0) & (index1 < N)
    # scatter drops entries whose index lies outside [0, N); positions stay those of the full input
    safe = torch.where(valid, index1, torch.zeros_like(index1))
    index = safe.view(1, E, 1).expand(B, E, K)
    if reduce == "sum":
        src_ok = torch.where(valid.view(1, E, 1), src, torch.zeros_like(src))
        out = torch.full((B, N, K), 9, dtype=dtype, device=DEV)
        capi.scatter_with_workspace(src.to(DEV), index1.to(DEV), out, None, B, E, K, N, 0, 1, 0, capi.SUM, 0)
        torch.cuda.synchronize()
        if not dtype.is_floating_point:
            assert_exact(out, oracle.scatter(src_ok, index, 1, None, N, "sum")[0], kind)
            return
        exact = oracle.scatter(src_ok.double(), index, 1, None, N, "sum")[0]
        absum = oracle.scatter(src_ok.double().abs(), index, 1, None, N, "sum")[0]
        if dtype == torch.bfloat16:
            assert_sum16_no_worse_than_reference(oracle, out, src_ok, index, safe, N, 1, exact, None, kind)
        else:
            err = (out.cpu().double() - exact).abs()
            assert bool((err <= RTOL[dtype] * (exact.abs() + absum) + 1e-30).all()), kind
        return
    # min / max: an entry outside [0, N) must not win, so give it the value that never does
    lose = (torch.finfo(dtype).min if reduce == "max" else torch.finfo(dtype).max) if dtype.is_floating_point else \
        (torch.iinfo(dtype).min if reduce == "max" else torch.iinfo(dtype).max)
    src_ok = torch.where(valid.view(1, E, 1), src, torch.full_like(src, lose))
    want, want_arg = oracle.scatter(src_ok, index, 1, None, N, reduce)
    out = torch.empty((B, N, K), dtype=dtype, device=DEV)
    arg = torch.empty((B, N, K), dtype=torch.long, device=DEV)
    capi.scatter_with_workspace(src.to(DEV), index1.to(DEV), out, arg, B, E, K, N, 0, 1, 0, capi.REDUCE[reduce], 0)
    torch.cuda.synchronize()
    assert_exact(out, want, kind)
    assert_exact(arg, want_arg, kind + " arg")


@pytest.mark.parametrize("reduce,dtype", product(["sum", "max"], [torch.float32, torch.float64, torch.int32]))
def test_scatter_sorted_index_per_batch_rows(capi, oracle, reduce, dtype, monkeypatch):
    """A batched index [B, E] whose rows are sorted one by one (different rows per batch, stride E): in order as a
    whole for the count pass of the buckets, row pointers per batch for the segmented reduction. The second batch
    row of the last case has one descent: the whole call then goes through the buckets."""
    monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    B, E, K, N = 3, 30000, 32, 900
    rng = np.random.default_rng(K + len(reduce))
    for descent in (False, True):
        idx = np.sort(rng.integers(0, N, size=(B, E)), axis=1)
        if descent:
            idx[1, E // 3], idx[1, E // 3 + 1] = N - 1, 0
        index2 = torch.from_numpy(idx)
        index = index2.view(B, E, 1).expand(B, E, K)
        if dtype.is_floating_point and reduce == "sum":
            src = torch.from_numpy(rng.standard_normal(size=(B, E, K))).to(dtype)
        else:
            src = random_values(rng, (B, E, K), dtype, ties=True)
        out = torch.full((B, N, K), 9, dtype=dtype, device=DEV)
        arg = torch.empty((B, N, K), dtype=torch.long, device=DEV) if reduce == "max" else None
        if dtype == torch.float64 and reduce == "max":
            continue  # 64-bit elements keep the two-pass kernels (no packed keys, no workspace)
        capi.scatter_with_workspace(src.to(DEV), index2.to(DEV), out, arg, B, E, K, N, E, 1, 0, capi.REDUCE[reduce], 0)
        torch.cuda.synchronize()
        want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
        if reduce == "max":
            assert_exact(out, want, f"descent={descent}")
            assert_exact(arg, want_arg, f"descent={descent} arg")
        elif not dtype.is_floating_point:
            assert_exact(out, want, f"descent={descent}")
        else:
            exact = oracle.scatter(src.double(), index, 1, None, N, "sum")[0]
            absum = oracle.scatter(src.double().abs(), index, 1, None, N, "sum")[0]
            err = (out.cpu().double() - exact).abs()
            assert bool((err <= RTOL[dtype] * (exact.abs() + absum) + 1e-30).all()), descent


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_scatter_with_workspace_agrees_with_plain_scatter_on_random_shapes(capi, seed, monkeypatch):
    """Forty random calls per seed (1-3 batches, 4-1024 columns, 1 - 1.2 M output rows, seven element types, uniform /
    Zipf / sorted / sorted with entries outside [0, N) / one descent / three distinct values, with and without a
    given out), buckets forced on: min / max with a workspace (buckets, column slices, slabs, the segmented
    reduction for a sorted index) give the bits of the call without workspace; floating sums stay within
    4 * min(n, 128) half-ulp roundings of the exact sum."""
    monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    rng = np.random.default_rng(seed)
    dtypes = [torch.float32, torch.bfloat16, torch.float16, torch.int32, torch.int16, torch.int8, torch.uint8]
    for case in range(40):
        dtype = dtypes[rng.integers(len(dtypes))]
        reduce = ["sum", "min", "max"][rng.integers(3)]
        B = int(rng.choice([1, 1, 1, 2, 3]))
        K = int(rng.choice([4, 8, 16, 24, 32, 48, 64, 96, 128, 256, 384, 512, 1024]))
        E = int(rng.integers(1, 60000))
        N = int(rng.choice([1, 7, 300, 5000, 70000, 300000, 1200000]))
        N = min(N, max(int(3e8 // (B * K)), 1))
        E = min(E, max(int(3e8 // (B * K)), 1))
        kind = ["uniform", "zipf", "sorted", "sorted-oor", "one-descent", "few-values"][rng.integers(6)]
        if kind == "zipf":
            idx = np.minimum(rng.zipf(1.3, size=E) - 1, N - 1)
        elif kind == "few-values":
            idx = rng.integers(0, min(N, 3), size=E)
        else:
            idx = rng.integers(0, N, size=E)
        if kind.startswith("sorted") or kind == "one-descent":
            idx = np.sort(idx)
        if kind == "sorted-oor" and E > 3:
            idx[-2:] = N + 3
            idx[0] = -5
        if kind == "one-descent" and E > 4:
            idx[E // 2], idx[E // 2 + 1] = N - 1, 0
        index = torch.from_numpy(idx.astype(np.int64)).to(DEV)
        what = (case, dtype, reduce, B, E, K, N, kind)
        if dtype.is_floating_point and reduce == "sum":
            src = torch.from_numpy(rng.standard_normal(size=(B, E, K))).to(dtype).to(DEV)
        else:
            v = rng.integers(-8, 9, size=(B, E, K))
            src = torch.from_numpy(np.abs(v) if dtype == torch.uint8 else v).to(dtype).to(DEV)
            if dtype.is_floating_point:
                src[:, ::5, ::3] = float("-inf") if reduce == "max" else float("inf")
        out_given = bool(rng.integers(2)) and reduce != "sum"
        prev = torch.from_numpy(rng.integers(-3, 4, size=(B, N, K))).to(dtype).to(DEV) if out_given else None
        res = []
        for fn in (capi.scatter, capi.scatter_with_workspace):
            out = prev.clone() if out_given else torch.full((B, N, K), 9, dtype=dtype, device=DEV)
            arg = torch.full((B, N, K), -7, dtype=torch.long, device=DEV) if reduce != "sum" else None
            fn(src, index, out, arg, B, E, K, N, 0, 1, 0, capi.REDUCE[reduce], out_given)
            torch.cuda.synchronize()
            res.append((out, arg))
        (o0, a0), (o1, a1) = res
        if reduce == "sum" and dtype.is_floating_point:
            valid = (index >= 0) & (index < N)
            vi = index[valid]
            exact = torch.zeros((B, N, K), dtype=torch.double, device=DEV).index_add_(1, vi, src[:, valid].double())
            sq = torch.zeros((B, N, K), dtype=torch.double, device=DEV).index_add_(1, vi, src[:, valid].double() ** 2)
            n_row = torch.bincount(vi, minlength=N).double().clamp(min=1, max=128).view(1, N, 1)
            u = {torch.float32: 2.0 ** -24, torch.bfloat16: 2.0 ** -9, torch.float16: 2.0 ** -12}[dtype]
            bound = u * 4 * n_row * torch.maximum(exact.abs(), sq.sqrt()) + 1e-30
            assert bool(((o1.double() - exact).abs() <= bound).all()), what
        else:
            assert torch.equal(o0, o1), what
            assert a0 is None or torch.equal(a0, a1), what


@pytest.mark.parametrize("shape,dtype", product(
    [(1, 30000, 1, 500), (1, 9000, 32, 300), (2, 5000, 8, 40), (1, 4000, 12, 70000)],
    [torch.float32, torch.bfloat16, torch.float16]))
def test_scatter_sum_lds_aggregated_variant(capi, oracle, shape, dtype, monkeypatch):
    """Sum through the workgroup-private accumulator table (forced on), skewed index;
    also the count entry point, which shares the kernel."""
    monkeypatch.setenv("TS_SCATTER_LDS", "2")
    monkeypatch.setenv("TS_SCATTER_EPB", "700")
    B, E, K, N = shape
    rng = np.random.default_rng(E + K)
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K))).to(dtype)
    p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
    index1 = torch.from_numpy(rng.choice(N, size=E, p=p / p.sum()))
    index = index1.view(1, E, 1).expand(B, E, K)
    exact = oracle.scatter(src.double(), index, 1, None, N, "sum")[0]
    absum = oracle.scatter(src.double().abs(), index, 1, None, N, "sum")[0]
    for out_given in (False, True):
        prev = torch.from_numpy(rng.standard_normal(size=(B, N, K))).to(dtype)
        out = prev.clone().to(DEV) if out_given else torch.empty((B, N, K), dtype=dtype, device=DEV)
        capi.scatter(src.to(DEV), index1.to(DEV), out, None, B, E, K, N, 0, 1, 0, capi.SUM, out_given)
        torch.cuda.synchronize()
        want = exact + (prev.double() if out_given else 0)
        rtol = 1e-5 if dtype == torch.float32 else 1e-2
        err = (out.cpu().double() - want).abs()
        bound = rtol * want.abs() + rtol * (absum + (prev.double().abs() if out_given else 0)).clamp(min=1e-30)
        assert bool((err <= bound).all()), float((err - bound).max())
    cnt = torch.empty((N,), dtype=torch.int32, device=DEV)
    capi.scatter_count(index1.to(DEV), cnt, 1, E, N, 0, 1)
    torch.cuda.synchronize()
    assert torch.equal(cnt.cpu(), torch.bincount(index1, minlength=N).int())


@pytest.mark.parametrize("shape,kind,dtype", product(
    [(1, 300000, 8, 40000), (1, 400000, 1, 90000), (2, 140000, 4, 9000), (1, 270000, 12, 30000),
     (1, 1_100_000, 8, 40000), (2, 1_060_000, 4, 90000), (1, 300_000, 32, 50000),
     # small inputs, in chunks of 64 entries and up: 2^17 elements and more, rows above 64 columns from 2^20
     (1, 140_000, 1, 5000), (1, 20_000, 7, 3000), (2, 5000, 16, 700), (1, 4200, 32, 100_000), (1, 2100, 64, 50),
     (3, 1500, 33, 40), (1, 9000, 128, 2000), (1, 1100, 128, 10), (1, 8300, 100, 300)],
    ["sorted", "shuffled", "zipf"], [torch.float32, torch.bfloat16]))
def test_scatter_sum_narrow_rows_sample_picks_the_kernel(capi, oracle, shape, kind, dtype):
    """Sums at sizes that the accumulator table takes: from 2^23 elements, with 256 bytes of workspace, a sample of
    the index sends a sorted index to the run kernel instead (word 0 of the workspace: 0) and any other to the table
    (1). Either way, and at the sizes below, the sum is the oracle's, with and without previous content in out."""
    B, E, K, N = shape
    if K >= 32 and dtype != torch.float32 and E < 32 * N:
        pytest.skip("wide rows of 2-byte elements only take the table under a contended index")
    rng = np.random.default_rng(E + K)
    src = torch.from_numpy(rng.standard_normal(size=(B, E, K))).to(dtype)
    if kind == "zipf":
        p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
        idx = rng.choice(N, size=E, p=p / p.sum())
    else:
        idx = rng.integers(0, N, size=E)
        if kind == "sorted":
            idx = np.sort(idx)
    index1 = torch.from_numpy(idx)
    index = index1.view(1, E, 1).expand(B, E, K)
    L = capi.lib()
    need = L.ts_scatter_workspace_bytes(capi._i(B), capi._i(E), capi._i(K), capi._i(N), capi.DTYPE[dtype], capi.SUM)
    # (rows of up to four floats from 2^21 entries: the value buckets, with scratch for the binned records)
    value_buckets = dtype == torch.float32 and K <= 4 and B * E >= (1 << 21 if K <= 2 else 3 << 20 if K == 3 else 1 << 22)
    by_sample = not value_buckets and B * E * K >= (1 << 23) and (K < 32 or dtype == torch.float32)
    if value_buckets:
        assert need >= 4 * B * E * (K + 1)
    else:
        assert need == (256 if by_sample else need) and need in (0, 256)
    exact = oracle.scatter(src.double(), index, 1, None, N, "sum")[0]
    absum = oracle.scatter(src.double().abs(), index, 1, None, N, "sum")[0]
    for out_given in (False, True):
        prev = torch.from_numpy(rng.standard_normal(size=(B, N, K))).to(dtype)
        out = prev.clone().to(DEV) if out_given else torch.empty((B, N, K), dtype=dtype, device=DEV)
        ws = capi.scatter_with_workspace(src.to(DEV), index1.to(DEV), out, None, B, E, K, N, 0, 1, 0, capi.SUM,
                                         out_given)
        torch.cuda.synchronize()
        if by_sample:
            assert int(ws[:4].view(torch.int32).item()) == (0 if kind == "sorted" else 1), kind
        want = exact + (prev.double() if out_given else 0)
        # bf16: every add into out rounds to 8 bits, as the reference's atomicAdd does (60 adds at magnitude 16 were
        # seen at 0.95e-2 of this bound's scale)
        rtol = 1e-5 if dtype == torch.float32 else 2e-2
        err = (out.cpu().double() - want).abs()
        bound = rtol * want.abs() + rtol * (absum + (prev.double().abs() if out_given else 0)).clamp(min=1e-30)
        assert bool((err <= bound).all()), float((err - bound).max())
        plain = prev.clone().to(DEV) if out_given else torch.empty((B, N, K), dtype=dtype, device=DEV)
        capi.scatter(src.to(DEV), index1.to(DEV), plain, None, B, E, K, N, 0, 1, 0, capi.SUM, out_given)
        torch.cuda.synchronize()
        perr = (plain.cpu().double() - want).abs()
        assert bool((perr <= bound).all()), "without workspace"


RUN_SHAPES = [
    # B, E, K, N
    (1, 5000, 1, 600), (1, 3000, 2, 40), (1, 2000, 3, 300), (2, 1500, 5, 64), (1, 4000, 16, 500),
    (1, 1500, 17, 100), (1, 1200, 64, 90), (1, 700, 100, 50), (1, 300, 130, 9), (3, 900, 8, 2),
]


def run_index(kind, rng, E, N):
    """Indices with runs of equal neighbours, as a message-passing index has them."""
    idx = np.sort(rng.integers(0, N, size=E))
    if kind == "sorted":
        return idx
    if kind == "hub":  # one node owns the middle third
        idx[E // 3: 2 * E // 3] = idx[E // 3]
        return idx
    # runs kept, order of the runs shuffled: a node shows up in several separate runs
    cuts = np.sort(rng.choice(np.arange(1, E), size=min(E - 1, 40), replace=False))
    pieces = np.split(idx, cuts)
    rng.shuffle(pieces)
    return np.concatenate(pieces)


@pytest.mark.parametrize("shape,kind,dtype", product(
    RUN_SHAPES, ["sorted", "hub", "pieces"],
    [torch.int32, torch.int64, torch.float32, torch.float64, torch.bfloat16, torch.float16,
     torch.int16, torch.int8, torch.uint8]))
def test_scatter_sum_runs_of_equal_indices(capi, oracle, shape, kind, dtype):
    """Sum with the wavefront pre-reduction of neighbouring equal indices: exact for
    integers, within tolerance of the exact sum for floats; count shares the kernel."""
    B, E, K, N = shape
    rng = np.random.default_rng(E * 7 + K)
    if dtype.is_floating_point:
        src = torch.from_numpy(rng.standard_normal(size=(B, E, K))).to(dtype)
    else:
        src = torch.from_numpy(rng.integers(-1000, 1000, size=(B, E, K))).to(dtype)
    index1 = torch.from_numpy(run_index(kind, rng, E, N))
    index = index1.view(1, E, 1).expand(B, E, K)
    for out_given in (False, True):
        if dtype.is_floating_point:
            prev = torch.from_numpy(rng.standard_normal(size=(B, N, K))).to(dtype)
        else:
            prev = torch.from_numpy(rng.integers(-1000, 1000, size=(B, N, K))).to(dtype)
        out = prev.clone().to(DEV) if out_given else torch.full((B, N, K), 9, dtype=dtype, device=DEV)
        capi.scatter(src.to(DEV), index1.to(DEV), out, None, B, E, K, N, 0, 1, 0, capi.SUM, out_given)
        torch.cuda.synchronize()
        if not dtype.is_floating_point:
            want = prev.clone() if out_given else None
            want = oracle.scatter(src, index, 1, want, None if out_given else N, "sum")[0]
            assert_exact(out, want, f"{kind} out_given={out_given}")
        else:
            exact = oracle.scatter(src.double(), index, 1, None, N, "sum")[0]
            absum = oracle.scatter(src.double().abs(), index, 1, None, N, "sum")[0]
            want = exact + (prev.double() if out_given else 0)
            rtol = RTOL[dtype]
            err = (out.cpu().double() - want).abs()
            bound = rtol * want.abs() + rtol * (absum + (prev.double().abs() if out_given else 0)).clamp(min=1e-30)
            if dtype in (torch.bfloat16, torch.float16) and K % 2 == 1:
                # odd rows of 16-bit floats take the plain kernel: element-type atomics that round after
                # every add (as the reference's do), so the error grows with the entries per slot
                cnt = oracle.scatter(torch.ones(B, E, K, dtype=torch.double), index, 1, None, N, "sum")[0]
                bound = bound + 2.0 ** -8 * cnt * absum
            assert bool((err <= bound).all()), (kind, out_given, float((err - bound).max()))
    cnt = torch.empty((N,), dtype=torch.int32, device=DEV)
    capi.scatter_count(index1.to(DEV), cnt, 1, E, N, 0, 1)
    torch.cuda.synchronize()
    assert torch.equal(cnt.cpu(), torch.bincount(index1, minlength=N).int())


@pytest.mark.parametrize("shape,kind,reduce,dtype", product(
    RUN_SHAPES, ["sorted", "hub", "pieces"], ["min", "max"],
    [torch.float32, torch.bfloat16, torch.float16, torch.int32, torch.uint8]))
def test_scatter_minmax_runs_of_equal_indices(capi, oracle, shape, kind, reduce, dtype):
    """min / max + arg with the wavefront pre-reduction of neighbouring equal indices,
    heavy ties (the first position has to win), with and without a given out."""
    B, E, K, N = shape
    rng = np.random.default_rng(E * 11 + K)
    src = random_values(rng, (B, E, K), dtype, ties=True)
    if dtype == torch.uint8:
        src = src.clamp(min=1) if reduce == "max" else src.clamp(max=254)  # stay off the initial value
    index1 = torch.from_numpy(run_index(kind, rng, E, N))
    index = index1.view(1, E, 1).expand(B, E, K)
    for out_given in (False, True):
        if out_given:
            prev = random_values(rng, (B, N, K), dtype, ties=True)
            want = prev.clone()
            _, want_arg = oracle.scatter(src, index, 1, want, None, reduce)
            out = prev.clone().to(DEV)
        else:
            want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
            out = torch.empty((B, N, K), dtype=dtype, device=DEV)
        arg = torch.empty((B, N, K), dtype=torch.long, device=DEV)
        capi.scatter(src.to(DEV), index1.to(DEV), out, arg, B, E, K, N, 0, 1, 0, capi.REDUCE[reduce], out_given)
        torch.cuda.synchronize()
        assert_exact(out, want, f"{kind} out_given={out_given}")
        assert_exact(arg, want_arg, f"{kind} out_given={out_given} arg")


HOT_INDEX_KINDS = ["hub", "zipf", "sorted_hub", "uniform"]


def hot_index(kind, rng, E, N):
    """Indices of more than 2^18 entries (the size from which the sum kernels keep their LDS table of
    hot rows): a hub that owns a fifth of the entries, a Zipf law, hub entries sprinkled over a
    sorted index, and a uniform index (no row gets confirmed)."""
    if kind == "zipf":
        return np.minimum(rng.zipf(1.3, size=E) - 1, N - 1)
    idx = rng.integers(0, N, size=E)
    if kind == "uniform":
        return idx
    if kind == "sorted_hub":
        idx = np.sort(idx)
    idx[rng.random(E) < 0.2] = N // 3
    return idx


@pytest.mark.parametrize("K,kind,dtype", product(
    [1, 3, 8, 64, 100], HOT_INDEX_KINDS,
    [torch.float32, torch.float64, torch.bfloat16, torch.float16, torch.int32, torch.int64]))
def test_scatter_sum_hot_rows(capi, oracle, K, kind, dtype):
    """Sum with the workgroup table of hot rows in play: exact for integers, within tolerance of
    the exact sum for floats, with and without a given out; count shares the kernel."""
    E = 300_000 if K <= 8 else 270_000
    N = 5000
    rng = np.random.default_rng(K * 101 + len(kind))
    index1 = torch.from_numpy(hot_index(kind, rng, E, N))
    index = index1.view(E, 1).expand(E, K)
    if dtype.is_floating_point:
        src = torch.from_numpy(rng.standard_normal(size=(E, K))).to(dtype)
    else:
        src = torch.from_numpy(rng.integers(-1000, 1000, size=(E, K))).to(dtype)
    for out_given in (False, True):
        prev = (torch.from_numpy(rng.standard_normal(size=(N, K))).to(dtype) if dtype.is_floating_point
                else torch.from_numpy(rng.integers(-1000, 1000, size=(N, K))).to(dtype))
        out = prev.clone().to(DEV) if out_given else torch.full((N, K), 9, dtype=dtype, device=DEV)
        capi.scatter(src.to(DEV), index1.to(DEV), out, None, 1, E, K, N, 0, 1, 0, capi.SUM, out_given)
        torch.cuda.synchronize()
        if not dtype.is_floating_point:
            want = oracle.scatter(src, index, 0, prev.clone() if out_given else None, None if out_given else N,
                                  "sum")[0]
            assert_exact(out, want, f"{kind} out_given={out_given}")
            continue
        exact = oracle.scatter(src.double(), index, 0, None, N, "sum")[0]
        if dtype in (torch.bfloat16, torch.float16):
            assert_sum16_no_worse_than_reference(oracle, out, src, index, index1, N, 0, exact,
                                                 prev if out_given else None, f"{kind} out_given={out_given}")
            continue
        absum = oracle.scatter(src.double().abs(), index, 0, None, N, "sum")[0]
        want = exact + (prev.double() if out_given else 0)
        rtol = RTOL[dtype]
        err = (out.cpu().double() - want).abs()
        bound = rtol * want.abs() + rtol * (absum + (prev.double().abs() if out_given else 0)).clamp(min=1e-30)
        assert bool((err <= bound).all()), (kind, out_given, float((err - bound).max()))
    cnt = torch.empty((N,), dtype=torch.int32, device=DEV)
    capi.scatter_count(index1.to(DEV), cnt, 1, E, N, 0, 1)
    torch.cuda.synchronize()
    assert torch.equal(cnt.cpu(), torch.bincount(index1, minlength=N).int())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_scatter_sum_single_16bit_columns_leave_neighbours_alone(capi, dtype):
    """Rows of one 16-bit column are added with a packed-pair atomic whose other half is +0.0: the
    neighbouring elements of a given out keep their bits (denormals, infinities, NaN; -0.0 may turn
    into +0.0), also when out starts or ends in the middle of a 32-bit word."""
    N = 64
    specials = torch.tensor([1e-40, -1e-40, float("inf"), float("-inf"), float("nan"), -0.0, 0.0, 1.5, 6e-8, -6e-8])
    for offset in (0, 1):
        buf = torch.zeros(N + 2, dtype=dtype)
        buf[:] = specials.to(dtype).repeat(7)[:N + 2]
        prev = buf[offset:offset + N].clone()
        dbuf = buf.to(DEV)
        out = dbuf[offset:offset + N]
        touched = torch.tensor([7, 8, 21, N - 1, 0])  # values 1.5 or zeros at those positions? set them
        prev_touched = prev.clone()
        src = torch.ones(len(touched), dtype=dtype)
        capi.scatter(src.to(DEV), touched.to(DEV), out, None, 1, len(touched), 1, N, 0, 1, 0, capi.SUM, True)
        torch.cuda.synchronize()
        got = dbuf.cpu()
        mask = torch.ones(N + 2, dtype=torch.bool)
        mask[touched + offset] = False
        a, b = _bits(got)[mask], _bits(buf)[mask]
        same = (a == b) | ((got[mask] == 0) & (buf[mask] == 0))
        assert bool(same.all()), (offset, got[mask][~same], buf[mask][~same])
        want = (prev_touched[touched].float() + 1).to(dtype)
        ok = (got[touched + offset] == want) | (want != want)
        assert bool(ok.all()), (offset, got[touched + offset], want)


def test_scatter_sum_plain_atomic_kernel_still_covered(capi, oracle, monkeypatch):
    """The one-atomic-per-element kernel (used for per-element indices) with a shared index."""
    monkeypatch.setenv("TS_SCATTER_RUNS", "0")
    B, E, K, N = 2, 3000, 6, 50
    rng = np.random.default_rng(5)
    src = torch.from_numpy(rng.integers(-1000, 1000, size=(B, E, K))).to(torch.int32)
    index1 = torch.from_numpy(np.sort(rng.integers(0, N, size=E)))
    want = oracle.scatter(src, index1.view(1, E, 1).expand(B, E, K), 1, None, N, "sum")[0]
    out = torch.empty((B, N, K), dtype=torch.int32, device=DEV)
    capi.scatter(src.to(DEV), index1.to(DEV), out, None, B, E, K, N, 0, 1, 0, capi.SUM, False)
    cnt = torch.empty((N,), dtype=torch.int32, device=DEV)
    capi.scatter_count(index1.to(DEV), cnt, 1, E, N, 0, 1)
    torch.cuda.synchronize()
    assert_exact(out, want)
    assert torch.equal(cnt.cpu(), torch.bincount(index1, minlength=N).int())


@pytest.mark.parametrize("reduce,dtype", product(["sum", "min", "max"], [torch.float32, torch.float64, torch.int64]))
def test_scatter_out_given_and_wide_types(capi, oracle, reduce, dtype):
    B, E, K, N = 2, 3000, 6, 40
    rng = np.random.default_rng(77)
    src = random_values(rng, (B, E, K), dtype, ties=True)
    index = torch.from_numpy(rng.integers(0, N - 3, size=(B, E, K)))
    prev = random_values(rng, (B, N, K), dtype, ties=True) * 0 + (6 if reduce == "min" else -6 if reduce == "max" else 1)
    prev[:, :5] = 100 if reduce == "max" else -100 if reduce == "min" else 2  # previous content that survives
    want = prev.clone()
    _, want_arg = oracle.scatter(src, index, 1, want, None, reduce)
    out = prev.clone().to(DEV)
    arg = torch.full((B, N, K), -5, dtype=torch.long, device=DEV) if reduce != "sum" else None
    capi.scatter(src.to(DEV), index.to(DEV), out, arg, B, E, K, N, E * K, K, 1, capi.REDUCE[reduce], True)
    torch.cuda.synchronize()
    assert_exact(out, want)
    if arg is not None:
        assert_exact(arg, want_arg)
    # fresh output with the same inputs
    want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
    out = torch.empty((B, N, K), dtype=dtype, device=DEV)
    capi.scatter(src.to(DEV), index.to(DEV), out, arg, B, E, K, N, E * K, K, 1, capi.REDUCE[reduce], False)
    torch.cuda.synchronize()
    assert_exact(out, want)
    if arg is not None:
        assert_exact(arg, want_arg)


def test_scatter_mean_pieces(capi, oracle):
    B, E, K, N = 2, 2000, 8, 64
    rng = np.random.default_rng(5)
    for dtype in (torch.float32, torch.int32):
        src = random_values(rng, (B, E, K), dtype, ties=True)
        index1 = torch.from_numpy(rng.integers(0, N - 2, size=E))
        want = oracle.op_scatter(src, index1, 1, None, N, "mean")
        out = torch.empty((B, N, K), dtype=dtype, device=DEV)
        cnt = torch.empty((N,), dtype=torch.int32, device=DEV)
        capi.scatter(src.to(DEV), index1.to(DEV), out, None, B, E, K, N, 0, 1, 0, capi.SUM, False)
        capi.scatter_count(index1.to(DEV), cnt, 1, E, N, 0, 1)
        for b in range(B):
            capi.divide_by_count(out[b], cnt, 1, N, K)
        torch.cuda.synchronize()
        if dtype == torch.int32:
            assert_exact(out, want)
        else:
            assert_close(out, want, 8.0 * E / N * 4, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float64])
def test_arg_backward(capi, oracle, dtype):
    rng, indptr, index = make_csr("zipf", 3, 500)
    E = index.numel()
    K = 12
    src = random_values(rng, (E, K), torch.float32, ties=True)
    _, arg = oracle.segment_csr(src, indptr, None, "max")
    g = torch.from_numpy(rng.standard_normal(size=(500, K))).to(dtype)
    want = oracle.arg_backward(g, arg, (E, K), 0)
    out = torch.full((E, K), 5, dtype=dtype, device=DEV)
    capi.arg_backward(g.to(DEV), arg.to(DEV), out, 1, 500, E, K)
    torch.cuda.synchronize()
    assert_exact(out, want)


def test_error_codes(capi):
    x = torch.zeros(4, 4, device=DEV)
    ptr = torch.tensor([0, 2, 4], device=DEV)
    with pytest.raises(capi.TsError, match="workspace"):
        with torch.cuda.device(0):
            rc = capi.lib().ts_segment_csr(capi._p(x), capi._p(ptr), capi._p(x), None, capi._i(1), capi._i(2),
                                           capi._i(4), capi._i(4), capi._i(0), 0, capi.SUM, None, 0, None)
            capi._check(rc)
    with pytest.raises(capi.TsError, match="unsupported"):
        capi.segment_csr(x, ptr, x, None, 1, 2, 4, 4, 0, capi.MUL)
    with pytest.raises(capi.TsError, match="device"):
        capi.gather_csr(x.cpu(), ptr, x, 1, 2, 4, 4, 0)


# ---- row pointers that do not start at 0 or do not end at E: entries outside [indptr[0], indptr[N]) belong to
# no row (csrc/cuda/segment_csr_cuda.cu:30-33 reduces [indptr[n], indptr[n+1]) only)
WINDOW_CASES = [
    # kind, rows, K, entries in front of the first row, entries behind the last row
    ("zipf", 2000, 64, 37, 11), ("hub", 900, 64, 5000, 0), ("short", 300, 1, 3, 9), ("zipf", 2500, 4, 700, 1),
    ("hub", 500, 128, 1, 2500), ("long", 9, 8, 30000, 5), ("short", 50, 200, 9000, 9000), ("hub", 300, 16, 2, 2),
]


def make_window(case, seed):
    kind, n, K, front, back = case
    rng, indptr, _ = make_csr(kind, seed, n)
    if kind != "short":
        indptr = indptr.clone()
        # the first rows empty too: row 0 is not the one that begins behind the entries in front
        indptr[1:3] = 0
    return rng, indptr + front, int(indptr[-1]) + front + back


@pytest.mark.parametrize("case,reduce,dtype", product(
    WINDOW_CASES, ["sum", "mean", "min", "max"], [torch.float32, torch.bfloat16]))
def test_segment_csr_window_of_entries(capi, oracle, case, reduce, dtype):
    n, K = case[1], case[2]
    rng, indptr, E = make_window(case, 300 + WINDOW_CASES.index(case))
    src = values(rng, (E, K), dtype, reduce)
    want, want_arg = oracle.segment_csr(src, indptr, None, reduce)
    out = torch.full((n, K), 7, dtype=dtype, device=DEV)
    arg = torch.full((n, K), -1, dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
    capi.segment_csr(src.to(DEV), indptr.to(DEV), out, arg, 1, n, E, K, 0, capi.REDUCE[reduce])
    torch.cuda.synchronize()
    if reduce in ("min", "max"):
        assert_exact(out, want, "values")
        assert_exact(arg, want_arg, "arg")
    else:
        scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max())
        assert_close(out, want, scale, dtype, "values")


@pytest.mark.parametrize("case,dtype", product(WINDOW_CASES, [torch.float32, torch.bfloat16]))
def test_gather_csr_and_mean_backward_window_of_entries(capi, oracle, case, dtype):
    """Positions of the output outside [indptr[0], indptr[N]) are left as they were."""
    n, K = case[1], case[2]
    rng, indptr, E = make_window(case, 400 + WINDOW_CASES.index(case))
    src = random_values(rng, (n, K), dtype, ties=False)
    lo, hi = int(indptr[0]), int(indptr[-1])
    want = torch.full((E, K), 3, dtype=dtype)
    want[lo:hi] = oracle.gather_csr(src, indptr - lo)
    out = torch.full((E, K), 3, dtype=dtype, device=DEV)
    capi.gather_csr(src.to(DEV), indptr.to(DEV), out, 1, n, E, K, 0)
    torch.cuda.synchronize()
    assert_exact(out, want)
    want[lo:hi] = oracle.segment_mean_csr_backward(src, indptr - lo, (hi - lo, K))
    out.fill_(3)
    capi.segment_mean_csr_backward(src.to(DEV), indptr.to(DEV), out, 1, n, E, K, 0)
    torch.cuda.synchronize()
    assert_exact(out, want)


@pytest.mark.parametrize("reduce", ["sum", "mean", "max"])
def test_segment_csr_batched_window_of_entries(capi, oracle, reduce):
    rng = np.random.default_rng(77)
    B, n, K, E = 3, 400, 32, 9000
    ptrs = []
    for b in range(B):
        deg = rng.multinomial(E - 40 * (b + 1), np.ones(n) / n)
        ptrs.append(np.concatenate([[0], np.cumsum(deg)]) + 13 * (b + 1))
    indptr = torch.from_numpy(np.stack(ptrs).astype(np.int64))
    src = values(rng, (B, E, K), torch.float32, reduce)
    want, want_arg = oracle.segment_csr(src, indptr, None, reduce)
    out = torch.empty((B, n, K), dtype=torch.float32, device=DEV)
    arg = torch.empty((B, n, K), dtype=torch.long, device=DEV) if reduce == "max" else None
    capi.segment_csr(src.to(DEV), indptr.to(DEV), out, arg, B, n, E, K, n + 1, capi.REDUCE[reduce])
    torch.cuda.synchronize()
    if reduce == "max":
        assert_exact(out, want)
        assert_exact(arg, want_arg)
    else:
        assert_close(out, want, float(src.abs().sum(1).max()), torch.float32)


# ---- more batch rows than a grid dimension holds (65535): the reference has no such limit
# (csrc/cuda/segment_csr_cuda.cu:144-160 puts the batch into the flat thread index)
@pytest.mark.parametrize("reduce,K", product(["sum", "mean", "max"], [1, 8]))
def test_segment_csr_and_gathers_with_70000_batch_rows(capi, oracle, reduce, K):
    rng = np.random.default_rng(78)
    B, n, E = 70000, 3, 7
    deg = rng.multinomial(E, np.ones(n) / n, size=B)
    indptr = torch.from_numpy(np.concatenate([np.zeros((B, 1), np.int64), np.cumsum(deg, 1)], 1).astype(np.int64))
    src = values(rng, (B, E, K), torch.float32, reduce)
    want, want_arg = oracle.segment_csr(src, indptr, None, reduce)
    out = torch.empty((B, n, K), dtype=torch.float32, device=DEV)
    arg = torch.empty((B, n, K), dtype=torch.long, device=DEV) if reduce == "max" else None
    dptr = indptr.to(DEV)
    capi.segment_csr(src.to(DEV), dptr, out, arg, B, n, E, K, n + 1, capi.REDUCE[reduce])
    torch.cuda.synchronize()
    if reduce == "max":
        assert_exact(out, want)
        assert_exact(arg, want_arg)
    else:
        assert_close(out, want, float(src.abs().sum(1).max()), torch.float32)
    if reduce == "sum":
        # the gathers and the index-keyed reduction over the same batches
        back = torch.empty((B, E, K), dtype=torch.float32, device=DEV)
        capi.gather_csr(out, dptr, back, B, n, E, K, n + 1)
        assert_exact(back, oracle.gather_csr(out.cpu(), indptr))
        index = torch.from_numpy(np.stack([np.repeat(np.arange(n), d) for d in deg]).astype(np.int64))
        capi.gather_coo(out, index.to(DEV), back, B, n, E, K, E)
        assert_exact(back, oracle.gather_coo(out.cpu(), index))
        out2 = torch.empty_like(out)
        capi.segment_coo(src.to(DEV), index.to(DEV), out2, None, None, B, n, E, K, E, capi.SUM, False)
        torch.cuda.synchronize()
        assert_close(out2, want, float(src.abs().sum(1).max()), torch.float32)


@pytest.mark.parametrize("reduce", ["sum", "max"])
def test_scatter_with_70000_batch_rows(capi, oracle, reduce):
    """scatter along the last dimension of a [70000, 16] tensor (the reference's default dim = -1)."""
    rng = np.random.default_rng(79)
    B, E, N = 70000, 16, 5
    src = values(rng, (B, E), torch.float32, reduce)
    index = torch.from_numpy(rng.integers(0, N, size=(B, E)).astype(np.int64))
    want, want_arg = oracle.scatter(src, index, 1, None, N, reduce)
    out = torch.empty((B, N), dtype=torch.float32, device=DEV)
    arg = torch.empty((B, N), dtype=torch.long, device=DEV) if reduce == "max" else None
    capi.scatter(src.to(DEV), index.to(DEV), out, arg, B, E, 1, N, E, 1, 0, capi.REDUCE[reduce], False)
    torch.cuda.synchronize()
    if reduce == "max":
        assert_exact(out, want)
        assert_exact(arg, want_arg)
    else:
        assert_close(out, want, float(src.abs().sum(1).max()), torch.float32)


def test_segment_csr_status_word_reports_rows_that_were_given_up(capi, oracle, monkeypatch):
    """The wait of the look-back is bounded. With the bound forced to "never wait" from the host (TS_CSR_SPIN=-1)
    every row that crosses a tile is given up: the kernels still finish normally, the status word is set, those
    rows read as empty (0, arg = E) and every other row is correct. Without the override the word stays 0
    (checked on every call of the other tests, see conftest)."""
    rng, indptr, index = make_csr("hub", 55, 900)
    n, K, E = 900, 64, index.numel()
    src = values(rng, (E, K), torch.float32, "max")
    want, want_arg = oracle.segment_csr(src, indptr, None, "max")
    out = torch.empty((n, K), device=DEV)
    arg = torch.empty((n, K), dtype=torch.long, device=DEV)
    nbytes = capi.lib().ts_segment_csr_workspace_bytes(capi._i(1), capi._i(n), capi._i(E), capi._i(K), 0, capi.MAX)
    monkeypatch.setattr(capi, "CHECK_STATUS", False)
    monkeypatch.setenv("TS_CSR_SPIN", "-1")
    ws = capi.segment_csr(src.to(DEV), indptr.to(DEV), out, arg, 1, n, E, K, 0, capi.MAX)
    assert capi.status_word(ws, nbytes) == 1
    got, got_arg = out.cpu(), arg.cpu()
    deg = indptr[1:] - indptr[:-1]
    given_up = (got_arg == E).all(1) & (deg > 0)
    assert int(given_up.sum()) >= 1 and bool((got[given_up] == 0).all())
    assert bool((deg[given_up] >= 2).all())  # a row must have two entries to cross a tile
    assert torch.equal(got[~given_up], want[~given_up]) and torch.equal(got_arg[~given_up], want_arg[~given_up])
    monkeypatch.delenv("TS_CSR_SPIN")
    ws = capi.segment_csr(src.to(DEV), indptr.to(DEV), out, arg, 1, n, E, K, 0, capi.MAX)
    assert capi.status_word(ws, nbytes) == 0
    assert_exact(out, want)
    assert_exact(arg, want_arg)


K1_CASES = [
    # E, N, index: one value per entry through the workspace path (per-workgroup tables handed over in slabs)
    (30001, 500, "zipf"), (50003, 20000, "zipf"), (20002, 300000, "uniform"), (9000, 7, "zipf"),
    (40000, 9000, "uniform"), (3, 10, "uniform"), (70000, 100000, "zipf"),
]


@pytest.mark.parametrize("case,reduce,dtype", product(K1_CASES, ["min", "max"], [torch.float32, torch.int32]))
def test_scatter_minmax_one_value_per_entry_with_workspace(capi, oracle, case, reduce, dtype, monkeypatch):
    """Forced on at a small size. Heavy ties, NaN / infinite / lowest() values, indices outside [0, N), a number of
    entries that is no multiple of four, output rows that share a table row (N > 8192), a uniform index (every
    entry misses the table and goes through the queue). The same workspace serves two calls in a row: the key
    table in its first bytes has to come back as zeros."""
    monkeypatch.setenv("TS_SCATTER_LDS", "2")
    E, N, kind = case
    rng = np.random.default_rng(E + N)
    src = random_values(rng, (1, E, 1), dtype, ties=True)
    if kind == "zipf":
        p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
        index = rng.choice(N, size=E, p=p / p.sum())
        index = (index * 7919) % N  # hot rows spread over the id space
    else:
        index = rng.integers(0, N, size=E)
    index = torch.from_numpy(index.astype(np.int64))
    if E > 100:
        index[5] = -1
        index[77] = N
        if dtype.is_floating_point:
            src[0, 11, 0] = float("nan")
            src[0, 13, 0] = float("-inf") if reduce == "max" else float("inf")
            lim = torch.finfo(dtype).min if reduce == "max" else torch.finfo(dtype).max
        else:
            lim = torch.iinfo(dtype).min if reduce == "max" else torch.iinfo(dtype).max
        src[0, 17, 0] = lim  # does not beat the initial value: counts as no entry
        index[17] = N - 1
        index[index == N - 1] = N - 1
    valid = (index >= 0) & (index < N)
    want, want_arg = oracle.scatter(src[:, valid], index[valid].view(1, -1, 1), 1, None, N, reduce)
    # positions of the oracle are those of the filtered input: map them back
    pos = torch.nonzero(valid).flatten()
    keep = want_arg < pos.numel()
    want_arg = torch.where(keep, pos[want_arg.clamp(max=max(pos.numel() - 1, 0))], torch.full_like(want_arg, E))
    nbytes = capi.lib().ts_scatter_workspace_bytes(capi._i(1), capi._i(E), capi._i(1), capi._i(N), capi.DTYPE[dtype],
                                                  capi.REDUCE[reduce])
    nzero = capi.lib().ts_scatter_workspace_zero_bytes(capi._i(1), capi._i(E), capi._i(1), capi._i(N),
                                                      capi.DTYPE[dtype], capi.REDUCE[reduce])
    assert nbytes > nzero >= N * 8
    ws = None
    for rep in range(2):
        out = torch.full((1, N, 1), 5, dtype=dtype, device=DEV)
        arg = torch.full((1, N, 1), -3, dtype=torch.long, device=DEV)
        ws = capi.scatter_with_workspace(src.to(DEV), index.to(DEV), out, arg, 1, E, 1, N, 0, 1, 0,
                                         capi.REDUCE[reduce], False, ws)
        torch.cuda.synchronize()
        assert_exact(out, want, f"values rep={rep}")
        assert_exact(arg, want_arg, f"arg rep={rep}")
        assert bool((ws[:nzero] == 0).all()), "the key table is handed back as zeros"


@pytest.mark.parametrize("reduce", ["min", "max"])
def test_scatter_k1_workspace_kept_across_calls_with_different_row_counts(capi, oracle, reduce):
    """One workspace, cleared once, reused for calls whose N goes up and down: the zero-on-entry part has one
    size for every N, so the slabs of a call with few rows never sit where a later call keeps its keys."""
    rng = np.random.default_rng(5)
    E = 200_000
    sizes = [100_000, 50_000, 100_000, 300, 524_288, 100_000]
    L = capi.lib()
    nbytes = max(L.ts_scatter_workspace_bytes(capi._i(1), capi._i(E), capi._i(1), capi._i(N), capi.DTYPE[torch.float32],
                                              capi.REDUCE[reduce]) for N in sizes)
    zeros = {L.ts_scatter_workspace_zero_bytes(capi._i(1), capi._i(E), capi._i(1), capi._i(N), capi.DTYPE[torch.float32],
                                               capi.REDUCE[reduce]) for N in sizes}
    assert len(zeros) == 1 and min(zeros) >= max(sizes) * 8, zeros
    nzero = zeros.pop()
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    ws[nzero:] = 0xA5          # whatever earlier calls may have left behind the key table
    ws[:nzero].zero_()
    for step, N in enumerate(sizes):
        src = torch.from_numpy(rng.integers(-50, 51, size=(1, E, 1)).astype(np.float32))
        index = torch.from_numpy(rng.integers(0, N, size=E).astype(np.int64))
        want, want_arg = oracle.scatter(src, index.view(1, -1, 1), 1, None, N, reduce)
        out = torch.empty((1, N, 1), dtype=torch.float32, device=DEV)
        arg = torch.empty((1, N, 1), dtype=torch.long, device=DEV)
        ws2 = capi.scatter_with_workspace(src.to(DEV), index.to(DEV), out, arg, 1, E, 1, N, 0, 1, 0,
                                          capi.REDUCE[reduce], False, ws)
        assert ws2.data_ptr() == ws.data_ptr()
        torch.cuda.synchronize()
        assert_exact(out, want, f"values step={step} N={N}")
        assert_exact(arg, want_arg, f"arg step={step} N={N}")
        assert bool((ws[:nzero] == 0).all()), "the key table is handed back as zeros"


@pytest.mark.parametrize("dtype", [torch.int32, torch.float64, torch.float32])
def test_scatter_mean_of_a_group_with_more_than_2_pow_24_entries(capi, oracle, dtype):
    """One group of 2^24 + 3 entries, one value per entry: the count of scatter mean is an exact integer (a count
    of ones in fp32 would stop at 2^24), as the reference's count in int32 / double is (csrc/scatter.cpp:131-141).
    float32: the reference's own count of ones in fp32 stalls at 2^24; here the exact count is rounded once."""
    E, N = (1 << 24) + 3, 3
    index = torch.zeros(E, dtype=torch.long)
    index[5] = 2                      # one entry elsewhere; row 1 stays empty
    src = torch.ones((1, E, 1), dtype=dtype)
    src[0, 7, 0] = 9
    cnt = torch.empty((N,), dtype=torch.int32, device=DEV)
    capi.scatter_count(index.to(DEV), cnt, 1, E, N, 0, 1)
    assert cnt.tolist() == [E - 1, 0, 1]
    out = torch.empty((1, N, 1), dtype=dtype, device=DEV)
    capi.scatter(src.to(DEV), index.to(DEV), out, None, 1, E, 1, N, 0, 1, 0, capi.SUM, False)
    capi.divide_by_count(out, cnt, 1, N, 1)
    torch.cuda.synchronize()
    if dtype == torch.float32:
        want = torch.tensor([float(np.float32(np.float32(E - 1 + 8) / np.float32(E - 1))), 0.0, 1.0]).view(1, N, 1)
        assert torch.allclose(out.cpu(), want, rtol=1e-6, atol=0)
    else:
        want = oracle.op_scatter(src, index.view(1, E, 1), 1, None, N, "mean")
        assert_exact(out, want)


@pytest.mark.parametrize("case,reduce", product([("hub", 900, 64), ("zipf", 3000, 64), ("long", 12, 64)],
                                                ["sum", "mean", "min", "max"]))
def test_segment_csr_two_launch_fallback(capi, oracle, case, reduce, monkeypatch):
    """TS_CSR_LOOKBACK=0: rows that cross tiles are finished by the second kernel instead of the look-back inside
    the first (the path 8- / 16-bit accumulators and rows of more than four column chunks always take, and the way
    out for 4- / 8-byte accumulators should the look-back ever misbehave). fp32, 64 columns, every reduction, next
    to the look-back run of the same input (sums may differ in the last bits: the second kernel adds the partial
    sums of a row front to back, the look-back back to front)."""
    kind, n, K = case
    rng, indptr, index = make_csr(kind, 77, n)
    E = index.numel()
    src = values(rng, (E, K), torch.float32, reduce)
    want, want_arg = oracle.segment_csr(src, indptr, None, reduce)
    for lookback in ("0", "1"):
        monkeypatch.setenv("TS_CSR_LOOKBACK", lookback)
        out = torch.full((n, K), 7, dtype=torch.float32, device=DEV)
        arg = torch.full((n, K), -1, dtype=torch.long, device=DEV) if reduce in ("min", "max") else None
        capi.segment_csr(src.to(DEV), indptr.to(DEV), out, arg, 1, n, E, K, 0, capi.REDUCE[reduce])
        torch.cuda.synchronize()
        if reduce in ("min", "max"):
            assert_exact(out, want, f"values lookback={lookback}")
            assert_exact(arg, want_arg, f"arg lookback={lookback}")
        else:
            scale = float(oracle.segment_csr(src.abs().double(), indptr, None, "sum")[0].max())
            assert_close(out, want, scale, torch.float32, f"values lookback={lookback}")


@pytest.mark.parametrize("reduce", ["min", "max"])
def test_scatter_k1_reports_a_wait_that_ran_out(capi, oracle, reduce, monkeypatch):
    """The producers of the one-value-per-entry kernel wait (bounded) for room in a queue in LDS. With the bound
    forced to "never wait" from the host (TS_K1_SPIN=0) a full queue loses entries: every kernel still exits
    normally, and the word behind the key table says so -- a result is either exact or flagged. With the default
    bound the same input is exact and the word stays 0."""
    monkeypatch.setenv("TS_SCATTER_LDS", "2")
    rng = np.random.default_rng(3)
    E, N = 400_000, 300_000                       # a uniform index: nearly every entry goes through a queue
    src = torch.from_numpy(rng.standard_normal((1, E, 1)).astype(np.float32))
    index = torch.from_numpy(rng.integers(0, N, size=E).astype(np.int64))
    want, want_arg = oracle.scatter(src, index.view(1, -1, 1), 1, None, N, reduce)
    L = capi.lib()
    nzero = L.ts_scatter_workspace_zero_bytes(capi._i(1), capi._i(E), capi._i(1), capi._i(N), capi.DTYPE[torch.float32],
                                              capi.REDUCE[reduce])
    assert nzero >= capi.STATUS_BYTES
    monkeypatch.setattr(capi, "CHECK_STATUS", False)
    for spin, must_be_clean in (("0", False), (None, True)):
        if spin is None:
            monkeypatch.delenv("TS_K1_SPIN")
        else:
            monkeypatch.setenv("TS_K1_SPIN", spin)
        out = torch.empty((1, N, 1), dtype=torch.float32, device=DEV)
        arg = torch.empty((1, N, 1), dtype=torch.long, device=DEV)
        ws = capi.scatter_with_workspace(src.to(DEV), index.to(DEV), out, arg, 1, E, 1, N, 0, 1, 0,
                                         capi.REDUCE[reduce], False, None)
        torch.cuda.synchronize()
        flagged = int(ws[nzero - capi.STATUS_BYTES:nzero - capi.STATUS_BYTES + 8].view(torch.int64).item()) != 0
        exact = torch.equal(out.cpu(), want) and torch.equal(arg.cpu(), want_arg)
        assert exact or flagged, "a result that lost entries must be flagged"
        if must_be_clean:
            assert exact and not flagged


PAYLOAD_CASES = [
    # B, E, N, index: sums and counts of one 4-byte value per entry through (row in bucket, value) words
    (1, 30001, 500, "uniform"), (1, 50003, 20000, "zipf"), (1, 70000, 300000, "uniform"), (2, 9001, 7, "zipf"),
    (3, 40000, 9000, "uniform"), (1, 3, 10, "uniform"), (1, 120000, 100000, "hub"), (1, 65536, 4096, "uniform"),
    (1, 100000, 9_000_000, "uniform"),   # more buckets than the sorting place pass takes
]


@pytest.mark.parametrize("case,dtype,out_given", product(PAYLOAD_CASES, [torch.float32, torch.int32], [False, True]))
def test_scatter_sum_of_single_values_through_buckets(capi, oracle, case, dtype, out_given, monkeypatch):
    """Forced on at small sizes (TS_SCATTER_BINNED=2). Indices outside [0, N), a hub row, an odd number of entries,
    several batch rows, `out` given (the sums are added on top), an output with more rows than entries."""
    monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    B, E, N, kind = case
    rng = np.random.default_rng(E + N)
    if dtype.is_floating_point:
        src = torch.from_numpy(rng.standard_normal(size=(B, E, 1)).astype(np.float32))
    else:
        src = torch.from_numpy(rng.integers(-1000, 1000, size=(B, E, 1)).astype(np.int32))
    if kind == "zipf":
        p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
        index = (rng.choice(N, size=(B, E), p=p / p.sum()) * 7919) % N
    elif kind == "hub":
        index = rng.integers(0, N, size=(B, E))
        index[:, rng.random(E) < 0.4] = N // 3
    else:
        index = rng.integers(0, N, size=(B, E))
    index = torch.from_numpy(index.astype(np.int64))
    if E > 100:
        index[0, 5] = -1
        index[-1, 77] = N
    valid = (index >= 0) & (index < N)
    prev = torch.from_numpy(rng.integers(-5, 6, size=(B, N, 1))).to(dtype) if out_given else torch.zeros((B, N, 1), dtype=dtype)
    want = prev.clone().double()
    for b in range(B):
        want[b, :, 0].index_add_(0, index[b][valid[b]], src[b, valid[b], 0].double())
    nbytes = capi.lib().ts_scatter_workspace_bytes(capi._i(B), capi._i(E), capi._i(1), capi._i(N), capi.DTYPE[dtype], capi.SUM)
    assert nbytes >= 8 * B * E, "the plan for single values asks for 8 bytes of scratch per entry"
    out = prev.clone().to(DEV)
    capi.scatter_with_workspace(src.to(DEV), index.to(DEV), out, None, B, E, 1, N, E, 1, 0, capi.SUM, out_given)
    torch.cuda.synchronize()
    assert capi.scatter_last_route() == "sum: single values in buckets, table or runs (sample)"
    if dtype.is_floating_point:
        mags = torch.zeros((B, N, 1), dtype=torch.float64)
        for b in range(B):
            mags[b, :, 0].index_add_(0, index[b][valid[b]], src[b, valid[b], 0].double().abs())
        err = (out.cpu().double() - want).abs()
        assert bool((err <= 1e-5 * want.abs() + 1e-5 * mags.max()).all()), float(err.max())
    else:
        assert torch.equal(out.cpu().double(), want)
    # the count of the same index
    cnt = torch.empty((B, N), dtype=torch.int32, device=DEV)
    used = capi.scatter_count_with_workspace(index.to(DEV), cnt, B, E, N, E, 1)
    assert used >= 8 * B * E
    want_cnt = torch.stack([torch.bincount(index[b][valid[b]], minlength=N) for b in range(B)]).int()
    assert torch.equal(cnt.cpu(), want_cnt)


@pytest.mark.parametrize("case,dtype,out_given,forced", product(
    PAYLOAD_CASES + [(1, 90001, 5000, "sorted"), (1, 200000, 30000, "skewed")], [torch.float32, torch.int32], [False, True],
    [True, False]))
def test_scatter_sum_and_count_in_one_call(capi, case, dtype, out_given, forced, monkeypatch):
    """ts_scatter_sum_count_with_workspace: sum and int32 count of one value per entry from one pass over the index when
    the value buckets take the call (forced on at these sizes), the two separate calls otherwise (forced = False: these
    sizes are below the buckets' threshold). A sorted index (run kernels behind the buckets) and a heavily skewed one
    (table kernel behind the buckets) leave both results to the kernels behind the buckets."""
    if forced:
        monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    B, E, N, kind = case
    rng = np.random.default_rng(E + N + 1)
    if dtype.is_floating_point:
        src = torch.from_numpy(rng.integers(-9, 10, size=(B, E, 1)).astype(np.float32))  # small integers: exact sums
    else:
        src = torch.from_numpy(rng.integers(-1000, 1000, size=(B, E, 1)).astype(np.int32))
    if kind == "zipf":
        p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
        index = (rng.choice(N, size=(B, E), p=p / p.sum()) * 7919) % N
    elif kind == "skewed":
        p = np.arange(1, N + 1, dtype=np.float64) ** -2.0
        index = (rng.choice(N, size=(B, E), p=p / p.sum()) * 7919) % N
    elif kind == "hub":
        index = rng.integers(0, N, size=(B, E))
        index[:, rng.random(E) < 0.4] = N // 3
    elif kind == "sorted":
        index = np.sort(rng.integers(0, N, size=(B, E)), axis=1)
    else:
        index = rng.integers(0, N, size=(B, E))
    index = torch.from_numpy(index.astype(np.int64))
    if E > 100 and kind != "sorted":
        index[0, 5] = -1
        index[-1, 77] = N
    valid = (index >= 0) & (index < N)
    prev = torch.from_numpy(rng.integers(-5, 6, size=(B, N, 1))).to(dtype) if out_given else torch.zeros((B, N, 1), dtype=dtype)
    want = prev.clone().double()
    for b in range(B):
        want[b, :, 0].index_add_(0, index[b][valid[b]], src[b, valid[b], 0].double())
    want_cnt = torch.stack([torch.bincount(index[b][valid[b]], minlength=N) for b in range(B)]).int()
    out = prev.clone().to(DEV)
    cnt = torch.full((B, N), -7, dtype=torch.int32, device=DEV)
    used = capi.scatter_sum_count_with_workspace(src.to(DEV), index.to(DEV), out, cnt, B, E, 1, N, E, 1, out_given)
    torch.cuda.synchronize()
    if forced:
        assert used >= 8 * B * E
    assert torch.equal(out.cpu().double(), want)
    assert torch.equal(cnt.cpu(), want_cnt)


SMALL_MEAN_CASES = [
    # B, E, K, N, kind
    (1, 1, 1, 1, "uniform"), (1, 63, 1, 7, "uniform"), (1, 1000, 1, 100, "sorted"), (2, 777, 3, 50, "uniform"),
    (1, 4000, 16, 300, "sorted"), (1, 2000, 16, 3, "hub"), (3, 300, 64, 40, "uniform"), (1, 500, 130, 20, "sorted"),
    (1, 65535, 1, 1000, "hub"), (1, 1023, 33, 2000, "uniform"),
]


TABLE_MEAN_CASES = [
    (1, 70000, 1, 1000, "hub"), (1, 5000, 16, 300, "uniform"), (2, 3000, 64, 100, "sorted"), (1, 40000, 3, 5000, "uniform"),
    (1, 300000, 2, 2000, "uniform"), (1, 150000, 8, 100, "sorted"), (1, 600000, 1, 50000, "uniform"),
]


@pytest.mark.parametrize("case,dtype,out_given", product(
    SMALL_MEAN_CASES + TABLE_MEAN_CASES,
    [torch.float32, torch.float64, torch.bfloat16, torch.float16, torch.int32, torch.int64], [False, True]))
def test_scatter_sum_and_count_in_the_launch_that_adds(capi, case, dtype, out_given):
    """ts_scatter_sum_count_with_workspace where the sum is one launch: one launch clears out and the counts (which
    hold rubbish before the call), one launch adds and counts -- below 2^16 elements the run kernel beside a count
    through runs, above the table kernel with a table of counts. Rows of one column, of an odd number of columns
    (16-bit elements then go one by one instead of in packed pairs), of 128 bytes and more (every slot walks its own
    part), several batch rows, a hub row, indices outside [0, N), `out` given."""
    B, E, K, N, kind = case
    small = B * E * K < 1 << 16
    if dtype in (torch.bfloat16, torch.float16) and E > 40 * N:
        pytest.skip("sums of that many entries are not exactly representable in 16 bits")
    if dtype in (torch.bfloat16, torch.float16) and kind == "hub":
        pytest.skip("the sum of a hub row is not exactly representable in 16 bits")
    rng = np.random.default_rng(E * 31 + K * 7 + N)
    src = torch.from_numpy(rng.integers(-9, 10, size=(B, E, K))).to(dtype)   # small integers: exact sums in every type
    if kind == "hub":
        index = rng.integers(0, N, size=(B, E))
        index[:, rng.random(E) < 0.5] = N // 2
    elif kind == "sorted":
        index = np.sort(rng.integers(0, N, size=(B, E)), axis=1)
    else:
        index = rng.integers(0, N, size=(B, E))
    index = torch.from_numpy(index.astype(np.int64))
    if E > 100 and kind != "sorted":
        index[0, 5] = -1
        index[-1, 77] = N
    valid = (index >= 0) & (index < N)
    prev = torch.from_numpy(rng.integers(-5, 6, size=(B, N, K))).to(dtype) if out_given else torch.zeros((B, N, K), dtype=dtype)
    want = prev.clone().double()
    for b in range(B):
        want[b].index_add_(0, index[b][valid[b]], src[b, valid[b]].double())
    want_cnt = torch.stack([torch.bincount(index[b][valid[b]], minlength=N) for b in range(B)]).int()
    out = (prev.clone() if out_given else torch.full((B, N, K), 3, dtype=dtype)).to(DEV)
    cnt = torch.full((B, N), -7, dtype=torch.int32, device=DEV)
    capi.scatter_sum_count_with_workspace(src.to(DEV), index.to(DEV), out, cnt, B, E, K, N, E, 1, out_given)
    torch.cuda.synchronize()
    if small:
        assert capi.scatter_last_route() == "sum: runs, entries per row counted by the same launch"
    elif dtype == torch.float32:
        slabs = K == 1 and B == 1 and 1 << 19 <= E < 1 << 21
        assert capi.scatter_last_route() == ("sum: single values, tables in slabs" if slabs else "sum: table")
    assert torch.equal(out.cpu().double(), want)
    assert torch.equal(cnt.cpu(), want_cnt)


SLAB_CASES = [
    # E, N, kind, forced (TS_SCATTER_SLABS=2: outside the sizes where the route applies by itself)
    (600_001, 100_000, "uniform", False), (1 << 20, 300_000, "zipf", False), (700_003, 5000, "sorted", False),
    (524_290, 524_288, "uniform", False), (2_000_000, 8192, "hub", False),
    (1, 5, "uniform", True), (4099, 100, "hub", True), (70_000, 9000, "uniform", True), (3, 1, "uniform", True),
]


@pytest.mark.parametrize("case,dtype,out_given,counted", product(
    SLAB_CASES, [torch.float32, torch.int32], [False, True], [False, True]))
def test_scatter_sum_of_single_values_through_slabs(capi, case, dtype, out_given, counted, monkeypatch):
    """Single 4-byte values between the sizes of the table kernel and of the value buckets: a table per workgroup,
    handed over in slabs, and the counts of scatter mean from the same launches. An index in random order, skewed,
    with a hub row, in order (tables with few rows are written back with atomics and their slabs stay unused), as
    many output rows as the route takes, indices outside [0, N), a number of entries that is no multiple of four,
    `out` given."""
    E, N, kind, forced = case
    if forced:
        monkeypatch.setenv("TS_SCATTER_SLABS", "2")
    rng = np.random.default_rng(E + N)
    src = torch.from_numpy(rng.integers(-9, 10, size=(1, E, 1))).to(dtype)   # small integers: exact sums
    if kind == "zipf":
        p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
        index = (rng.choice(N, size=(1, E), p=p / p.sum()) * 7919) % N
    elif kind == "hub":
        index = rng.integers(0, N, size=(1, E))
        index[:, rng.random(E) < 0.4] = N // 3
    elif kind == "sorted":
        index = np.sort(rng.integers(0, N, size=(1, E)), axis=1)
    else:
        index = rng.integers(0, N, size=(1, E))
    index = torch.from_numpy(index.astype(np.int64))
    if E > 100 and kind != "sorted":
        index[0, 5] = -1
        index[0, 77] = N
    valid = (index >= 0) & (index < N)
    prev = torch.from_numpy(rng.integers(-5, 6, size=(1, N, 1))).to(dtype) if out_given else torch.zeros((1, N, 1), dtype=dtype)
    want = prev.clone().double()
    want[0, :, 0].index_add_(0, index[0][valid[0]], src[0, valid[0], 0].double())
    want_cnt = torch.bincount(index[0][valid[0]], minlength=N).int().view(1, N)
    out = (prev.clone() if out_given else torch.full((1, N, 1), 3, dtype=dtype)).to(DEV)
    if counted:
        cnt = torch.full((1, N), -7, dtype=torch.int32, device=DEV)
        capi.scatter_sum_count_with_workspace(src.to(DEV), index.to(DEV), out, cnt, 1, E, 1, N, E, 1, out_given)
    else:
        capi.scatter_with_workspace(src.to(DEV), index.to(DEV), out, None, 1, E, 1, N, E, 1, 0, capi.SUM, out_given)
    torch.cuda.synchronize()
    if counted and E < 1 << 16:   # (a small sum that counts as well has its own launch)
        assert capi.scatter_last_route() == "sum: runs, entries per row counted by the same launch"
    else:
        assert capi.scatter_last_route() == "sum: single values, tables in slabs"
    assert torch.equal(out.cpu().double(), want)
    if counted:
        assert torch.equal(cnt.cpu(), want_cnt)


VALUE_ROW_CASES = [
    # B, E, K, N, kind, forced (TS_SCATTER_BINNED=2: below the size from which the value buckets take a call)
    (1, (3 << 20) + 77, 3, 300_000, "uniform", False), (1, (1 << 21) + 2, 2, 1_000_000, "uniform", False),
    (1, 3_200_001, 3, 40_000, "zipf", False), (1, 2_200_000, 2, 5000, "sorted", False),
    (1, 90_001, 2, 5000, "uniform", True), (2, 50_003, 3, 3000, "hub", True), (1, 70_000, 2, 9000, "zipf", True),
    (1, 30_000, 3, 200_000, "uniform", True), (3, 20_001, 2, 100, "uniform", True), (1, 40_000, 3, 700, "sorted", True),
    (1, (1 << 22) + 5, 4, 700_000, "uniform", False), (2, 33_333, 4, 2500, "hub", True), (1, 3, 4, 2, "uniform", True),
]


@pytest.mark.parametrize("case,dtype,out_given,counted", product(
    VALUE_ROW_CASES, [torch.float32, torch.int32], [False, True], [False, True]))
def test_scatter_sum_of_narrow_rows_through_value_buckets(capi, case, dtype, out_given, counted, monkeypatch):
    """Rows of two to four 4-byte values under an index in no order: the values travel in binned records (the values,
    then the row in the bucket), and the counts of scatter mean come from the same pass. Row widths that are no power of
    two, several batch rows, a hub row, a skewed and a sorted index (which the sample hands to the table / run
    kernels behind the buckets), indices outside [0, N), `out` given."""
    B, E, K, N, kind, forced = case
    if forced:
        monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    rng = np.random.default_rng(E + N + K)
    src = torch.from_numpy(rng.integers(-9, 10, size=(B, E, K))).to(dtype)   # small integers: exact sums
    if kind == "zipf":
        p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
        index = (rng.choice(N, size=(B, E), p=p / p.sum()) * 7919) % N
    elif kind == "hub":
        index = rng.integers(0, N, size=(B, E))
        index[:, rng.random(E) < 0.4] = N // 3
    elif kind == "sorted":
        index = np.sort(rng.integers(0, N, size=(B, E)), axis=1)
    else:
        index = rng.integers(0, N, size=(B, E))
    index = torch.from_numpy(index.astype(np.int64))
    if kind != "sorted" and E > 100:
        index[0, 5] = -1
        index[-1, 77] = N
    valid = (index >= 0) & (index < N)
    prev = torch.from_numpy(rng.integers(-5, 6, size=(B, N, K))).to(dtype) if out_given else torch.zeros((B, N, K), dtype=dtype)
    want = prev.clone().double()
    for b in range(B):
        want[b].index_add_(0, index[b][valid[b]], src[b, valid[b]].double())
    want_cnt = torch.stack([torch.bincount(index[b][valid[b]], minlength=N) for b in range(B)]).int()
    out = (prev.clone() if out_given else torch.full((B, N, K), 3, dtype=dtype)).to(DEV)
    if counted:
        cnt = torch.full((B, N), -7, dtype=torch.int32, device=DEV)
        capi.scatter_sum_count_with_workspace(src.to(DEV), index.to(DEV), out, cnt, B, E, K, N, E, 1, out_given)
    else:
        capi.scatter_with_workspace(src.to(DEV), index.to(DEV), out, None, B, E, K, N, E, 1, 0, capi.SUM, out_given)
    torch.cuda.synchronize()
    assert capi.scatter_last_route() == "sum: single values in buckets, table or runs (sample)"
    assert torch.equal(out.cpu().double(), want)
    if counted:
        assert torch.equal(cnt.cpu(), want_cnt)


def test_scatter_sum_of_single_values_sorted_index_keeps_the_run_kernels(capi, oracle, monkeypatch):
    """A sorted index: the sample sends the call to the kernels that combine runs; the bucket passes return at once."""
    monkeypatch.setenv("TS_SCATTER_BINNED", "2")
    rng = np.random.default_rng(8)
    E, N = 90_001, 5000
    index = torch.from_numpy(np.sort(rng.integers(0, N, size=E)).astype(np.int64))
    src = torch.from_numpy(rng.integers(-9, 10, size=(1, E, 1)).astype(np.float32))     # small integers: exact
    want, _ = oracle.scatter(src, index.view(1, -1, 1), 1, None, N, "sum")
    out = torch.zeros((1, N, 1), device=DEV)
    capi.scatter_with_workspace(src.to(DEV), index.to(DEV), out, None, 1, E, 1, N, 0, 1, 0, capi.SUM, False)
    assert_exact(out, want)
