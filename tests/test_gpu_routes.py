"""Which kernels the scatter dispatcher picks for the measured configurations.

The dispatcher chooses by sizes, element type and workspace; a threshold edit can silently send a configuration
down another path. These tests pin the route (ts_scatter_last_route, a host-side note left by the launcher) of C1,
C4 with one and with 32 values per entry, and of the extra shapes of the benchmark table, next to a value check
(column totals, arg invariants) so that the route that is asserted is also a route that works; the values of the same
calls are compared with the CPU oracle in test_gpu_fullsize.py."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture(scope="module")
def env():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import pytorch_scatter_amd as ts
    from pytorch_scatter_amd import capi
    from pytorch_scatter_amd import workloads as wl
    return ts, capi, wl


def _check_sum(got, src, index, N):
    """Cheap global check (the values of these calls are compared with the CPU oracle element by element in
    test_gpu_fullsize.py): every entry lands in exactly one row, so the column totals of out equal those of src."""
    want = src.double().sum(0)
    scale = src.double().abs().sum(0)
    assert bool(((got.double().sum(0) - want).abs() <= 1e-5 * scale).all())


def _check_max(got, arg, src, index, N):
    """arg invariants: the position points at an entry of that row which holds the row's value; rows without
    entries read 0 / E."""
    E = src.shape[0]
    hit = arg < E
    a = arg.clamp(max=E - 1)
    assert torch.equal(torch.gather(src, 0, a)[hit], got[hit])
    rows = torch.arange(N, device=DEV).view(-1, 1).expand_as(arg)
    assert torch.equal(index[a][hit], rows[hit])
    assert bool((got[~hit] == 0).all())
    assert int(hit[:, 0].sum()) == int(torch.unique(index).numel())


def test_route_c1(env):
    ts, capi, wl = env
    w = wl.c1_scatter_sum()
    src, index = wl.scatter_values(w, DEV), w.index.to(DEV)
    got = ts.scatter_sum(src, index, 0, None, w.N)
    assert capi.scatter_last_route() == "sum: table"
    _check_sum(got, src, index, w.N)


@pytest.mark.parametrize("K,route", [(1, "min/max: slabs, one value per entry"),
                                     (32, "min/max: buckets or segmented reduction (index checked)")])
def test_route_c4_max(env, K, route):
    ts, capi, wl = env
    w = wl.c4_scatter_minmax(K)
    src, index = wl.scatter_values(w, DEV), w.index.to(DEV)
    got, arg = ts.scatter_max(src, index, 0, None, w.N)
    assert capi.scatter_last_route() == route
    _check_max(got, arg, src, index, w.N)


def test_route_c4_k32_sum_and_sorted_k64(env):
    ts, capi, wl = env
    w = wl.c4_scatter_minmax(32)
    src, index = wl.scatter_values(w, DEV), w.index.to(DEV)
    got = ts.scatter_sum(src, index, 0, None, w.N)
    assert capi.scatter_last_route() == "sum: buckets or segmented reduction (index checked)"
    _check_sum(got, src, index, w.N)
    del src, got
    w3 = wl.c3_segment_coo()
    index = w3.index.to(DEV)
    src = torch.randn((w3.E, 64), device=DEV)
    got = ts.scatter_sum(src, index, 0, None, w3.N)
    assert capi.scatter_last_route() == "sum: buckets or segmented reduction (index checked)"
    _check_sum(got, src, index, w3.N)
    got, arg = ts.scatter_max(src, index, 0, None, w3.N)
    assert capi.scatter_last_route() == "min/max: buckets or segmented reduction (index checked)"
    _check_max(got, arg, src, index, w3.N)


def test_route_narrow_rows_unsorted(env):
    ts, capi, wl = env
    wz = wl.c4_scatter_minmax(1)
    g = torch.Generator().manual_seed(0)
    index = (wz.index[torch.randperm(wz.E, generator=g)] * 10 % 1_000_000).to(DEV)
    src = torch.randn((wz.E, 8), device=DEV)
    got = ts.scatter_sum(src, index, 0, None, 1_000_000)
    route_sum = capi.scatter_last_route()
    _check_sum(got, src, index, 1_000_000)
    got, arg = ts.scatter_max(src, index, 0, None, 1_000_000)
    assert capi.scatter_last_route() == "min/max: runs or table (sample)"
    _check_max(got, arg, src, index, 1_000_000)
    assert route_sum == "sum: table or runs (sample)"


@pytest.mark.parametrize("E,route", [((1 << 21) + 4096, "sum: single values in buckets, table or runs (sample)"),
                                     ((1 << 21) - 4096, "sum: single values, tables in slabs"),
                                     ((1 << 19) + 4096, "sum: single values, tables in slabs"),
                                     ((1 << 19) - 4096, "sum: table")])
def test_route_single_values_either_side_of_the_value_buckets(env, E, route):
    """One float per entry under an index in random order (the width-1 column of the benchmark table): value
    buckets from 2^21 entries, tables handed over in slabs from 2^19, the accumulator table below."""
    ts, capi, _ = env
    g = torch.Generator().manual_seed(E)
    N = 270_000
    index = torch.randint(0, N, (E,), generator=g).to(DEV)
    src = torch.randn((E, 1), device=DEV)
    got = ts.scatter_sum(src, index, 0, None, N)
    assert capi.scatter_last_route() == route
    _check_sum(got, src, index, N)
    want = torch.zeros((N, 1), dtype=torch.float64, device=DEV).index_add_(0, index, src.double())
    assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-4)
