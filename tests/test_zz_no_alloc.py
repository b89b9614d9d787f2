"""ts_segment_csr_static, the entry point that allocates nothing: its scratch is a device array inside the
library. Checked through the C ABI against ts_segment_csr (same kernels, caller's workspace) bit for bit, on two
calls in a row that share the array, the second with a smaller input; inputs beyond the array are refused."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(seed, n, K, dtype, zipf):
    rng = np.random.default_rng(seed)
    deg = np.minimum(rng.zipf(zipf, size=n), 5000)
    deg[rng.random(n) < 0.1] = 0
    indptr = torch.from_numpy(np.concatenate([[0], np.cumsum(deg)]).astype(np.int64))
    E = int(indptr[-1])
    src = torch.from_numpy(rng.integers(-8, 9, size=(E, K)).astype(np.float32)).to(dtype)  # exact ties for min / max
    return src, indptr, E


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K", [1, 64, 300])
@pytest.mark.parametrize("reduce", ["sum", "mean", "min", "max"])
def test_static_scratch_matches_workspace_call(reduce, K, dtype):
    from pytorch_scatter_amd import capi
    dev = torch.device("cuda:0")
    r = capi.REDUCE[reduce]
    # two calls in a row on the same array: a large input first, then a smaller one
    for seed, n in ((1, 30000 if K <= 64 else 6000), (2, 1500)):
        src, indptr, E = _case(seed, n, K, dtype, 1.6)
        src, indptr = src.to(dev), indptr.to(dev)
        want = torch.empty((n, K), dtype=dtype, device=dev)
        got = torch.full((n, K), 7, dtype=dtype, device=dev)
        arg_want = torch.empty((n, K), dtype=torch.int64, device=dev) if r >= capi.MIN else None
        arg_got = torch.full((n, K), -5, dtype=torch.int64, device=dev) if r >= capi.MIN else None
        capi.segment_csr(src, indptr, want, arg_want, 1, n, E, K, 0, r)
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        capi.segment_csr_static(src, indptr, got, arg_got, 1, n, E, K, 0, r)
        assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), (reduce, K, dtype, n)
        if arg_got is not None:
            assert torch.equal(arg_got, arg_want)


def test_static_scratch_batched_indptr():
    from pytorch_scatter_amd import capi
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5)
    B, n, K = 3, 4000, 32
    deg = rng.integers(0, 9, size=(B, n))
    E = int(deg.sum(1).max())
    deg[:, -1] += E - deg.sum(1)  # every batch row of indptr ends at E
    indptr = torch.from_numpy(np.concatenate([np.zeros((B, 1), np.int64), np.cumsum(deg, 1)], 1)).to(dev)
    src = torch.randn((B, E, K), device=dev)
    for r in (capi.SUM, capi.MAX):
        want, got = torch.empty((B, n, K), device=dev), torch.empty((B, n, K), device=dev)
        aw = torch.empty((B, n, K), dtype=torch.int64, device=dev)
        ag = torch.empty_like(aw)
        capi.segment_csr(src, indptr, want, aw, B, n, E, K, n + 1, r)
        capi.segment_csr_static(src, indptr, got, ag, B, n, E, K, n + 1, r)
        assert torch.equal(got, want)
        if r == capi.MAX:
            assert torch.equal(ag, aw)


def test_static_scratch_refuses_inputs_beyond_the_array():
    from pytorch_scatter_amd import capi
    dev = torch.device("cuda:0")
    n, E, K = 1000, 120000, 1024  # rows of 4 KB: the partial results of the tiles need more than the array holds
    need = capi.lib().ts_segment_csr_workspace_bytes(capi._i(1), capi._i(n), capi._i(E), capi._i(K), 0, capi.SUM)
    assert need > capi.STATIC_SCRATCH_BYTES
    src = torch.zeros((E, K), device=dev)
    indptr = (torch.arange(n + 1, device=dev) * (E // n)).to(torch.int64)
    out = torch.full((n, K), 3.0, device=dev)
    with pytest.raises(capi.TsError, match="workspace"):
        capi.segment_csr_static(src, indptr, out, None, 1, n, E, K, 0, capi.SUM)
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())  # nothing was launched
    want = torch.empty_like(out)
    capi.segment_csr(src, indptr, want, None, 1, n, E, K, 0, capi.SUM)  # the workspace call takes it
    assert bool((want == 0).all())
