"""The registered operators (torch.ops.torch_scatter.* through the Python API)
on the GPU against the reference's known-answer tables, with the reference's
own test matrix: forward (eager and TorchScript), gradcheck, `out=`,
non-contiguous inputs, zero-size tensors, broadcasting, composites.
Follows test/test_scatter.py, test_segment.py, test_gather.py,
test_zero_tensors.py, test_broadcasting.py and test/composite/*."""
from itertools import product

import numpy as np
import pytest
import torch
from torch.autograd import gradcheck

from helpers import DTYPES, REDUCTIONS, load_cases, random_csr, random_values, tensor

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")

SCATTER = load_cases("scatter_cases")
SEGMENT = load_cases("segment_cases")
GATHER = load_cases("gather_cases")


@pytest.fixture(scope="module")
def ts():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import pytorch_scatter_amd
    return pytorch_scatter_amd


@pytest.mark.parametrize("ci,reduce,dtype", product(range(len(SCATTER)), REDUCTIONS + ["mul"], DTYPES))
def test_scatter_forward(ts, ci, reduce, dtype):
    case = SCATTER[ci]
    if reduce not in case:
        pytest.skip("table has no entry for this reduction")
    src = tensor(case["src"], dtype, DEV)
    index = tensor(case["index"], torch.long, DEV)
    expected = tensor(case[reduce], dtype, DEV)
    fn = getattr(ts, "scatter_" + reduce)
    jit = torch.jit.script(fn)
    out1 = fn(src, index, case["dim"])
    out2 = jit(src, index, case["dim"])
    if isinstance(out1, tuple):
        out1, arg1 = out1
        out2, arg2 = out2
        if "arg_" + reduce in case:
            assert torch.all(arg1 == tensor(case["arg_" + reduce], torch.long, DEV))
        assert arg1.tolist() == arg2.tolist()
    assert torch.all(out1 == expected)
    assert out1.tolist() == out2.tolist()


@pytest.mark.parametrize("ci,reduce", product(range(6), REDUCTIONS + ["mul"]))
def test_scatter_backward(ts, ci, reduce):
    case = SCATTER[ci]
    src = tensor(case["src"], torch.double, DEV).requires_grad_()
    index = tensor(case["index"], torch.long, DEV)
    assert gradcheck(ts.scatter, (src, index, case["dim"], None, None, reduce))


@pytest.mark.parametrize("ci,reduce,dtype", product(range(6), REDUCTIONS + ["mul"], DTYPES))
def test_scatter_out(ts, ci, reduce, dtype):
    case = SCATTER[ci]
    src = tensor(case["src"], dtype, DEV)
    index = tensor(case["index"], torch.long, DEV)
    expected = tensor(case[reduce], dtype, DEV)
    out = torch.full_like(expected, -2)
    getattr(ts, "scatter_" + reduce)(src, index, case["dim"], out)
    if reduce in ("sum", "add"):
        expected = expected - 2
    elif reduce in ("mul", "mean"):
        expected = out  # not checkable from the table (as upstream)
    elif reduce == "min":
        expected = expected.fill_(-2)
    elif reduce == "max":
        expected[expected == 0] = -2
    assert torch.all(out == expected)


@pytest.mark.parametrize("ci,reduce,dtype", product(range(6), REDUCTIONS + ["mul"], DTYPES))
def test_scatter_non_contiguous(ts, ci, reduce, dtype):
    case = SCATTER[ci]
    src = tensor(case["src"], dtype, DEV)
    index = tensor(case["index"], torch.long, DEV)
    expected = tensor(case[reduce], dtype, DEV)
    if src.dim() > 1:
        src = src.transpose(0, 1).contiguous().transpose(0, 1)
    if index.dim() > 1:
        index = index.transpose(0, 1).contiguous().transpose(0, 1)
    out = getattr(ts, "scatter_" + reduce)(src, index, case["dim"])
    if isinstance(out, tuple):
        out, arg = out
        assert torch.all(arg == tensor(case["arg_" + reduce], torch.long, DEV))
    assert torch.all(out == expected)


@pytest.mark.parametrize("ci,reduce,dtype", product(range(len(SEGMENT)), REDUCTIONS, DTYPES))
def test_segment_forward(ts, ci, reduce, dtype):
    case = SEGMENT[ci]
    if reduce not in case:
        pytest.skip("table has no entry for this reduction")
    src = tensor(case["src"], dtype, DEV)
    index = tensor(case["index"], torch.long, DEV)
    indptr = tensor(case["indptr"], torch.long, DEV)
    expected = tensor(case[reduce], dtype, DEV)
    for name, idx in (("_csr", indptr), ("_coo", index)):
        fn = getattr(ts, "segment_" + reduce + name)
        jit = torch.jit.script(fn)
        out1 = fn(src, idx)
        out2 = jit(src, idx)
        if isinstance(out1, tuple):
            out1, arg1 = out1
            out2, arg2 = out2
            assert torch.all(arg1 == tensor(case["arg_" + reduce], torch.long, DEV))
            assert arg1.tolist() == arg2.tolist()
        assert torch.all(out1 == expected), name
        assert out1.tolist() == out2.tolist()


@pytest.mark.parametrize("ci,reduce", product(range(6), REDUCTIONS))
def test_segment_backward(ts, ci, reduce):
    case = SEGMENT[ci]
    src = tensor(case["src"], torch.double, DEV).requires_grad_()
    index = tensor(case["index"], torch.long, DEV)
    indptr = tensor(case["indptr"], torch.long, DEV)
    assert gradcheck(ts.segment_csr, (src, indptr, None, reduce))
    assert gradcheck(ts.segment_coo, (src, index, None, None, reduce))


@pytest.mark.parametrize("ci,reduce,dtype", product(range(6), REDUCTIONS, DTYPES))
def test_segment_out(ts, ci, reduce, dtype):
    case = SEGMENT[ci]
    src = tensor(case["src"], dtype, DEV)
    index = tensor(case["index"], torch.long, DEV)
    indptr = tensor(case["indptr"], torch.long, DEV)
    expected = tensor(case[reduce], dtype, DEV)
    out = torch.full_like(expected, -2)
    getattr(ts, "segment_" + reduce + "_csr")(src, indptr, out)   # csr overwrites
    assert torch.all(out == expected)
    out.fill_(-2)
    getattr(ts, "segment_" + reduce + "_coo")(src, index, out)    # coo accumulates
    if reduce in ("sum", "add"):
        expected = expected - 2
    elif reduce == "mean":
        expected = out
    elif reduce == "min":
        expected = expected.fill_(-2)
    elif reduce == "max":
        expected[expected == 0] = -2
    assert torch.all(out == expected)


@pytest.mark.parametrize("ci,reduce,dtype", product(range(6), REDUCTIONS, DTYPES))
def test_segment_non_contiguous(ts, ci, reduce, dtype):
    case = SEGMENT[ci]
    src = tensor(case["src"], dtype, DEV)
    index = tensor(case["index"], torch.long, DEV)
    indptr = tensor(case["indptr"], torch.long, DEV)
    expected = tensor(case[reduce], dtype, DEV)
    if src.dim() > 1:
        src = src.transpose(0, 1).contiguous().transpose(0, 1)
    if index.dim() > 1:
        index = index.transpose(0, 1).contiguous().transpose(0, 1)
    if indptr.dim() > 1:
        indptr = indptr.transpose(0, 1).contiguous().transpose(0, 1)
    for name, idx in (("_csr", indptr), ("_coo", index)):
        out = getattr(ts, "segment_" + reduce + name)(src, idx)
        if isinstance(out, tuple):
            out, arg = out
            assert torch.all(arg == tensor(case["arg_" + reduce], torch.long, DEV))
        assert torch.all(out == expected)


@pytest.mark.parametrize("ci,dtype", product(range(len(GATHER)), DTYPES))
def test_gather_forward_out_non_contiguous(ts, ci, dtype):
    case = GATHER[ci]
    src = tensor(case["src"], dtype, DEV)
    index = tensor(case["index"], torch.long, DEV)
    indptr = tensor(case["indptr"], torch.long, DEV)
    expected = tensor(case["expected"], dtype, DEV)
    assert torch.all(ts.gather_csr(src, indptr) == expected)
    assert torch.all(ts.gather_coo(src, index) == expected)
    size = list(src.size())
    size[index.dim() - 1] = index.size(-1)
    out = src.new_full(size, -2)
    ts.gather_csr(src, indptr, out)
    assert torch.all(out == expected)
    out.fill_(-2)
    ts.gather_coo(src, index, out)
    assert torch.all(out == expected)
    if src.dim() > 1:
        src = src.transpose(0, 1).contiguous().transpose(0, 1)
    if index.dim() > 1:
        index = index.transpose(0, 1).contiguous().transpose(0, 1)
        indptr = indptr.transpose(0, 1).contiguous().transpose(0, 1)
    assert torch.all(ts.gather_csr(src, indptr) == expected)
    assert torch.all(ts.gather_coo(src, index) == expected)


@pytest.mark.parametrize("ci", range(len(GATHER)))
def test_gather_backward(ts, ci):
    case = GATHER[ci]
    src = tensor(case["src"], torch.double, DEV).requires_grad_()
    index = tensor(case["index"], torch.long, DEV)
    indptr = tensor(case["indptr"], torch.long, DEV)
    assert gradcheck(ts.gather_csr, (src, indptr, None)) is True
    assert gradcheck(ts.gather_coo, (src, index, None)) is True


@pytest.mark.parametrize("reduce,dtype", product(REDUCTIONS, [torch.float, torch.double]))
def test_zero_elements(ts, reduce, dtype):
    x = torch.randn(0, 0, 0, 16, dtype=dtype, device=DEV, requires_grad=True)
    index = tensor([], torch.long, DEV)
    indptr = tensor([], torch.long, DEV)
    for out in (ts.scatter(x, index, dim=0, dim_size=0, reduce=reduce),
                ts.segment_coo(x, index, dim_size=0, reduce=reduce),
                ts.gather_coo(x, index),
                ts.segment_csr(x, indptr, reduce=reduce),
                ts.gather_csr(x, indptr)):
        out.backward(torch.randn_like(out))
        assert out.size() == (0, 0, 0, 16)


@pytest.mark.parametrize("reduce", REDUCTIONS)
def test_broadcasting(ts, reduce):
    B, C, H, W = (4, 3, 8, 8)
    src = torch.randn((B, C, H, W), device=DEV)
    index = torch.randint(0, H, (H,)).to(DEV, torch.long)
    assert ts.scatter(src, index, dim=2, dim_size=H, reduce=reduce).size() == (B, C, H, W)
    index = torch.randint(0, H, (B, 1, H, W)).to(DEV, torch.long)
    assert ts.scatter(src, index, dim=2, dim_size=H, reduce=reduce).size() == (B, C, H, W)


def test_scatter_matches_oracle_with_full_shape_index(ts, oracle):
    rng = np.random.default_rng(0)
    src = random_values(rng, (4, 3, 8, 5), torch.float, ties=True)
    for shape, dim in (((8,), 2), ((4, 1, 8, 5), 2), ((4, 3, 8, 5), 1), ((5,), 3), ((4,), 0)):
        index = torch.from_numpy(rng.integers(0, 6, size=shape))
        if len(shape) == 4 and shape[1] == 1:
            index = index.expand(4, 3, 8, 5)
        for reduce in ("sum", "mean", "min", "max", "mul"):
            want = oracle.op_scatter(src, index, dim, None, 7, reduce)
            got = getattr(ts, "scatter_" + reduce)(src.to(DEV), index.to(DEV), dim, None, 7)
            if isinstance(got, tuple):
                assert torch.equal(got[1].cpu(), want[1]), (shape, dim, reduce)
                got, want = got[0], want[0]
            assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-5), (shape, dim, reduce)


def test_fused_mean_backward_matches_closed_form(ts, oracle):
    rng = np.random.default_rng(1)
    indptr, index = random_csr(rng, 300, 40)
    E = index.numel()
    for dtype in (torch.float, torch.bfloat16):
        src = torch.from_numpy(rng.standard_normal((E, 24))).to(dtype).to(DEV).requires_grad_()
        g = torch.from_numpy(rng.standard_normal((300, 24))).to(dtype)
        ts.segment_csr(src, indptr.to(DEV), reduce="mean").backward(g.to(DEV))
        want = oracle.segment_mean_csr_backward(g, indptr, (E, 24))
        assert torch.equal(src.grad.cpu(), want)
        src.grad = None
        ts.segment_coo(src, index.to(DEV), dim_size=300, reduce="mean").backward(g.to(DEV))
        _, count = oracle.segment_coo(src.detach().cpu(), index, None, 300, "mean")
        want = oracle.segment_mean_coo_backward(g, index, count, (E, 24))
        assert torch.equal(src.grad.cpu(), want)
        src.grad = None


def test_min_max_backward_matches_reference_formula(ts, oracle):
    rng = np.random.default_rng(2)
    indptr, index = random_csr(rng, 200, 12)
    E = index.numel()
    src_cpu = random_values(rng, (E, 6), torch.double, ties=True)
    g = torch.from_numpy(rng.standard_normal((200, 6)))
    perm = torch.from_numpy(rng.permutation(E))
    for reduce in ("min", "max"):
        for fn, idx in ((ts.segment_csr, indptr), (ts.segment_coo, index)):
            src = src_cpu.clone().to(DEV).requires_grad_()
            args = (src, idx.to(DEV), None, reduce) if fn is ts.segment_csr else (src, idx.to(DEV), None, 200, reduce)
            fn(*args).backward(g.to(DEV))
            _, arg = oracle.segment_csr(src_cpu, indptr, None, reduce)
            assert torch.equal(src.grad.cpu(), oracle.arg_backward(g, arg, (E, 6), 0))
        src = src_cpu[perm].clone().to(DEV).requires_grad_()
        ts.scatter(src, index[perm].to(DEV), 0, None, 200, reduce).backward(g.to(DEV))
        _, arg = oracle.scatter(src_cpu[perm], oracle.broadcast(index[perm], src_cpu, 0), 0, None, 200, reduce)
        assert torch.equal(src.grad.cpu(), oracle.arg_backward(g, arg, (E, 6), 0))


def test_composites_against_dense_torch(ts):
    # test/composite/test_softmax.py, test_logsumexp.py, test_std.py
    src = torch.tensor([0.2, 0, 0.2, -2.1, 3.2, 7, -1, float("-inf")], device=DEV)
    index = torch.tensor([0, 1, 0, 1, 1, 2, 4, 4], device=DEV)
    out = ts.scatter_softmax(src, index)
    groups = [[0, 2], [1, 3, 4], [5], [6, 7]]
    for g in groups:
        assert torch.allclose(out[g], torch.softmax(src[g], dim=-1))
    out = ts.scatter_log_softmax(src, index)
    for g in groups:
        assert torch.allclose(out[g], torch.log_softmax(src[g], dim=-1))
    out = ts.scatter_logsumexp(src, index)
    want = torch.stack([torch.logsumexp(src[g], dim=-1) for g in groups[:3]] +
                       [torch.tensor(0.0, device=DEV), torch.logsumexp(src[groups[3]], dim=-1)])
    assert torch.allclose(out, want)
    src = torch.tensor([[2.0, 0, 1, 4, 3], [0, 2, 1, 3, 4]], device=DEV, requires_grad=True)
    index = torch.tensor([[0, 0, 0, 0, 0], [1, 1, 1, 1, 1]], device=DEV)
    out = ts.scatter_std(src, index, dim=-1, unbiased=True)
    std = src.std(dim=-1, unbiased=True)[0]
    assert torch.allclose(out, torch.tensor([[std, 0], [0, std]], device=DEV))
    out.backward(torch.randn_like(out))


def test_errors_follow_reference_conventions(ts):
    src = torch.randn(6, 4, device=DEV)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        ts.segment_csr(src, torch.tensor([0, 3, 6], device=DEV), torch.empty(5, 4, device=DEV))
    with pytest.raises(RuntimeError, match="Input mismatch"):
        ts.gather_csr(src, torch.tensor([0, 3, 6], device=DEV))
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        ts.scatter_sum(src, torch.tensor([0, 1, 0, 1, 2, 2]), 0)


def test_ops_on_a_side_stream_and_in_a_hip_graph(ts, oracle):
    """Launches go to the caller's current stream and nothing allocates outside the
    caching allocator or synchronises (with `out` / `dim_size` given), so a step
    can be captured into a HIP graph; every replay is checked against eager."""
    rng = np.random.default_rng(3)
    indptr_c, index_c = random_csr(rng, 4000, 30)
    E = index_c.numel()
    indptr, index = indptr_c.to(DEV), index_c.to(DEV)
    perm = torch.from_numpy(rng.permutation(E)).to(DEV)
    src = torch.randn(E, 32, device=DEV)
    out_mean = torch.empty(4000, 32, device=DEV)
    back = torch.empty(E, 32, device=DEV)

    def step():
        ts.segment_csr(src, indptr, out_mean, "mean")
        ts.gather_csr(out_mean, indptr, back)
        mx, arg = ts.scatter_max(back[perm], index[perm], 0, None, 4000)
        sm = ts.segment_coo(src, index, None, 4000, "sum")
        return mx, arg, sm

    # side stream
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        mx_s, arg_s, sm_s = step()
    side.synchronize()
    with torch.no_grad():
        mx_e, arg_e, sm_e = step()
    torch.cuda.synchronize()
    want_mean, _ = oracle.segment_csr(src.cpu(), indptr_c, None, "mean")
    assert torch.allclose(out_mean.cpu(), want_mean, rtol=1e-5, atol=1e-5)
    assert torch.equal(mx_s, mx_e) and torch.equal(arg_s, arg_e) and torch.equal(sm_s, sm_e)

    # graph capture and replays with changing inputs
    g = torch.cuda.CUDAGraph()
    with torch.no_grad():
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()  # warm-up on the capture stream
        torch.cuda.current_stream().wait_stream(side)
        with torch.cuda.graph(g):
            mx_g, arg_g, sm_g = step()
        for i in range(3):
            src.copy_(torch.randn(E, 32, device=DEV))
            g.replay()
            torch.cuda.synchronize()
            got = (mx_g.clone(), arg_g.clone(), sm_g.clone(), out_mean.clone())
            mx_e, arg_e, sm_e = step()
            torch.cuda.synchronize()
            assert torch.equal(got[0], mx_e) and torch.equal(got[1], arg_e), i
            assert torch.equal(got[2], sm_e) and torch.equal(got[3], out_mean), i


def test_segment_csr_under_graph_replay(ts, oracle):
    """Rows that cross tiles are finished inside the kernel through carry flags in the workspace; their
    readers clear them, so replays of a captured launch (same arguments, same workspace) stay correct.
    Three replays with fresh inputs and eager work in between, each checked."""
    g = torch.Generator().manual_seed(11)
    deg = torch.randint(0, 40, (3000,), generator=g)
    deg[100] = 9000  # a row that spans several tiles
    indptr = torch.cat([torch.zeros(1, dtype=torch.long), deg.cumsum(0)])
    E = int(indptr[-1])
    static_src = torch.zeros(E, 32, device=DEV)
    out_sum = torch.empty(3000, 32, device=DEV)
    out_max = torch.empty(3000, 32, device=DEV)
    dptr = indptr.to(DEV)
    for _ in range(2):  # warm-up outside the capture
        ts.segment_sum_csr(static_src, dptr, out_sum)
        ts.segment_max_csr(static_src, dptr, out_max)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ts.segment_sum_csr(static_src, dptr, out_sum)
        arg = ts.segment_max_csr(static_src, dptr, out_max)[1]
    for rep in range(3):
        src = torch.randn(E, 32, generator=g)
        static_src.copy_(src.to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        want_sum = oracle.segment_csr(src.double(), indptr, None, "sum")[0]
        want_max, want_arg = oracle.segment_csr(src, indptr, None, "max")
        assert torch.allclose(out_sum.cpu().double(), want_sum, rtol=1e-5, atol=1e-3), rep
        assert torch.equal(out_max.cpu(), want_max) and torch.equal(arg.cpu(), want_arg), rep
        # eager work between the replays, through the same operators
        eager = ts.segment_sum_csr(static_src, dptr)
        assert torch.allclose(eager, out_sum, rtol=1e-5, atol=1e-3)


def test_scatter_mean_counts_from_the_index(ts, oracle):
    """scatter_mean with one index per row counts the entries straight from the index (fp32 counts,
    one clamp-cast-divide kernel): same results as the reference's sum / count on the oracle wherever
    its count is exact, floor division for integers, batched [B, E] index, `out=`, and backward."""
    g = torch.Generator().manual_seed(9)
    for dtype in (torch.float32, torch.float64, torch.int32, torch.int64):
        src = (torch.randn(500, 6, generator=g) * 50).to(dtype)
        index = torch.randint(0, 40, (500,), generator=g)
        got = ts.scatter_mean(src.to(DEV), index.to(DEV), 0, None, 45)
        want = oracle.op_scatter(src, index, 0, None, 45, "mean")
        if dtype.is_floating_point:
            assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-5)
        else:
            assert torch.equal(got.cpu(), want)
    # batched index along dim 1, accumulate into a given out (the whole of out is divided, as upstream)
    src = torch.randn(3, 200, 5, generator=g)
    index = torch.randint(0, 9, (3, 200), generator=g)
    prev = torch.randn(3, 9, 5, generator=g)
    out = prev.clone().to(DEV)
    ts.scatter_mean(src.to(DEV), index.to(DEV), 1, out)
    want = oracle.op_scatter(src, index, 1, prev.clone(), None, "mean")
    assert torch.allclose(out.cpu(), want, rtol=1e-5, atol=1e-5)
    # fp16 groups of ~1500 entries (sums of ones stay exact up to 2048 in fp16)
    index = torch.randint(0, 3, (4500,), generator=g)
    got = ts.scatter_mean(torch.ones(4500, 4, dtype=torch.float16, device=DEV), index.to(DEV), 0, None, 4)
    assert torch.equal(got.cpu(), torch.tensor([[1.0] * 4] * 3 + [[0.0] * 4], dtype=torch.float16))
    # backward: grad_out[group] / count
    src = torch.randn(300, 4, generator=g, dtype=torch.double).to(DEV).requires_grad_(True)
    index = torch.randint(0, 20, (300,), generator=g)
    grad = torch.randn(25, 4, generator=g, dtype=torch.double)
    ts.scatter_mean(src, index.to(DEV), 0, None, 25).backward(grad.to(DEV))
    count = torch.bincount(index, minlength=25).clamp(min=1).double()
    assert torch.allclose(src.grad.cpu(), (grad / count.view(-1, 1))[index], rtol=1e-12)


@pytest.mark.parametrize("reduce", ["sum", "mean", "min", "max"])
def test_segment_csr_row_pointers_that_start_behind_zero(ts, reduce):
    """indptr[0] > 0 and indptr[-1] < E: only [indptr[n], indptr[n+1]) is reduced
    (csrc/cuda/segment_csr_cuda.cu:30-33); forward and backward against the oracle."""
    import ts_oracle
    rng = np.random.default_rng(91)
    n, K, front, back = 700, 64, 41, 17
    deg = np.minimum(rng.zipf(1.7, size=n), 3000)
    indptr = torch.from_numpy(np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)) + front
    E = int(indptr[-1]) + back
    src = random_values(rng, (E, K), torch.float32, ties=reduce in ("min", "max"))
    want, want_arg = ts_oracle.segment_csr(src, indptr, None, reduce)
    x = src.to(DEV).requires_grad_()
    got = ts.segment_csr(x, indptr.to(DEV), None, reduce)
    if reduce in ("min", "max"):
        assert torch.equal(got.detach().cpu(), want)
    else:
        scale = float(ts_oracle.segment_csr(src.abs(), indptr, None, "sum")[0].max())
        assert bool(((got.detach().cpu() - want).abs() <= 1e-5 * want.abs() + 1e-5 * scale).all())
    g = torch.from_numpy(rng.standard_normal((n, K)).astype(np.float32))
    got.backward(g.to(DEV))
    grad = x.grad.cpu()
    # entries outside the window take no part; the reference's sum / mean backward gathers into torch::empty
    # (csrc/segment_csr.cpp:70-78, 94-111) and so defines the gradient inside the window only
    inner = indptr - front
    if reduce == "sum":
        assert torch.equal(grad[front:E - back], ts_oracle.gather_csr(g, inner))
    elif reduce == "mean":
        assert torch.equal(grad[front:E - back], ts_oracle.segment_mean_csr_backward(g, inner, (E - front - back, K)))
    else:
        assert torch.equal(grad, ts_oracle.arg_backward(g, want_arg, (E, K), 0))


@pytest.mark.parametrize("reduce", ["sum", "mean", "max"])
def test_scatter_along_the_last_dim_of_100000_rows(ts, reduce):
    """More leading rows than a grid dimension holds: src [100000, 16], dim = -1 (the reference's default)."""
    import ts_oracle
    rng = np.random.default_rng(92)
    src = random_values(rng, (100000, 16), torch.float32, ties=reduce == "max")
    index = torch.from_numpy(rng.integers(0, 6, size=(100000, 16)).astype(np.int64))
    want = ts_oracle.op_scatter(src, index, -1, None, 6, reduce)
    got = ts.scatter(src.to(DEV), index.to(DEV), -1, None, 6, reduce)
    if reduce == "max":
        assert torch.equal(got.cpu(), want[0])
        arg = ts.scatter_max(src.to(DEV), index.to(DEV), -1, None, 6)[1]
        assert torch.equal(arg.cpu(), ts_oracle.scatter(src, index, 1, None, 6, "max")[1])
    else:
        assert bool(((got.cpu() - want).abs() <= 1e-5 * want.abs() + 1e-5 * float(src.abs().sum(1).max())).all())


def test_segment_csr_with_100000_leading_rows(ts):
    import ts_oracle
    rng = np.random.default_rng(93)
    B, n, E, K = 100000, 2, 5, 4
    cut = rng.integers(0, E + 1, size=B)
    indptr = torch.from_numpy(np.stack([np.zeros(B, np.int64), cut, np.full(B, E)], 1).astype(np.int64))
    src = random_values(rng, (B, E, K), torch.float32, ties=True)
    got, arg = ts.segment_max_csr(src.to(DEV), indptr.to(DEV))
    want, want_arg = ts_oracle.segment_csr(src, indptr, None, "max")
    assert torch.equal(got.cpu(), want) and torch.equal(arg.cpu(), want_arg)
    assert torch.equal(ts.gather_csr(got, indptr.to(DEV)).cpu(), ts_oracle.gather_csr(want, indptr))


@pytest.mark.parametrize("reduce", ["sum", "mean", "min", "max"])
def test_scatter_large_sorted_index_through_the_operators(ts, oracle, reduce):
    """77 MB of 128-byte rows under a sorted index with gaps: above the sizes from which the operators hand the
    scatter kernels a workspace, where the count pass of the buckets finds the index in order and the segmented
    reduction finishes the call. Same results as the oracle (sums in another order of additions), -inf entries
    and empty rows included, and the backward through arg / the index. The same index with two entries swapped
    goes through the buckets and gives the same values."""
    g = torch.Generator().manual_seed(11)
    E, K, N = 600_000, 32, 20_000
    index = torch.sort(torch.randint(0, N // 2, (E,), generator=g) * 2)[0]
    src = torch.randint(-8, 9, (E, K), generator=g).float()
    src[::13, ::5] = float("-inf") if reduce == "max" else (float("inf") if reduce == "min" else 1.0)
    want = oracle.op_scatter(src, index, 0, None, N, reduce)
    for swapped in (False, True):
        idx = index.clone()
        s = src
        if swapped:
            # the two entries change places together with their rows: the same scatter, no longer in order
            i, j = E // 2, E // 2 + 40
            perm = torch.arange(E)
            perm[i], perm[j] = j, i
            idx, s = index[perm], src[perm]
        x = s.to(DEV).requires_grad_(reduce in ("sum", "mean"))
        got = getattr(ts, "scatter_" + reduce)(x, idx.to(DEV), 0, None, N)
        if reduce in ("min", "max"):
            assert torch.equal(got[0].cpu(), want[0]), swapped
            if not swapped:
                assert torch.equal(got[1].cpu(), want[1])
            else:  # positions follow the entries that changed places
                ref = want[1].clone()
                ref[want[1] == i], ref[want[1] == j] = j, i
                assert torch.equal(got[1].cpu(), ref)
        else:
            assert torch.allclose(got.detach().cpu(), want, rtol=1e-5, atol=1e-4), swapped
            grad = torch.randn(N, K, generator=g)
            got.backward(grad.to(DEV))
            count = torch.bincount(idx, minlength=N).clamp(min=1).float().view(-1, 1)
            expect = (grad / count if reduce == "mean" else grad)[idx]
            assert torch.allclose(x.grad.cpu(), expect, rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("dtype,K", product([torch.int8, torch.uint8, torch.int16], [1, 6]))
def test_scatter_sum_of_narrow_integers_under_a_hub(ts, dtype, K):
    """8- and 16-bit integer sums run in int32 and are cast back: the result wraps like the narrow type's own
    arithmetic (what the reference's atomAdd on these types gives), also on top of previous content in `out`,
    and a row that takes a third of the entries does not take longer than the rest."""
    g = torch.Generator().manual_seed(3)
    E, N = 60000, 500
    index = torch.where(torch.rand(E, generator=g) < 0.3, torch.tensor(7), torch.randint(0, N, (E,), generator=g))
    src = torch.randint(0, 100, (E, K), generator=g).to(dtype)
    prev = torch.randint(0, 50, (N, K), generator=g).to(dtype)
    want = torch.zeros((N, K), dtype=torch.int64).index_add_(0, index, src.long())
    got = ts.scatter(src.to(DEV), index.to(DEV), 0, None, N, "sum")
    assert got.dtype == dtype and torch.equal(got.cpu(), want.to(dtype))
    out = prev.clone().to(DEV)
    res = ts.scatter(src.to(DEV), index.to(DEV), 0, out, None, "sum")
    assert res.data_ptr() == out.data_ptr()
    assert torch.equal(out.cpu(), (want + prev.long()).to(dtype))
    mean = ts.scatter(src.to(DEV), index.to(DEV), 0, None, N, "mean")
    count = torch.bincount(index, minlength=N).clamp(min=1).to(dtype).view(N, 1)
    assert torch.equal(mean.cpu(), torch.div(want.to(dtype), count, rounding_mode="floor"))


@pytest.mark.parametrize("dtype,K,E", product([torch.float32, torch.float64, torch.int32, torch.int64], [1, 5, 100],
                                              [30000, 200_000]))
def test_scatter_mul_under_a_hub(ts, dtype, K, E):
    """Products of a row that takes a third of the entries: below 2^16 elements the lanes of a wavefront combine
    before the compare-and-swap in memory, above the factors of a row meet in the table in LDS; the result is the
    product whatever the order."""
    g = torch.Generator().manual_seed(4)
    N = 300
    if E * K > 4_000_000:
        pytest.skip("covered by the smaller input")
    index = torch.where(torch.rand(E, generator=g) < 0.3, torch.tensor(11), torch.randint(0, N, (E,), generator=g))
    integer = not dtype.is_floating_point
    if integer:
        # a factor of 3 now and then (at most 3^39 per row: fits 64 bits), signs at random
        src = torch.where(torch.rand((E, K), generator=g) < 0.01 * 30000 / E, 3, 1).to(dtype) * \
            torch.where(torch.rand((E, K), generator=g) < 0.5, 1, -1).to(dtype)
    else:
        src = (torch.rand((E, K), generator=g, dtype=torch.float64) * (600.0 / E) + (1 - 300.0 / E)).to(dtype)
    for out_given in (False, True):
        prev = torch.where(torch.rand((N, K), generator=g) < 0.5, 2, -1).to(dtype)
        out = prev.clone().to(DEV) if out_given else None
        got = ts.scatter(src.to(DEV), index.to(DEV), 0, out, None if out_given else N, "mul").cpu()
        start = prev.double() if out_given else torch.ones((N, K), dtype=torch.float64)
        want = start.scatter_reduce(0, index.view(E, 1).expand(E, K), src.double(), "prod")
        if integer:
            start64 = prev.long() if out_given else torch.ones((N, K), dtype=torch.int64)
            wrapped = start64.scatter_reduce(0, index.view(E, 1).expand(E, K), src.long(), "prod")
            assert torch.equal(got.long(), wrapped.to(dtype).long())
        else:
            assert torch.allclose(got.double(), want, rtol=1e-4 if dtype == torch.float32 else 1e-11)


@pytest.mark.parametrize("dtype", [torch.float32, torch.int64])
def test_scatter_mean_with_one_index_row_for_every_batch_row(ts, dtype):
    """An index row expanded over the batch rows (stride 0) is counted once; the result is that of the same index
    written out per batch row, forward and backward."""
    g = torch.Generator().manual_seed(8)
    B, E, N = 37, 500, 23
    row = torch.randint(0, N - 2, (E,), generator=g)
    src = torch.randn((B, E), generator=g).mul(10).to(dtype)
    shared = row.view(1, E).expand(B, E)
    a = ts.scatter(src.to(DEV), shared.to(DEV).expand(B, E), 1, None, N, "mean")
    b = ts.scatter(src.to(DEV), shared.contiguous().to(DEV), 1, None, N, "mean")
    # float sums come from atomics in whatever order; the counts, and with them the integer means, are exact
    assert torch.allclose(a, b, rtol=1e-5, atol=1e-5) if dtype.is_floating_point else torch.equal(a, b)
    if dtype.is_floating_point:
        x = src.to(DEV).requires_grad_(True)
        y = ts.scatter(x, row.to(DEV).view(1, E).expand(B, E), 1, None, N, "mean")
        (gx,) = torch.autograd.grad(y, x, torch.ones_like(y))
        count = torch.bincount(row, minlength=N).clamp(min=1).float()
        assert torch.allclose(gx.cpu(), (1.0 / count)[row].view(1, E).expand(B, E))


@pytest.mark.parametrize("reduce", ["min", "max"])
def test_scatter_of_single_values_with_a_changing_number_of_output_rows(ts, oracle, reduce):
    """Mini-batches with a varying node count on one stream: the operator keeps one workspace per stream for
    min / max of one 4-byte value per entry, and what a call with few output rows leaves behind its key table
    must not be read as keys by a later call with more output rows."""
    rng = np.random.default_rng(11)
    E = 300_000
    for step, N in enumerate([100_000, 50_000, 100_000, 7, 524_288, 50_001, 100_000]):
        src = torch.from_numpy(rng.integers(-50, 51, size=E).astype(np.float32))
        index = torch.from_numpy(rng.integers(0, N, size=E).astype(np.int64))
        got, arg = getattr(ts, "scatter_" + reduce)(src.to(DEV), index.to(DEV), 0, None, N)
        want, want_arg = oracle.scatter(src, index, 0, None, N, reduce)
        assert torch.equal(got.cpu(), want), f"values step={step} N={N}"
        assert torch.equal(arg.cpu(), want_arg), f"arg step={step} N={N}"


def test_operators_raise_when_a_row_was_given_up(ts):
    """TS_CHECK_STATUS=1 (set for the whole test run): after a segment reduction the operators read the two status
    words back and raise if a row that crosses tiles was given up. The give-up is forced from the host on
    well-formed row pointers (TS_CSR_SPIN=-1: no tile waits for another, every kernel exits normally); without
    the override the same call returns the sums."""
    import os
    K = 64
    indptr = torch.tensor([0, 200, 5000, 9000], device=DEV)      # rows of thousands of entries cross tiles
    src = torch.randn((9000, K), device=DEV)
    old = os.environ.get("TS_CSR_SPIN")
    os.environ["TS_CSR_SPIN"] = "-1"
    try:
        with pytest.raises(RuntimeError, match="given up"):
            ts.segment_csr(src, indptr, None, "sum")
        with pytest.raises(RuntimeError, match="given up"):
            ts.segment_coo(src, torch.repeat_interleave(torch.arange(3, device=DEV), indptr[1:] - indptr[:-1]), None, 3, "sum")
    finally:
        if old is None:
            del os.environ["TS_CSR_SPIN"]
        else:
            os.environ["TS_CSR_SPIN"] = old
    out = ts.segment_csr(src, indptr, None, "sum")
    assert torch.allclose(out[1], src[200:5000].double().sum(0).float(), rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("kind", ["uniform", "zipf", "sorted"])
def test_scatter_mean_of_single_values_counts_with_the_sum(kind):
    """scatter_mean of one float per entry at a size where the value buckets take the sum: sum and count come from
    one call (torch_ops.cpp: scatter_hip with mean_count). Values, gradient, and an integer input."""
    import pytorch_scatter_amd as ts
    g = torch.Generator().manual_seed(5)
    E, N = (1 << 21) + 1234, 300_000
    if kind == "zipf":
        w = torch.arange(1, N + 1, dtype=torch.float64) ** -1.1
        index = torch.multinomial(w, E, replacement=True, generator=g)
    else:
        index = torch.randint(0, N, (E,), generator=g)
    if kind == "sorted":
        index = index.sort().values
    index = index.to(DEV)
    src = torch.randn((E,), generator=g).to(DEV).requires_grad_(True)
    out = ts.scatter_mean(src, index, 0, None, N)
    cnt = torch.bincount(index, minlength=N).clamp(min=1).double()
    want = torch.zeros(N, dtype=torch.float64, device=DEV).index_add_(0, index, src.detach().double()) / cnt
    mags = torch.zeros(N, dtype=torch.float64, device=DEV).index_add_(0, index, src.detach().double().abs()) / cnt
    assert bool(((out.double() - want).abs() <= 1e-5 * (want.abs() + mags)).all())
    grad_out = torch.randn((N,), generator=g).to(DEV)
    (grad,) = torch.autograd.grad(out, src, grad_out)
    assert torch.allclose(grad.double(), (grad_out.double() / cnt)[index], rtol=1e-6, atol=0)
    isrc = torch.randint(-50, 50, (E,), generator=g, dtype=torch.int32).to(DEV)
    iout = ts.scatter_mean(isrc, index, 0, None, N)
    isum = torch.zeros(N, dtype=torch.int64, device=DEV).index_add_(0, index, isrc.long())
    assert torch.equal(iout.long(), torch.div(isum, cnt.long(), rounding_mode="floor"))
