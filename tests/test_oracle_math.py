"""The CPU oracle against what the mathematics and library routines fix:
torch equivalents, closed forms, brute force on tiny inputs, and the 16-bit
float conversions against torch's own."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import random_csr, random_values


def test_half_and_bf16_conversions_match_torch(oracle):
    # every binary16 pattern -> float, and a float sweep -> binary16 / bfloat16
    import subprocess, os, tempfile
    here = os.path.dirname(os.path.abspath(oracle.__file__))
    src = r'''
    #include "ts_oracle_types.h"
    void h2f(const uint16_t*a, float*o, long n){for(long i=0;i<n;i++){tso_half h; h.x=a[i]; o[i]=tso_half_to_float(h);}}
    void f2h(const float*a, uint16_t*o, long n){for(long i=0;i<n;i++) o[i]=tso_float_to_half(a[i]).x;}
    void f2b(const float*a, uint16_t*o, long n){for(long i=0;i<n;i++) o[i]=tso_float_to_bf16(a[i]).x;}
    '''
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "conv.c")
        so = os.path.join(d, "conv.so")
        open(c, "w").write(src)
        subprocess.check_call(["gcc", "-O2", "-shared", "-fPIC", "-I", here, c, "-o", so])
        lib = ctypes.CDLL(so)
        pats = np.arange(65536, dtype=np.uint16)
        out = np.empty(65536, dtype=np.float32)
        lib.h2f(pats.ctypes.data_as(ctypes.c_void_p), out.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(65536))
        want = torch.from_numpy(pats.view(np.int16)).view(torch.half).float().numpy()
        nan = np.isnan(want)  # signalling-NaN payloads are quieted by hardware converts: compare as NaN
        assert np.array_equal(np.isnan(out), nan)
        assert np.array_equal(out.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
        rng = np.random.default_rng(0)
        bits = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
        # add values around every half rounding boundary
        halfs = torch.from_numpy(pats.view(np.int16)).view(torch.half).float().numpy()
        near = np.concatenate([np.nextafter(halfs, np.inf), np.nextafter(halfs, -np.inf), halfs,
                               (halfs.astype(np.float64) * (1 + 2.0**-11)).astype(np.float32)])
        f = np.concatenate([bits.view(np.float32), near.astype(np.float32)])
        f = f[~np.isnan(f)]
        n = f.size
        got = np.empty(n, dtype=np.uint16)
        lib.f2h(f.ctypes.data_as(ctypes.c_void_p), got.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(n))
        want = torch.from_numpy(f).half().view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(got, want)
        lib.f2b(f.ctypes.data_as(ctypes.c_void_p), got.ctypes.data_as(ctypes.c_void_p), ctypes.c_long(n))
        want = torch.from_numpy(f).bfloat16().view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("dtype", [torch.float, torch.double, torch.long, torch.int])
def test_scatter_sum_equals_scatter_add(oracle, dtype):
    rng = np.random.default_rng(1)
    src = random_values(rng, (300, 7), dtype)
    index = torch.from_numpy(rng.integers(0, 40, size=300))
    got = oracle.op_scatter(src, index, 0, None, 40, "sum")
    want = torch.zeros(40, 7, dtype=dtype).index_add_(0, index, src)
    assert torch.equal(got, want)


@pytest.mark.parametrize("reduce,torch_reduce", [("max", "amax"), ("min", "amin")])
def test_scatter_minmax_equals_scatter_reduce(oracle, reduce, torch_reduce):
    rng = np.random.default_rng(2)
    src = random_values(rng, (4, 200, 5), torch.float, ties=False)
    index = torch.from_numpy(rng.integers(0, 30, size=(4, 200, 5)))
    got, arg = oracle.op_scatter(src, index, 1, None, 33, reduce)
    want = torch.zeros(4, 33, 5).scatter_reduce_(1, index, src, torch_reduce, include_self=False)
    assert torch.equal(got, want)
    # arg invariants: points at an element of the slot holding the value
    filled = arg < 200
    picked = torch.gather(src, 1, arg.clamp(max=199))
    assert torch.equal(picked[filled], got[filled])
    assert torch.equal(torch.gather(index, 1, arg.clamp(max=199))[filled],
                       torch.arange(33).view(1, 33, 1).expand(4, 33, 5)[filled])
    assert torch.all(got[~filled] == 0)


def _brute_scatter(src, index, dim, N, reduce):
    """Literal (b, e, k) triple loop, first occurrence wins ties."""
    src = src.double()
    shape = list(src.shape)
    shape[dim] = N
    out = [None] * int(np.prod(shape))
    out = np.full(shape, np.nan)
    cnt = np.zeros(shape, dtype=np.int64)
    arg = np.full(shape, src.shape[dim], dtype=np.int64)
    it = np.ndindex(*src.shape)
    for pos in it:
        o = list(pos)
        o[dim] = int(index[pos])
        o = tuple(o)
        v = float(src[pos])
        if cnt[o] == 0:
            out[o] = v
            arg[o] = pos[dim]
        elif reduce in ("sum", "mean"):
            out[o] += v
        elif reduce == "mul":
            out[o] *= v
        elif (reduce == "min" and v < out[o]) or (reduce == "max" and v > out[o]):
            out[o] = v
            arg[o] = pos[dim]
        cnt[o] += 1
    if reduce == "mean":
        out = out / np.maximum(cnt, 1)
    out[cnt == 0] = 1 if reduce == "mul" else 0
    return torch.from_numpy(out), torch.from_numpy(arg)


@pytest.mark.parametrize("reduce", ["sum", "mean", "mul", "min", "max"])
@pytest.mark.parametrize("dim", [0, 1, 2])
def test_scatter_brute_force_with_ties(oracle, reduce, dim):
    rng = np.random.default_rng(3 + dim)
    src = random_values(rng, (3, 9, 4), torch.double)
    if reduce == "mul":
        src = src.clamp(-2, 2)
    index = torch.from_numpy(rng.integers(0, 6, size=(3, 9, 4)))
    N = 7
    got = oracle.op_scatter(src, index, dim, None, N, reduce)
    want, want_arg = _brute_scatter(src, index, dim, N, reduce)
    if isinstance(got, tuple):
        got, arg = got
        assert torch.equal(arg, want_arg)
    assert torch.allclose(got, want, rtol=0, atol=1e-12)


@pytest.mark.parametrize("reduce", ["sum", "mean", "min", "max"])
def test_segment_ops_agree_with_scatter_on_sorted_input(oracle, reduce):
    # the identity the reference's benchmark asserts (benchmark/scatter_segment.py:48-74)
    rng = np.random.default_rng(5)
    indptr, index = random_csr(rng, 50, 9)
    src = random_values(rng, (index.numel(), 6), torch.double)
    a = oracle.op_scatter(src, index, 0, None, 50, reduce)
    b, b2 = oracle.segment_coo(src, index, None, 50, reduce)
    c, c2 = oracle.segment_csr(src, indptr, None, reduce)
    if isinstance(a, tuple):
        a, a2 = a
        assert torch.equal(a2, b2) and torch.equal(a2, c2)
    assert torch.equal(a, b) and torch.equal(a, c)


def test_segment_csr_against_reduceat(oracle):
    rng = np.random.default_rng(6)
    indptr, index = random_csr(rng, 80, 12, p_empty=0.0)
    src = random_values(rng, (index.numel(), 3), torch.double, ties=False)
    starts = indptr[:-1].numpy()
    want_sum = np.add.reduceat(src.numpy(), starts, axis=0)
    want_max = np.maximum.reduceat(src.numpy(), starts, axis=0)
    assert np.allclose(oracle.segment_csr(src, indptr, None, "sum")[0].numpy(), want_sum, rtol=1e-13)
    assert np.array_equal(oracle.segment_csr(src, indptr, None, "max")[0].numpy(), want_max)
    deg = (indptr[1:] - indptr[:-1]).double().unsqueeze(-1)
    assert np.allclose(oracle.segment_csr(src, indptr, None, "mean")[0].numpy(), want_sum / deg.numpy(), rtol=1e-13)


def test_gathers_against_library_routines(oracle):
    rng = np.random.default_rng(7)
    indptr, index = random_csr(rng, 60, 7)
    src = random_values(rng, (60, 5), torch.float, ties=False)
    deg = indptr[1:] - indptr[:-1]
    assert torch.equal(oracle.gather_csr(src, indptr), torch.repeat_interleave(src, deg, dim=0))
    assert torch.equal(oracle.gather_coo(src, index), src.index_select(0, index))


def test_gather_coo_rejects_decreasing_index(oracle):
    src = torch.arange(4.0)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        oracle.gather_coo(src, torch.tensor([0, 2, 1]))


def test_bf16_segment_mean_rounding_order(oracle):
    # fp32 accumulate -> one rounding to bf16 -> divide by the bf16-rounded count
    # (csrc/cpu/segment_csr_cpu.cpp:62-86, csrc/cpu/reducer.h:74-75)
    rng = np.random.default_rng(8)
    deg = np.array([1, 3, 257, 300, 0, 1000])
    indptr = torch.from_numpy(np.concatenate([[0], np.cumsum(deg)]).astype(np.int64))
    src = torch.from_numpy(rng.standard_normal((int(deg.sum()), 4))).bfloat16()
    got = oracle.segment_csr(src, indptr, None, "mean")[0]
    for n, d in enumerate(deg):
        rows = src[indptr[n]:indptr[n + 1]].float()
        acc = torch.zeros(4)
        for r in rows:
            acc = acc + r
        s = acc.bfloat16()
        c = torch.tensor(float(max(d, 1))).bfloat16()
        want = (s.float() / c.float()).bfloat16()
        assert torch.equal(got[n], want), n


def test_mean_backward_closed_form(oracle):
    rng = np.random.default_rng(9)
    indptr, index = random_csr(rng, 30, 6)
    E = index.numel()
    g = random_values(rng, (30, 4), torch.double, ties=False)
    deg = (indptr[1:] - indptr[:-1]).clamp(min=1).double().unsqueeze(-1)
    want = (g / deg).index_select(0, index)
    assert torch.allclose(oracle.segment_mean_csr_backward(g, indptr, (E, 4)), want, rtol=1e-14)
    _, count = oracle.segment_coo(torch.zeros(E, 4, dtype=torch.double), index, None, 30, "mean")
    assert torch.allclose(oracle.segment_mean_coo_backward(g, index, count, (E, 4)), want, rtol=1e-14)


def test_arg_backward_routes_gradient_to_winner(oracle):
    rng = np.random.default_rng(10)
    indptr, index = random_csr(rng, 20, 5)
    E = index.numel()
    src = random_values(rng, (E, 3), torch.double)
    out, arg = oracle.segment_csr(src, indptr, None, "max")
    g = torch.ones(20, 3, dtype=torch.double)
    grad = oracle.arg_backward(g, arg, (E, 3), 0)
    assert grad.shape == (E, 3)
    # one unit of gradient per non-empty slot, none for the sentinel
    assert grad.sum().item() == (arg < E).sum().item()
