"""TEST INFRASTRUCTURE ONLY -- host half of the CPU oracle.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module, and only as the checker or as the timed
CPU baseline. The shipped package never imports it.

The arithmetic lives in ``ts_oracle.c`` (plain C, single thread). This file
restates what the reference's host code does around those loops -- shape
checks, expansion of the index, allocation and initial fill of the outputs --
and the op-level maths of the autograd layer, each function citing the
reference lines it follows. Tensors are ``torch`` CPU tensors used purely as
typed buffers.
"""
import ctypes
import os
import subprocess
from typing import Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libts_oracle.so")

SUM, MEAN, MUL, DIV, MIN, MAX = range(6)
REDUCE = {"sum": SUM, "add": SUM, "mean": MEAN, "mul": MUL, "div": DIV,
          "min": MIN, "max": MAX}

DTYPE = {torch.float32: 0, torch.float64: 1, torch.float16: 2,
         torch.bfloat16: 3, torch.int32: 4, torch.int64: 5, torch.int16: 6,
         torch.int8: 7, torch.uint8: 8}


def build() -> str:
    """Compile libts_oracle.so (always recompiles)."""
    subprocess.check_call(["make", "-B", "-C", _HERE, "libts_oracle.so"],
                          stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in ("tso_scatter", "tso_segment_csr", "tso_gather_csr",
                     "tso_segment_coo", "tso_gather_coo"):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def _p(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(0 if t is None or t.numel() == 0 else t.data_ptr())


def _i64arr(xs):
    return (ctypes.c_int64 * max(len(xs), 1))(*xs)


def _info(t: torch.Tensor):
    return (_p(t), ctypes.c_int(t.dim()), _i64arr(list(t.shape)),
            _i64arr(list(t.stride())))


def _check(cond: bool):
    # CHECK_INPUT, csrc/cpu/utils.h:6
    if not cond:
        raise RuntimeError("Input mismatch")


def _i64(v):
    return ctypes.c_int64(int(v))


def _init_value(dtype: torch.dtype, reduce: int):
    # Reducer::init, csrc/cpu/reducer.h:44-53
    if reduce in (MUL, DIV):
        return 1
    if reduce in (MIN, MAX):
        info = torch.finfo(dtype) if dtype.is_floating_point else torch.iinfo(dtype)
        return info.max if reduce == MIN else info.min
    return 0


def broadcast(index: torch.Tensor, other: torch.Tensor, dim: int) -> torch.Tensor:
    """csrc/scatter.cpp:25-33."""
    if index.dim() == 1:
        for _ in range(dim):
            index = index.unsqueeze(0)
    for _ in range(index.dim(), other.dim()):
        index = index.unsqueeze(-1)
    return index.expand(list(other.shape))


# --------------------------------------------------------------------- scatter
def scatter(src, index, dim, out=None, dim_size=None, reduce="sum"
            ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """scatter_cpu, csrc/cpu/scatter_cpu.cpp:7-87 (index already broadcast)."""
    r = REDUCE[reduce]
    _check(src.dim() == index.dim())
    for i in range(index.dim() - 1):
        _check(src.size(i) >= index.size(i))
    src = src.contiguous()
    out_given = out is not None
    if out_given:
        out = out.contiguous()
        for i in range(out.dim()):
            if i != dim:
                _check(src.size(i) == out.size(i))
    else:
        sizes = list(src.shape)
        if dim_size is not None:
            sizes[dim] = dim_size
        elif index.numel() == 0:
            sizes[dim] = 0
        else:
            sizes[dim] = 1 + int(index.max())
        out = torch.empty(sizes, dtype=src.dtype)
    arg_out = None
    if r in (MIN, MAX):
        arg_out = torch.full_like(out, src.size(dim), dtype=torch.int64)
    if src.numel() == 0:
        if not out_given:
            out.fill_(0)
        return out, arg_out
    B = 1
    for i in range(dim):
        B *= src.size(i)
    E = src.size(dim)
    K = src.numel() // (B * E)
    N = out.size(dim)
    rc = lib().tso_scatter(_p(src), *_info(index), _p(out), _p(arg_out),
                           _i64(B), _i64(E), _i64(K), _i64(N),
                           DTYPE[src.dtype], r, int(out_given))
    assert rc == 0, rc
    return out, arg_out


def op_scatter(src, index, dim=-1, out=None, dim_size=None, reduce="sum"):
    """Forward of the registered scatter ops, csrc/scatter.cpp:54-233.

    Returns ``out`` for sum/mul/mean and ``(out, arg_out)`` for min/max.
    """
    r = REDUCE[reduce]
    dim = src.dim() + dim if dim < 0 else dim
    if r != MEAN:
        res = scatter(src, broadcast(index, src, dim), dim, out, dim_size, reduce)
        return res if r in (MIN, MAX) else res[0]
    # ScatterMean::forward, csrc/scatter.cpp:117-146
    old_index = index
    out, _ = scatter(src, broadcast(index, src, dim), dim, out, dim_size, "sum")
    ones = torch.ones(list(old_index.shape), dtype=src.dtype)
    cdim = old_index.dim() - 1 if old_index.dim() <= dim else dim
    count, _ = scatter(ones, old_index, cdim, None, out.size(dim), "sum")
    count.masked_fill_(count < 1, 1)
    count = broadcast(count, out, dim)
    if out.is_floating_point():
        out.true_divide_(count)
    else:
        out.div_(count, rounding_mode="floor")
    return out


# ----------------------------------------------------------------- segment_csr
def _expand_indptr(src, indptr):
    sizes = list(indptr.shape)
    for i in range(indptr.dim() - 1):
        sizes[i] = src.size(i)
    return indptr.expand(sizes)


def segment_csr(src, indptr, out=None, reduce="sum"
                ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """segment_csr_cpu, csrc/cpu/segment_csr_cpu.cpp:8-92."""
    r = REDUCE[reduce]
    _check(src.dim() >= indptr.dim())
    indptr = _expand_indptr(src, indptr)
    dim = indptr.dim() - 1
    src = src.contiguous()
    out_given = out is not None
    if out_given:
        out = out.contiguous()
        for i in range(out.dim()):
            if i != dim:
                _check(src.size(i) == out.size(i))
        _check(src.numel() == 0 or out.size(dim) == indptr.size(dim) - 1)
    else:
        sizes = list(src.shape)
        sizes[dim] = max(indptr.size(dim) - 1, 0)
        out = torch.empty(sizes, dtype=src.dtype)
    arg_out = None
    if r in (MIN, MAX):
        arg_out = torch.full(list(out.shape), src.size(dim), dtype=torch.int64)
    if src.numel() == 0:
        if not out_given:
            out.fill_(0)
        return out, arg_out
    N = out.size(dim) * (indptr.numel() // indptr.size(-1))
    K = out.numel() // N
    E = src.size(dim)
    rc = lib().tso_segment_csr(_p(src), *_info(indptr), _p(out), _p(arg_out),
                               _i64(N), _i64(K), _i64(E), DTYPE[src.dtype], r)
    assert rc == 0, rc
    return out, arg_out


def gather_csr(src, indptr, out=None) -> torch.Tensor:
    """gather_csr_cpu, csrc/cpu/segment_csr_cpu.cpp:94-162."""
    _check(src.dim() >= indptr.dim())
    indptr = _expand_indptr(src, indptr)
    dim = indptr.dim() - 1
    _check(src.size(dim) == 0 or src.size(dim) == indptr.size(dim) - 1)
    src = src.contiguous()
    out_given = out is not None
    if out_given:
        out = out.contiguous()
        for i in range(out.dim()):
            if i != dim:
                _check(src.size(i) == out.size(i))
    else:
        sizes = list(src.shape)
        sizes[dim] = int(indptr.flatten()[-1]) if src.numel() > 0 else 0
        out = torch.empty(sizes, dtype=src.dtype)
    if src.numel() == 0:
        if not out_given:
            out.fill_(0)
        return out
    N = src.size(dim) * (indptr.numel() // indptr.size(-1))
    K = src.numel() // N
    E = out.size(dim)
    rc = lib().tso_gather_csr(_p(src), *_info(indptr), _p(out), _i64(N),
                              _i64(K), _i64(E), DTYPE[src.dtype])
    assert rc == 0, rc
    return out


# ----------------------------------------------------------------- segment_coo
def segment_coo(src, index, out=None, dim_size=None, reduce="sum"
                ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """segment_coo_cpu, csrc/cpu/segment_coo_cpu.cpp:8-141.

    Second result: arg_out (min/max), count (mean) or None (sum).
    """
    r = REDUCE[reduce]
    _check(src.dim() >= index.dim())
    sizes = list(index.shape)
    for i in range(index.dim()):
        sizes[i] = src.size(i)
    index = index.expand(sizes)
    dim = index.dim() - 1
    src = src.contiguous()
    out_given = out is not None
    if out_given:
        out = out.contiguous()
        for i in range(out.dim()):
            if i != dim:
                _check(src.size(i) == out.size(i))
    else:
        sizes = list(src.shape)
        if dim_size is not None:
            sizes[dim] = dim_size
        elif index.numel() == 0:
            sizes[dim] = 0
        else:
            sizes[dim] = 1 + int(index.select(dim, index.size(dim) - 1).max())
        out = torch.empty(sizes, dtype=src.dtype)
    second = None
    if r in (MIN, MAX):
        second = torch.full_like(out, src.size(dim), dtype=torch.int64)
    elif r == MEAN:
        sizes = list(index.shape)
        sizes[dim] = out.size(dim)
        second = torch.zeros(sizes, dtype=out.dtype)
    if src.numel() == 0:
        if not out_given:
            out.fill_(0)
        return out, second
    B = index.numel() // src.size(dim)
    E = src.size(dim)
    K = src.numel() // index.numel()
    N = out.size(dim)
    rc = lib().tso_segment_coo(_p(src), *_info(index), _p(out), _p(second),
                               _i64(B), _i64(E), _i64(K), _i64(N),
                               DTYPE[src.dtype], r, int(out_given))
    assert rc == 0, rc
    return out, second


def gather_coo(src, index, out=None) -> torch.Tensor:
    """gather_coo_cpu, csrc/cpu/segment_coo_cpu.cpp:143-215."""
    _check(src.dim() >= index.dim())
    for i in range(index.dim() - 1):
        _check(src.size(i) == index.size(i))
    dim = index.dim() - 1
    src = src.contiguous()
    out_given = out is not None
    if out_given:
        out = out.contiguous()
        for i in range(src.dim()):
            if i != dim:
                _check(src.size(i) == out.size(i))
    else:
        sizes = list(src.shape)
        sizes[dim] = index.size(dim)
        out = torch.empty(sizes, dtype=src.dtype)
    if src.numel() == 0:
        if not out_given:
            out.fill_(0)
        return out
    B = index.numel() // out.size(dim)
    E = index.size(dim)
    K = out.numel() // index.numel()
    N = src.size(dim)
    rc = lib().tso_gather_coo(_p(src), *_info(index), _p(out), _i64(B), _i64(E),
                              _i64(K), _i64(N), DTYPE[src.dtype])
    _check(rc == 0)
    return out


# ------------------------------------------------------ backward closed forms
def arg_backward(grad_out, arg_out, src_shape, dim):
    """min/max backward: csrc/scatter.cpp:184-196, segment_coo.cpp:132-144,
    segment_csr.cpp:130-142 -- scatter into a buffer with one extra slot that
    swallows the sentinel, then drop that slot."""
    shape = list(src_shape)
    shape[dim] += 1
    grad_in = torch.zeros(shape, dtype=grad_out.dtype)
    grad_in.scatter_(dim, arg_out, grad_out)
    return grad_in.narrow(dim, 0, shape[dim] - 1)


def segment_mean_csr_backward(grad_out, indptr, src_shape):
    """SegmentMeanCSR::backward, csrc/segment_csr.cpp:94-111."""
    grad_in = torch.empty(list(src_shape), dtype=grad_out.dtype)
    if grad_in.numel() > 0:
        gather_csr(grad_out, indptr, grad_in)
        count = (indptr.narrow(-1, 1, indptr.size(-1) - 1)
                 - indptr.narrow(-1, 0, indptr.size(-1) - 1)).to(grad_in.dtype)
        count = gather_csr(count, indptr, None)
        for _ in range(grad_out.dim() - indptr.dim()):
            count = count.unsqueeze(-1)
        grad_in.true_divide_(count)
    return grad_in


def segment_mean_coo_backward(grad_out, index, count, src_shape):
    """SegmentMeanCOO::backward, csrc/segment_coo.cpp:99-112."""
    grad_in = torch.empty(list(src_shape), dtype=grad_out.dtype)
    gather_coo(grad_out, index, grad_in)
    count = gather_coo(count, index, None)
    for _ in range(grad_out.dim() - index.dim()):
        count = count.unsqueeze(-1)
    grad_in.true_divide_(count)
    return grad_in


# ------------------------------------------------- group statistics (Python layer)
# The reference composes these in Python from scatter_max / scatter_sum, gather
# and ATen elementwise ops; the same sequence here, on the oracle's scatter.
# Pinned by the reference's own checks (test/composite/test_softmax.py:6-54,
# test_logsumexp.py:5-45, test_std.py:5-20: per-group torch.softmax /
# log_softmax / logsumexp / std) in tests/test_oracle_golden.py.
def _py_broadcast(index, other, dim):
    """torch_scatter/utils.py:4-13."""
    dim = other.dim() + dim if dim < 0 else dim
    return broadcast(index, other, dim), dim


def scatter_softmax(src, index, dim=-1, dim_size=None):
    """torch_scatter/composite/softmax.py:8-29."""
    index, dim = _py_broadcast(index, src, dim)
    group_max = scatter(src, index, dim, None, dim_size, "max")[0]
    e = (src - group_max.gather(dim, index)).exp_()
    total = scatter(e, index, dim, None, dim_size, "sum")[0]
    return e.div(total.gather(dim, index))


def scatter_log_softmax(src, index, dim=-1, eps=1e-12, dim_size=None):
    """torch_scatter/composite/softmax.py:32-59."""
    index, dim = _py_broadcast(index, src, dim)
    group_max = scatter(src, index, dim, None, dim_size, "max")[0]
    z = src - group_max.gather(dim, index)
    total = scatter(z.exp(), index, dim, None, dim_size, "sum")[0]
    return z.sub_(total.add_(eps).log_().gather(dim, index))


def scatter_logsumexp(src, index, dim=-1, out=None, dim_size=None, eps=1e-12):
    """torch_scatter/composite/logsumexp.py:8-57."""
    index, dim = _py_broadcast(index, src, dim)
    if out is not None:
        dim_size = out.size(dim)
    elif dim_size is None:
        dim_size = int(index.max()) + 1
    size = list(src.shape)
    size[dim] = dim_size
    group_max = torch.full(size, float("-inf"), dtype=src.dtype)
    scatter(src, index, dim, group_max, dim_size, "max")
    z = src - group_max.gather(dim, index)
    z.masked_fill_(torch.isnan(z), float("-inf"))
    orig = None
    if out is not None:
        orig = out.clone()
        out = out.sub_(group_max).exp_()
    total = scatter(z.exp_(), index, dim, out, dim_size, "sum")[0]
    res = total.add_(eps).log_().add_(group_max)
    if orig is None:
        return res.nan_to_num_(neginf=0.0)
    mask = ~res.isfinite()
    res[mask] = orig[mask]
    return res


def scatter_std(src, index, dim=-1, out=None, dim_size=None, unbiased=True):
    """torch_scatter/composite/std.py:8-41."""
    if out is not None:
        dim_size = out.size(dim)
    dim = src.dim() + dim if dim < 0 else dim
    count_dim = index.dim() - 1 if index.dim() <= dim else dim
    ones = torch.ones(list(index.shape), dtype=src.dtype)
    count = scatter(ones, index, count_dim, None, dim_size, "sum")[0]
    index = broadcast(index, src, dim)
    total = scatter(src, index, dim, None, dim_size, "sum")[0]
    count = broadcast(count, total, dim).clamp(1)
    mean = total.div(count)
    dev = src - mean.gather(dim, index)
    sq = scatter(dev * dev, index, dim, out, dim_size, "sum")[0]
    if unbiased:
        count = count.sub(1).clamp_(1)
    return sq.div(count + 1e-6).sqrt()


def scatter_std_backward(src, grad_out, index, dim=-1, dim_size=None, unbiased=True):
    """What autograd derives for scatter_std above: the same sequence
    (composite/std.py:19-41) on differentiable torch ops (index_add for the
    sums), differentiated by torch. Returns (std, grad_src). A group whose std is 0
    gets NaN, from the derivative of sqrt at 0."""
    index, dim = _py_broadcast(index, src, dim)
    if dim_size is None:
        dim_size = int(index.max()) + 1
    x = src.detach().clone().requires_grad_(True)
    shape = list(x.shape)
    shape[dim] = dim_size

    def group_sum(v):
        return torch.zeros(shape, dtype=v.dtype).scatter_add(dim, index, v)

    count = group_sum(torch.ones_like(x)).clamp(1)
    dev = x - (group_sum(x) / count).gather(dim, index)
    sq = group_sum(dev * dev)
    if unbiased:
        count = count.sub(1).clamp(1)
    std = (sq / (count + 1e-6)).sqrt()
    grad, = torch.autograd.grad(std, x, grad_out)
    return std.detach(), grad


def scatter_softmax_backward(result, grad_out, index, dim=-1, dim_size=None, log_space=False):
    """What autograd derives for the two functions above (closed form; the
    reference has no explicit backward, it differentiates through its ops):
    softmax: y * (g - sum_group(y * g)); log_softmax: g - exp(y) * sum_group(g)."""
    index, dim = _py_broadcast(index, result, dim)
    if dim_size is None:
        dim_size = int(index.max()) + 1
    if log_space:
        total = scatter(grad_out, index, dim, None, dim_size, "sum")[0]
        return grad_out - result.exp() * total.gather(dim, index)
    total = scatter(result * grad_out, index, dim, None, dim_size, "sum")[0]
    return result * (grad_out - total.gather(dim, index))


def scatter_logsumexp_backward(src, result, grad_out, index, dim=-1):
    """What autograd derives for scatter_logsumexp above (closed form):
    grad_out[group] * exp(src - result[group]); entries that dropped out of the
    forward sum (NaN) get 0."""
    index, dim = _py_broadcast(index, src, dim)
    w = (src - result.gather(dim, index)).exp()
    w = torch.where(torch.isnan(w), torch.zeros_like(w), w)
    return grad_out.gather(dim, index) * w


# ---- index formats. The reference has no routine for these steps (its benchmark reads
# row and rowptr from the same scipy matrix, benchmark/scatter_segment.py:38-41); the
# definitions are restated with plain loops so that tests can pin them against
# numpy / scipy library routines.
def index_to_indptr(index, dim_size):
    """indptr[r] = number of entries with index < r (1-D sorted index)."""
    ptr = [0] * (dim_size + 1)
    for v in index.tolist():
        for r in range(max(v + 1, 0), dim_size + 1):
            ptr[r] += 1
    return torch.tensor(ptr, dtype=torch.long)


def indptr_to_index(indptr):
    out = []
    p = indptr.tolist()
    for r in range(len(p) - 1):
        out.extend([r] * (p[r + 1] - p[r]))
    return torch.tensor(out, dtype=torch.long)


def sort_index(index, dim_size):
    """Stable counting sort: (perm, indptr)."""
    buckets = [[] for _ in range(dim_size)]
    for e, v in enumerate(index.tolist()):
        buckets[v].append(e)
    perm, ptr = [], [0]
    for b in buckets:
        perm.extend(b)
        ptr.append(len(perm))
    return torch.tensor(perm, dtype=torch.long), torch.tensor(ptr, dtype=torch.long)
