"""Group-wise statistics over the entries that share an index: softmax,
log-softmax, logsumexp and standard deviation (API of
torch_scatter/composite/{softmax,logsumexp,std}.py). Softmax, log-softmax
and logsumexp are fused operators; std is composed from the scatter
operators."""
from typing import Optional

import torch

from .scatter import scatter_sum


def _expand_index(index: torch.Tensor, like: torch.Tensor, dim: int) -> torch.Tensor:
    # a 1-D index addresses `dim`; missing trailing dims are broadcast
    # (torch_scatter/utils.py:4-13)
    dim = dim + like.dim() if dim < 0 else dim
    if index.dim() == 1:
        shape = [1] * like.dim()
        shape[dim] = index.numel()
        index = index.view(shape)
    while index.dim() < like.dim():
        index = index.unsqueeze(-1)
    return index.expand(like.size())


def _require_float(src: torch.Tensor, name: str):
    if not torch.is_floating_point(src):
        raise ValueError(f"`{name}` can only be computed over tensors with "
                         "floating point data types.")


def scatter_softmax(src: torch.Tensor, index: torch.Tensor, dim: int = -1,
                    dim_size: Optional[int] = None) -> torch.Tensor:
    """``exp(src - max) / sum(exp(src - max))`` over the entries that share an
    index along ``dim`` (torch_scatter/composite/softmax.py:8-29). One operator:
    three passes over ``src`` forward, two backward, when every column of a row
    belongs to the same group; otherwise composed from the scatter operators."""
    _require_float(src, "scatter_softmax")
    return torch.ops.torch_scatter.scatter_softmax(src, index, dim, dim_size, False, 0.0)


def scatter_log_softmax(src: torch.Tensor, index: torch.Tensor, dim: int = -1,
                        eps: float = 1e-12, dim_size: Optional[int] = None) -> torch.Tensor:
    """``(src - max) - log(sum(exp(src - max)) + eps)`` over the entries that
    share an index (torch_scatter/composite/softmax.py:32-59)."""
    _require_float(src, "scatter_log_softmax")
    return torch.ops.torch_scatter.scatter_softmax(src, index, dim, dim_size, True, eps)


def scatter_logsumexp(src: torch.Tensor, index: torch.Tensor, dim: int = -1,
                      out: Optional[torch.Tensor] = None, dim_size: Optional[int] = None,
                      eps: float = 1e-12) -> torch.Tensor:
    """``log(sum(exp(src)) + eps)`` over the entries that share an index, stabilised by
    the group maximum; groups without entries give 0
    (torch_scatter/composite/logsumexp.py:8-57). One fused operator (two passes over
    ``src`` forward, one backward) unless ``out`` is given or the index differs between
    the columns of a row; then the same sequence as upstream on the scatter operators."""
    _require_float(src, "scatter_logsumexp")
    return torch.ops.torch_scatter.scatter_logsumexp(src, index, dim, out, dim_size, eps)


def scatter_std(src: torch.Tensor, index: torch.Tensor, dim: int = -1,
                out: Optional[torch.Tensor] = None, dim_size: Optional[int] = None,
                unbiased: bool = True) -> torch.Tensor:
    if out is not None:
        dim_size = out.size(dim)
    dim = dim + src.dim() if dim < 0 else dim
    count_dim = index.dim() - 1 if index.dim() <= dim else dim
    count = scatter_sum(torch.ones(index.size(), dtype=src.dtype, device=src.device),
                        index, count_dim, None, dim_size)
    full_index = _expand_index(index, src, dim)
    total = scatter_sum(src, full_index, dim, None, dim_size)
    count = _expand_index(count, total, dim).clamp(1)
    centred = src - total.div(count).gather(dim, full_index)
    sq = scatter_sum(centred * centred, full_index, dim, out, dim_size)
    denom = count.sub(1).clamp_(1) if unbiased else count
    return sq.div(denom + 1e-6).sqrt()
