"""Group-wise statistics over the entries that share an index: softmax,
log-softmax, logsumexp and standard deviation (API of
torch_scatter/composite/{softmax,logsumexp,std}.py). Softmax and log-softmax
are one fused operator; logsumexp and std are composed from the scatter
operators."""
from typing import Optional

import torch

from .scatter import scatter_max, scatter_sum


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
    _require_float(src, "scatter_logsumexp")
    index = _expand_index(index, src, dim)
    if out is not None:
        dim_size = out.size(dim)
    elif dim_size is None:
        dim_size = int(index.max()) + 1
    shape = list(src.size())
    shape[dim] = dim_size
    # groups without entries keep -inf so that they drop out of the result
    group_max = torch.full(shape, float("-inf"), dtype=src.dtype, device=src.device)
    scatter_max(src, index, dim, group_max, dim_size)
    z = src - group_max.gather(dim, index)
    z.masked_fill_(torch.isnan(z), float("-inf"))
    previous: Optional[torch.Tensor] = None
    if out is not None:
        previous = out.clone()
        out = out.sub_(group_max).exp_()
    total = scatter_sum(z.exp_(), index, dim, out, dim_size)
    result = total.add_(eps).log_().add_(group_max)
    if previous is None:
        return result.nan_to_num_(neginf=0.0)
    bad = ~result.isfinite()
    result[bad] = previous[bad]
    return result


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
