"""Group-wise statistics over the entries that share an index: softmax,
log-softmax, logsumexp and standard deviation (API of
torch_scatter/composite/{softmax,logsumexp,std}.py), each one registered
operator."""
from typing import Optional

import torch


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
    """``sqrt(sum((src - mean)^2) / (count - 1 + 1e-6))`` over the entries that share an
    index (``count`` instead of ``count - 1`` if not ``unbiased``;
    torch_scatter/composite/std.py:8-41). Group sums and counts come from the scatter
    kernels, the squared deviations from one fused pass; with ``out`` given or an index
    that differs between the columns of a row, the same sequence as upstream on the
    scatter operators. Counts are exact (fp32) where upstream counts in the element type."""
    return torch.ops.torch_scatter.scatter_std(src, index, dim, out, dim_size, unbiased)
