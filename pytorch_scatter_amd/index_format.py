"""Index formats either side of the reductions, and scatter for an index that is
used many times.

The reference has no operator for these steps: its callers bring ``row`` and
``rowptr`` from the same sparse matrix (benchmark/scatter_segment.py:38-41) and
``segment_coo`` asks for a sorted index (torch_scatter/segment_coo.py:80-83).

* :func:`index_to_indptr` / :func:`indptr_to_index`: sorted index <-> row pointers.
* :class:`SortedIndex`: sorts an unsorted 1-D index once (stable), keeping the row
  numbers ``perm`` and the row pointers ``indptr`` of the sorted order.
* :func:`scatter_sorted`: ``scatter`` with such a plan, run as a segmented
  reduction over permuted rows: one pass over ``src``, no atomics, results that
  do not depend on scheduling (the same bits on every call).
"""
from typing import Optional, Tuple, Union

import torch


def index_to_indptr(index: torch.Tensor, dim_size: int) -> torch.Tensor:
    """Row pointers ``[..., dim_size + 1]`` of an index ``[..., E]`` sorted along
    its last dimension: ``indptr[..., r]`` is the first position whose index is
    ``>= r``."""
    return torch.ops.torch_scatter.index_to_indptr(index, dim_size)


def indptr_to_index(indptr: torch.Tensor, num_entries: Optional[int] = None) -> torch.Tensor:
    """The sorted index ``[..., E]`` of row pointers ``[..., N + 1]``; ``E`` is read
    back from ``indptr[..., -1]`` unless ``num_entries`` is given."""
    return torch.ops.torch_scatter.indptr_to_index(indptr, num_entries)


class SortedIndex:
    """A 1-D index sorted once for many scatters.

    ``perm`` (int32): positions of the entries in sorted order, equal values in
    order of position; ``indptr``: row pointers of the sorted order;
    ``index[perm.long()]`` is sorted. Building the plan synchronises once (it
    checks that every value lies in ``[0, dim_size)``).
    """

    def __init__(self, index: torch.Tensor, dim_size: Optional[int] = None):
        if index.dim() != 1:
            raise ValueError("SortedIndex expects a one-dimensional index")
        if dim_size is None:
            dim_size = int(index.max()) + 1 if index.numel() > 0 else 0
        self.index = index
        self.dim_size = int(dim_size)
        self.perm, self.indptr = torch.ops.torch_scatter.sort_index(index, self.dim_size)

    def sorted_index(self) -> torch.Tensor:
        return torch.ops.torch_scatter.indptr_to_index(self.indptr, self.index.numel())


def scatter_sorted(src: torch.Tensor, plan: SortedIndex, dim: int = -1,
                   reduce: str = "sum") -> Union[torch.Tensor, Tuple[torch.Tensor, torch.Tensor]]:
    """``scatter(src, plan.index, dim, dim_size=plan.dim_size, reduce=reduce)`` through
    the plan. ``sum`` and ``mean`` return the result, ``min`` and ``max`` the pair
    ``(values, positions)`` like ``scatter_min`` / ``scatter_max`` (first position
    wins ties, an empty slot reports ``src.size(dim)``). Differentiable in ``src``.
    Sums of 16-bit floats accumulate in fp32 here (``scatter`` adds in the element
    type)."""
    if reduce == "add":
        reduce = "sum"
    if reduce not in ("sum", "mean", "min", "max"):
        raise ValueError(f"scatter_sorted: unknown reduce '{reduce}'")
    out, arg = torch.ops.torch_scatter.scatter_sorted(src, plan.index, plan.perm, plan.indptr, dim, reduce)
    return (out, arg) if reduce in ("min", "max") else out
