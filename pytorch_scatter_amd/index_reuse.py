"""A front-end that turns ``scatter`` into a segmented reduction when an index is
used again (message passing over a fixed graph: every layer, every epoch).

Off by default. With :func:`enable_index_reuse`, ``scatter_sum / mean / min /
max`` with a one-dimensional index, no ``out`` and rows of at least 64 bytes look
the index up by identity (storage address, version counter, length, ``dim_size``):
the first sighting runs the atomic kernels as usual, the second sorts the index
once (:class:`~pytorch_scatter_amd.index_format.SortedIndex`, one
synchronisation) and from then on every call runs
:func:`~pytorch_scatter_amd.index_format.scatter_sorted`: one pass over ``src``,
no atomics, the same bits on every call. The cache keeps a reference to every
index it has seen, so an address cannot come back with other contents, and an
in-place change of an index bumps its version counter and with it the key.
Sums of 16-bit floats accumulate in fp32 on this path (``scatter`` adds in the
element type), so a result can change in its last bits between the first calls
(atomic kernels) and the later ones (plan).

Caveats. The key is an identity, not a checksum. Writes that do not bump the
version counter leave a stale plan behind, and every later call silently uses
the old permutation: ``index.data.copy_(...)``, in-place updates through a
``detach()``-ed alias, writes through a raw pointer or a DLPack capsule, custom
operators that take ``data_ptr()``. After such a write call
:func:`disable_index_reuse` (and enable again), use a fresh tensor, or pass an
explicit :class:`~pytorch_scatter_amd.index_format.SortedIndex` to
``scatter_sorted``. The cache holds strong references to at most ``max_plans``
index tensors; their device memory stays allocated while they are cached.
"""
import os
from collections import OrderedDict
from typing import Optional

import torch

from .index_format import SortedIndex

_MIN_ROW_BYTES = 64
_DTYPES = (torch.float32, torch.float64, torch.float16, torch.bfloat16, torch.int32, torch.int64, torch.int16,
           torch.int8, torch.uint8)

_enabled = False
_max_plans = 8
_cache: "OrderedDict[tuple, list]" = OrderedDict()  # key -> [index (kept alive), sightings, plan or None]


def enable_index_reuse(max_plans: int = 8) -> None:
    """Turn the front-end on; at most ``max_plans`` indices are remembered (least recently used first out)."""
    global _enabled, _max_plans
    _enabled = True
    _max_plans = max(int(max_plans), 1)


def disable_index_reuse() -> None:
    """Turn the front-end off and drop every remembered index and plan."""
    global _enabled
    _enabled = False
    _cache.clear()


def index_reuse_enabled() -> bool:
    return _enabled


def plan_for(src: torch.Tensor, index: torch.Tensor, dim: int, out: Optional[torch.Tensor],
             dim_size: Optional[int]) -> Optional[SortedIndex]:
    """The plan of ``index`` if this call qualifies and the index has been seen before, else None."""
    if not _enabled or out is not None or index.dim() != 1 or src.dim() == 0:
        return None
    if not (src.is_cuda and index.is_cuda) or index.dtype != torch.long or src.dtype not in _DTYPES:
        return None
    d = dim + src.dim() if dim < 0 else dim
    if d < 0 or d >= src.dim() or index.numel() == 0 or src.size(d) != index.numel():
        return None
    row_bytes = src.element_size()
    for s in src.shape[d + 1:]:
        row_bytes *= s
    if row_bytes < _MIN_ROW_BYTES:
        return None
    key = (index.data_ptr(), index._version, index.numel(), index.stride(0), dim_size, index.device.index)
    entry = _cache.get(key)
    if entry is None:
        _cache[key] = [index, 1, None]
        while len(_cache) > _max_plans:
            _cache.popitem(last=False)
        return None
    _cache.move_to_end(key)
    entry[1] += 1
    if entry[2] is None:
        entry[2] = SortedIndex(index, dim_size)
    return entry[2]


if os.environ.get("TS_INDEX_REUSE", "0") not in ("", "0"):
    enable_index_reuse()
