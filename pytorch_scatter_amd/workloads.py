"""Synthetic inputs of the five measurement configurations (seed 0).

Index structures are drawn with numpy on the host (cheap: they are 8 bytes per
entry); feature tensors are drawn on the device. Every generator takes a
``scale`` in (0, 1] that shrinks the number of rows/entries proportionally, so
that parity tests and the CPU baseline can use a bounded sample of the same
distribution.
"""
from dataclasses import dataclass
from typing import Optional

import numpy as np
import torch


@dataclass
class CsrWorkload:
    name: str
    indptr: torch.Tensor   # int64 [N+1], host
    index: torch.Tensor    # int64 [E], host (row id of every entry)
    N: int
    E: int
    K: int
    dtype: torch.dtype


def _csr_from_degrees(deg: np.ndarray):
    indptr = np.zeros(deg.size + 1, dtype=np.int64)
    np.cumsum(deg, out=indptr[1:])
    index = np.repeat(np.arange(deg.size, dtype=np.int64), deg)
    return torch.from_numpy(indptr), torch.from_numpy(index)


def c2_segment_csr(scale: float = 1.0, mean16: bool = False) -> CsrWorkload:
    """100000 segments, degrees Zipf(2.0) clipped to [1, 512], fp32 [E, 64].

    The literal draw has mean degree ~4.7; ``mean16=True`` is the variant whose
    mean degree is ~16 (every degree multiplied by 3.4 and rounded, clipped to
    the same [1, 512])."""
    rng = np.random.default_rng(0)
    n = max(int(100000 * scale), 16)
    deg = np.clip(rng.zipf(2.0, size=n), 1, 512).astype(np.int64)
    if mean16:
        deg = np.clip(np.rint(deg * 3.4), 1, 512).astype(np.int64)
    indptr, index = _csr_from_degrees(deg)
    return CsrWorkload("C2" + ("-mean16" if mean16 else ""), indptr, index, n, int(indptr[-1]), 64,
                       torch.float32)


def c3_segment_coo(scale: float = 1.0) -> CsrWorkload:
    """1M non-empty segments with Poisson(8)+1 entries; ids increase with random
    gaps (each id is followed by an unused one with probability 1/16), so some
    output rows stay empty. fp32 [E, 128], U(-1, 1)."""
    rng = np.random.default_rng(0)
    n_seg = max(int(1_000_000 * scale), 16)
    deg_seg = (rng.poisson(8.0, size=n_seg) + 1).astype(np.int64)
    step = 1 + (rng.random(n_seg) < 1.0 / 16).astype(np.int64)
    ids = np.cumsum(step) - 1
    N = int(ids[-1]) + 1
    deg = np.zeros(N, dtype=np.int64)
    deg[ids] = deg_seg
    indptr, index = _csr_from_degrees(deg)
    return CsrWorkload("C3", indptr, index, N, int(indptr[-1]), 128, torch.float32)


def c5_gnn(scale: float = 1.0) -> CsrWorkload:
    """N = 2.4M nodes, out-degree Zipf(1.8) clipped at the cap that makes the
    mean ~26 (E ~ 62M), bf16 [., 128]."""
    rng = np.random.default_rng(0)
    n = max(int(2_400_000 * scale), 16)
    raw = rng.zipf(1.8, size=n).astype(np.int64)
    lo, hi = 1, int(raw.max())
    target = 26.0
    while lo < hi:  # smallest cap whose clipped mean reaches the target
        mid = (lo + hi) // 2
        if np.minimum(raw, mid).mean() >= target:
            hi = mid
        else:
            lo = mid + 1
    deg = np.minimum(raw, lo)
    indptr, index = _csr_from_degrees(deg)
    return CsrWorkload("C5", indptr, index, n, int(indptr[-1]), 128, torch.bfloat16)


@dataclass
class ScatterWorkload:
    name: str
    index: torch.Tensor          # int64 [E], host
    N: int
    E: int
    K: int
    dtype: torch.dtype
    tie_src: Optional[torch.Tensor] = None   # positions whose value is copied ...
    tie_dst: Optional[torch.Tensor] = None   # ... onto these positions (same node)


def c1_scatter_sum() -> ScatterWorkload:
    """src fp32 [200000, 16], index uniform in [0, 10000)."""
    g = torch.Generator().manual_seed(0)
    index = torch.randint(0, 10000, (200000,), generator=g)
    return ScatterWorkload("C1", index, 10000, 200000, 16, torch.float32)


def c4_scatter_minmax(K: int, scale: float = 1.0) -> ScatterWorkload:
    """E = 10M entries over N = 100000 nodes, node drawn with p_i ~ i^-1.2 (the
    hottest node holds ~19.6 % of the entries), order shuffled; 5 % of the
    entries are exact copies of another entry of the same node."""
    rng = np.random.default_rng(0)
    N = 100000
    E = max(int(10_000_000 * scale), 1000)
    p = np.arange(1, N + 1, dtype=np.float64) ** -1.2
    p /= p.sum()
    index = rng.choice(N, size=E, p=p).astype(np.int64)
    order = np.argsort(index, kind="stable")
    same_as_prev = np.zeros(E, dtype=bool)
    same_as_prev[1:] = index[order][1:] == index[order][:-1]
    cand = np.nonzero(same_as_prev)[0]          # sorted positions that have a predecessor in their node
    pick = cand[rng.random(cand.size) < 0.05 * E / max(cand.size, 1)]
    dst = order[pick]
    src = order[pick - 1]
    return ScatterWorkload(f"C4-K{K}", torch.from_numpy(index), N, E, K, torch.float32,
                           torch.from_numpy(src), torch.from_numpy(dst))


def scatter_values(w: ScatterWorkload, device, seed: int = 0) -> torch.Tensor:
    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn((w.E, w.K), generator=g, device=device, dtype=torch.float32).to(w.dtype)
    if w.tie_src is not None:
        # copies of copies are resolved in order of increasing position so ties stay exact
        x[w.tie_dst.to(device)] = x[w.tie_src.to(device)]
    return x


def edge_values(w: CsrWorkload, device, rows: Optional[int] = None, seed: int = 0,
                uniform: bool = False) -> torch.Tensor:
    """[rows or E, K] features, drawn in chunks to bound temporary memory."""
    n = w.E if rows is None else rows
    g = torch.Generator(device=device).manual_seed(seed)
    out = torch.empty((n, w.K), dtype=w.dtype, device=device)
    step = 1 << 22
    for s in range(0, n, step):
        e = min(s + step, n)
        if uniform:
            chunk = torch.rand((e - s, w.K), generator=g, device=device, dtype=torch.float32) * 2 - 1
        else:
            chunk = torch.randn((e - s, w.K), generator=g, device=device, dtype=torch.float32)
        out[s:e] = chunk.to(w.dtype)
    return out


# ---- algorithmic bytes: every input/output tensor counted once -------------
def bytes_segment(E, N, K, s, with_arg=False, coo=False):
    idx = E * 8 if coo else (N + 1) * 8
    return E * K * s + idx + N * K * s + (N * K * 8 if with_arg else 0)


def bytes_gather(E, N, K, s, coo=False):
    idx = E * 8 if coo else (N + 1) * 8
    return N * K * s + idx + E * K * s


def bytes_scatter(E, N, K, s, with_arg=False):
    return E * K * s + E * 8 + N * K * s + (N * K * 8 if with_arg else 0)
