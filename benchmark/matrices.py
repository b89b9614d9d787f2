"""Sparse-matrix row structures and timing helpers for the benchmark scripts.

The reference times its operators on four SuiteSparse matrices that it downloads
(benchmark/scatter_segment.py:12-28). There is no network here, so each matrix is
replaced by a synthetic row structure with the same number of rows, the same number
of stored entries and a row-length distribution of the same kind (figures from the
collection's published statistics; the full symmetric pattern is counted, which is
what `loadmat(...).tocsr()` yields there). A real `.mat` file can be given instead
(`--mat`), read the way the reference reads it (benchmark/scatter_segment.py:37-41).
"""
import time
from dataclasses import dataclass

import numpy as np
import torch


@dataclass(frozen=True)
class Profile:
    group: str
    name: str
    rows: int
    entries: int
    kind: str       # 'web': heavy-tailed row lengths, 'mesh': narrow band around the mean
    longest: int    # longest row


# short rows / long rows, in the reference's order (benchmark/scatter_segment.py:12-19)
PROFILES = [
    Profile('DIMACS10', 'citationCiteseer', 268_495, 2_313_294, 'web', 1_318),
    Profile('SNAP', 'web-Stanford', 281_903, 2_312_497, 'web', 255),
    Profile('Janna', 'StocF-1465', 1_465_137, 21_005_389, 'mesh', 189),
    Profile('GHS_psdef', 'ldoor', 952_203, 46_522_475, 'mesh', 77),
]


@dataclass
class RowStructure:
    label: str
    rowptr: torch.Tensor    # int64 [rows + 1]
    row: torch.Tensor       # int64 [entries], sorted (COO row of every stored entry)
    row_shuffled: torch.Tensor

    @property
    def rows(self):
        return self.rowptr.numel() - 1

    @property
    def entries(self):
        return self.row.numel()

    @property
    def avg_row_len(self):
        return self.entries / max(self.rows, 1)


def _row_lengths(p: Profile, rng, scale: float) -> np.ndarray:
    rows = max(int(p.rows * scale), 1)
    target = max(int(p.entries * scale), rows)
    if p.kind == 'web':
        # lognormal body, clipped at the longest row of the real matrix; sigma 1.0 gives the
        # long tail of link / citation counts
        deg = np.exp(rng.normal(0.0, 1.0, rows))
    else:
        # finite-element stencils: most rows near the mean, none far from it
        deg = np.clip(rng.normal(1.0, 0.18, rows), 0.2, None)
    deg = deg * (target / deg.sum())
    deg = np.clip(np.rint(deg), 1, p.longest).astype(np.int64)
    # bring the total to the real matrix's count by touching rows at random
    diff = target - int(deg.sum())
    while diff != 0:
        step = 1 if diff > 0 else -1
        pick = rng.integers(0, rows, size=min(abs(diff), rows))
        ok = (deg[pick] + step >= 1) & (deg[pick] + step <= p.longest)
        pick = np.unique(pick[ok])
        deg[pick] += step
        diff -= step * len(pick)
    return deg


def _structure(label, indptr: np.ndarray, device, seed) -> RowStructure:
    rowptr = torch.from_numpy(indptr.astype(np.int64)).to(device)
    counts = rowptr[1:] - rowptr[:-1]
    row = torch.repeat_interleave(torch.arange(counts.numel(), device=device), counts)
    g = torch.Generator(device='cpu').manual_seed(seed)
    perm = torch.randperm(row.numel(), generator=g).to(device)
    return RowStructure(label, rowptr, row, row[perm])


def synthetic(p: Profile, device, scale: float = 1.0, seed: int = 0) -> RowStructure:
    rng = np.random.default_rng(seed)
    deg = _row_lengths(p, rng, scale)
    indptr = np.zeros(len(deg) + 1, dtype=np.int64)
    np.cumsum(deg, out=indptr[1:])
    return _structure(f'{p.group}/{p.name} (synthetic)', indptr, device, seed)


def from_mat(path: str, device, seed: int = 0) -> RowStructure:
    from scipy.io import loadmat
    mat = loadmat(path)['Problem'][0][0][2].tocsr()
    return _structure(path, np.asarray(mat.indptr), device, seed)


def structures(args):
    if args.mat:
        return [from_mat(m, args.device) for m in args.mat]
    wanted = [p for p in PROFILES if not args.only or p.name in args.only]
    return [synthetic(p, args.device, args.scale) for p in wanted]


def timed(fn, x, iters: int, with_backward: bool) -> float:
    """Seconds for `iters` back-to-back calls, the way the reference measures
    (benchmark/scatter_segment.py:82-106): wall clock between two device
    synchronisations, forward under no_grad or forward + autograd.grad with the
    output as the incoming gradient. Out of memory counts as infinitely slow."""
    sync = torch.cuda.synchronize if x.is_cuda else (lambda: None)
    try:
        sync()
        t0 = time.perf_counter()
        if with_backward:
            x = x.requires_grad_()
            for _ in range(iters):
                out = fn(x)
                out = out[0] if isinstance(out, tuple) else out
                torch.autograd.grad(out, x, out, only_inputs=True)
        else:
            with torch.no_grad():
                for _ in range(iters):
                    fn(x)
        sync()
        return time.perf_counter() - t0
    except RuntimeError as e:
        if 'out of memory' not in str(e):
            raise
        torch.cuda.empty_cache()
        return float('inf')


def bold(text, on=True):
    return f'\033[1m{text}\033[0m' if on else text


def print_table(title, sizes, rows, plain=False):
    """rows: list of (label, [seconds per size]); the fastest entry of each column is set in bold."""
    best = [min(t[c] for _, t in rows) for c in range(len(sizes))]
    width = max(len(label) for label, _ in rows)
    mark = (lambda s, on=True: s) if plain else bold
    print(mark(title))
    print('\t'.join([' ' * width] + [f'{s:>7}' for s in sizes]))
    for label, t in rows:
        print('\t'.join([mark(label.ljust(width))] +
                        [mark(f'{v:.5f}', v == b) for v, b in zip(t, best)]))
    print()
