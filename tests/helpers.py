"""Shared helpers for the test-suite: fixture loading and seeded generators."""
import json
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# dtype matrix of the reference's tests (torch_scatter/testing.py:7-10)
DTYPES = [torch.half, torch.bfloat16, torch.float, torch.double, torch.int, torch.long]
ALL_DTYPES = DTYPES + [torch.int16, torch.int8, torch.uint8]
REDUCTIONS = ["sum", "add", "mean", "min", "max"]


def load_cases(name):
    with open(os.path.join(GOLDEN, name + ".json")) as f:
        return json.load(f)["cases"]


def tensor(x, dtype, device="cpu"):
    return None if x is None else torch.tensor(x, device=device).to(dtype)


def random_csr(rng, n_rows, max_deg, p_empty=0.2):
    deg = rng.integers(1, max_deg + 1, size=n_rows)
    deg[rng.random(n_rows) < p_empty] = 0
    indptr = np.zeros(n_rows + 1, dtype=np.int64)
    np.cumsum(deg, out=indptr[1:])
    index = np.repeat(np.arange(n_rows, dtype=np.int64), deg)
    return torch.from_numpy(indptr), torch.from_numpy(index)


def random_values(rng, shape, dtype, ties=True):
    """Values with many exact ties (small integer grid) so that arg tie-breaking
    is exercised; representable exactly in every dtype of the matrix."""
    if ties:
        x = rng.integers(-8, 9, size=shape).astype(np.float64)
    else:
        x = rng.standard_normal(size=shape)
    t = torch.from_numpy(x)
    if dtype == torch.uint8:
        t = t.abs()
    return t.to(dtype)
