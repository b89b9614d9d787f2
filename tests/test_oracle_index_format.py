"""The oracle's index-format routines (plain loops) against library routines:
numpy searchsorted / repeat / stable argsort and scipy's COO -> CSR conversion."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch


@pytest.mark.parametrize("E,N", [(0, 0), (0, 5), (1, 1), (200, 17), (500, 3), (300, 400)])
def test_formats_against_numpy_and_scipy(oracle, E, N):
    rng = np.random.default_rng(E + N)
    idx = rng.integers(0, max(N, 1), size=E) if N > 0 else np.zeros(0, dtype=np.int64)
    srt = np.sort(idx)
    ptr = oracle.index_to_indptr(torch.from_numpy(srt), N)
    assert ptr.tolist() == np.searchsorted(srt, np.arange(N + 1), side="left").tolist()
    assert oracle.indptr_to_index(ptr).tolist() == np.repeat(np.arange(N), np.diff(ptr.numpy())).tolist() == srt.tolist()
    perm, ptr2 = oracle.sort_index(torch.from_numpy(idx), N)
    assert perm.tolist() == np.argsort(idx, kind="stable").tolist()
    assert ptr2.tolist() == ptr.tolist()
    if E > 0:
        m = sp.coo_matrix((np.ones(E), (idx, np.arange(E))), shape=(N, E)).tocsr()
        assert m.indptr.tolist() == ptr.tolist()
