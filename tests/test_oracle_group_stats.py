"""The oracle's softmax / log-softmax / logsumexp / std over groups, pinned by
the checks of the reference's own tests (test/composite/test_softmax.py:6-54,
test_logsumexp.py:5-45, test_std.py:5-20) and by the per-group library
routines on seeded random inputs. The closed-form backward is pinned against
autograd through those library routines."""
import pytest
import torch


def _groups(index, n):
    return [(index == g).nonzero().flatten() for g in range(n)]


def test_softmax_reference_vectors(oracle):
    # test/composite/test_softmax.py:6-26 and :30-50
    src = torch.tensor([0.2, 0, 0.2, -2.1, 3.2, 7, -1, float("-inf")])
    index = torch.tensor([0, 1, 0, 1, 1, 2, 4, 4])
    for fn, lib in ((oracle.scatter_softmax, torch.softmax), (oracle.scatter_log_softmax, torch.log_softmax)):
        out = fn(src, index)
        o0 = lib(torch.tensor([0.2, 0.2]), dim=-1)
        o1 = lib(torch.tensor([0, -2.1, 3.2]), dim=-1)
        o2 = lib(torch.tensor([7], dtype=torch.float), dim=-1)
        o4 = lib(torch.tensor([-1, float("-inf")]), dim=-1)
        want = torch.stack([o0[0], o1[0], o0[1], o1[1], o1[2], o2[0], o4[0], o4[1]])
        assert torch.allclose(out, want)


def test_logsumexp_reference_vectors(oracle):
    # test/composite/test_logsumexp.py:5-32
    src = torch.tensor([0.5, 0.5, 0.0, -2.1, 3.2, 7.0, -1.0, -100.0])
    index = torch.tensor([0, 0, 1, 1, 1, 2, 4, 4])
    out = oracle.scatter_logsumexp(src, index)
    for part, got in zip(src.split([2, 3, 1, 0, 2]), out.unbind()):
        if part.numel() > 0:
            assert got.tolist() == torch.logsumexp(part, dim=0).tolist()
        else:
            assert got.item() == 0.0
    # :35-45, accumulate into a given out
    out = torch.tensor([-10.0, -10.0])
    res = oracle.scatter_logsumexp(torch.tensor([-1.0, -50.0]), torch.tensor([0, 0]), out=out)
    assert res.allclose(torch.tensor([-0.9999, -10.0]), atol=1e-4)


def test_std_reference_vectors(oracle):
    # test/composite/test_std.py:5-15
    src = torch.tensor([[2, 0, 1, 4, 3], [0, 2, 1, 3, 4]], dtype=torch.float)
    index = torch.tensor([[0, 0, 0, 0, 0], [1, 1, 1, 1, 1]], dtype=torch.long)
    out = oracle.scatter_std(src, index, dim=-1, unbiased=True)
    std = src.std(dim=-1, unbiased=True)[0]
    assert torch.allclose(out, torch.tensor([[std, 0], [0, std]]))


@pytest.mark.parametrize("dim,shape", [(0, (200, 3)), (1, (2, 150, 4)), (-1, (3, 90))])
def test_against_library_routines(oracle, dim, shape):
    g = torch.Generator().manual_seed(7)
    src = torch.randn(shape, generator=g, dtype=torch.double) * 3
    d = dim if dim >= 0 else len(shape) + dim
    n = 11
    index = torch.randint(0, n - 1, (shape[d],), generator=g)  # group n-1 stays empty
    idx_shape = [1] * len(shape)
    idx_shape[d] = shape[d]
    full = index.view(idx_shape).expand(shape)
    soft = oracle.scatter_softmax(src, full, dim, n)
    logsoft = oracle.scatter_log_softmax(src, full, dim, 1e-12, n)
    lse = oracle.scatter_logsumexp(src, full, dim, None, n)
    std = oracle.scatter_std(src, full, dim, None, n, True)
    for grp, sel in enumerate(_groups(index, n)):
        if sel.numel() == 0:
            assert float(lse.select(d, grp).abs().max()) == 0.0
            assert float(std.select(d, grp).abs().max()) == 0.0
            continue
        part = src.index_select(d, sel)
        assert torch.allclose(soft.index_select(d, sel), torch.softmax(part, d), rtol=1e-12, atol=1e-15)
        assert torch.allclose(logsoft.index_select(d, sel), torch.log_softmax(part, d), rtol=1e-9, atol=1e-9)
        assert torch.allclose(lse.select(d, grp), torch.logsumexp(part, d), rtol=1e-9, atol=1e-9)
        if sel.numel() > 1:
            assert torch.allclose(std.select(d, grp), part.std(d, unbiased=True), rtol=1e-5)


@pytest.mark.parametrize("log_space", [False, True])
def test_softmax_backward_closed_form(oracle, log_space):
    g = torch.Generator().manual_seed(3)
    src = (torch.randn(120, 5, generator=g, dtype=torch.double) * 2).requires_grad_(True)
    index = torch.randint(0, 9, (120,), generator=g)
    grad = torch.randn(120, 5, generator=g, dtype=torch.double)
    lib = torch.log_softmax if log_space else torch.softmax
    out = torch.zeros_like(src)
    for sel in _groups(index, 9):
        if sel.numel() > 0:
            out = out.index_copy(0, sel, lib(src.index_select(0, sel), 0))
    out.backward(grad)
    y = (oracle.scatter_log_softmax(src.detach(), index, 0, 0.0, 9) if log_space
         else oracle.scatter_softmax(src.detach(), index, 0, 9))
    got = oracle.scatter_softmax_backward(y, grad, index, 0, 9, log_space)
    assert torch.allclose(got, src.grad, rtol=1e-9, atol=1e-12)


def test_logsumexp_backward_closed_form(oracle):
    g = torch.Generator().manual_seed(4)
    src = (torch.randn(150, 4, generator=g, dtype=torch.double) * 2).requires_grad_(True)
    index = torch.randint(0, 8, (150,), generator=g)  # group 8 stays empty
    grad = torch.randn(9, 4, generator=g, dtype=torch.double)
    rows = []
    for sel in _groups(index, 9):
        rows.append(torch.logsumexp(src.index_select(0, sel), 0) if sel.numel() else torch.zeros(4, dtype=torch.double))
    torch.stack(rows).backward(grad)
    y = oracle.scatter_logsumexp(src.detach(), index, 0, None, 9)
    got = oracle.scatter_logsumexp_backward(src.detach(), y, grad, index, 0)
    assert torch.allclose(got, src.grad, rtol=1e-9, atol=1e-12)


@pytest.mark.parametrize("unbiased", [True, False])
def test_std_backward_against_library_std(oracle, unbiased):
    """The gradient the oracle derives for scatter_std is that of torch's own std taken
    group by group (up to the 1e-6 in the divisor); a one-entry group gives NaN."""
    g = torch.Generator().manual_seed(9)
    src = torch.randn(150, 4, generator=g, dtype=torch.double) * 2 + 1
    index = torch.randint(0, 7, (150,), generator=g)
    index[0] = 7  # a group of one entry
    grad = torch.randn(9, 4, generator=g, dtype=torch.double)
    std, got = oracle.scatter_std_backward(src, grad, index, 0, 9, unbiased)
    assert torch.equal(std, oracle.scatter_std(src, index.view(-1, 1).expand(150, 4), 0, None, 9, unbiased))
    ref = src.clone().requires_grad_(True)
    total = sum((ref.index_select(0, sel).std(0, unbiased=unbiased) * grad[grp]).sum()
                for grp, sel in enumerate(_groups(index, 9)) if sel.numel() > 1)
    total.backward()
    keep = index != 7
    assert torch.allclose(got[keep], ref.grad[keep], rtol=1e-5, atol=1e-9)
    assert bool(torch.isnan(got[~keep]).all())
