"""The CPU oracle against every known-answer table the reference's tests hold
(tests/golden/*.json), over the reference's dtype matrix."""
from itertools import product

import pytest
import torch

from helpers import DTYPES, REDUCTIONS, load_cases, tensor

SCATTER = load_cases("scatter_cases")
SEGMENT = load_cases("segment_cases")
GATHER = load_cases("gather_cases")


def _want(case, reduce, dtype):
    return tensor(case[reduce], dtype)


@pytest.mark.parametrize("ci,reduce,dtype", product(range(len(SCATTER)), REDUCTIONS + ["mul"], DTYPES))
def test_scatter_forward(oracle, ci, reduce, dtype):
    case = SCATTER[ci]
    if reduce not in case:
        pytest.skip("table has no entry for this reduction")
    src = tensor(case["src"], dtype)
    index = tensor(case["index"], torch.long)
    got = oracle.op_scatter(src, index, case["dim"], None, None, reduce)
    if isinstance(got, tuple):
        got, arg = got
        if "arg_" + reduce in case:
            assert torch.equal(arg, tensor(case["arg_" + reduce], torch.long))
    assert torch.all(got == _want(case, reduce, dtype))


@pytest.mark.parametrize("ci,reduce,dtype", product(range(6), REDUCTIONS, DTYPES))
def test_scatter_out(oracle, ci, reduce, dtype):
    # test/test_scatter.py:127-152
    case = SCATTER[ci]
    src = tensor(case["src"], dtype)
    index = tensor(case["index"], torch.long)
    expected = _want(case, reduce, dtype)
    out = torch.full_like(expected, -2)
    oracle.op_scatter(src, index, case["dim"], out, None, reduce)
    if reduce in ("sum", "add"):
        expected = expected - 2
    elif reduce == "mean":
        return
    elif reduce == "min":
        expected = expected.fill_(-2)
    elif reduce == "max":
        expected[expected == 0] = -2
    assert torch.all(out == expected)


@pytest.mark.parametrize("ci,reduce,dtype", product(range(len(SEGMENT)), REDUCTIONS, DTYPES))
def test_segment_forward(oracle, ci, reduce, dtype):
    case = SEGMENT[ci]
    if reduce not in case:
        pytest.skip("table has no entry for this reduction")
    src = tensor(case["src"], dtype)
    index = tensor(case["index"], torch.long)
    indptr = tensor(case["indptr"], torch.long)
    want = _want(case, reduce, dtype)
    for got, second in (oracle.segment_csr(src, indptr, None, reduce),
                        oracle.segment_coo(src, index, None, None, reduce)):
        if reduce in ("min", "max"):
            assert torch.equal(second, tensor(case["arg_" + reduce], torch.long))
        assert torch.all(got == want)


@pytest.mark.parametrize("ci,reduce,dtype", product(range(6), REDUCTIONS, DTYPES))
def test_segment_out(oracle, ci, reduce, dtype):
    # test/test_segment.py:132-161: csr overwrites, coo accumulates
    case = SEGMENT[ci]
    src = tensor(case["src"], dtype)
    index = tensor(case["index"], torch.long)
    indptr = tensor(case["indptr"], torch.long)
    expected = _want(case, reduce, dtype)
    out = torch.full_like(expected, -2)
    oracle.segment_csr(src, indptr, out, reduce)
    assert torch.all(out == expected)
    out.fill_(-2)
    oracle.segment_coo(src, index, out, None, reduce)
    if reduce in ("sum", "add"):
        expected = expected - 2
    elif reduce == "mean":
        return
    elif reduce == "min":
        expected = expected.fill_(-2)
    elif reduce == "max":
        expected[expected == 0] = -2
    assert torch.all(out == expected)


@pytest.mark.parametrize("ci,dtype", product(range(len(GATHER)), DTYPES))
def test_gather_forward_and_out(oracle, ci, dtype):
    case = GATHER[ci]
    src = tensor(case["src"], dtype)
    index = tensor(case["index"], torch.long)
    indptr = tensor(case["indptr"], torch.long)
    want = tensor(case["expected"], dtype)
    assert torch.all(oracle.gather_csr(src, indptr) == want)
    assert torch.all(oracle.gather_coo(src, index) == want)
    size = list(src.size())
    size[index.dim() - 1] = index.size(-1)
    out = src.new_full(size, -2)
    oracle.gather_csr(src, indptr, out)
    assert torch.all(out == want)
    out.fill_(-2)
    oracle.gather_coo(src, index, out)
    assert torch.all(out == want)


@pytest.mark.parametrize("ci,reduce", product(range(6), REDUCTIONS))
def test_non_contiguous_index(oracle, ci, reduce):
    # test/test_segment.py:164-191, test/test_scatter.py:155-173
    case = SEGMENT[ci]
    src = tensor(case["src"], torch.float)
    index = tensor(case["index"], torch.long)
    indptr = tensor(case["indptr"], torch.long)
    if src.dim() > 1:
        src = src.transpose(0, 1).contiguous().transpose(0, 1)
    if index.dim() > 1:
        index = index.transpose(0, 1).contiguous().transpose(0, 1)
        indptr = indptr.transpose(0, 1).contiguous().transpose(0, 1)
    want = _want(case, reduce, torch.float)
    assert torch.all(oracle.segment_csr(src, indptr, None, reduce)[0] == want)
    assert torch.all(oracle.segment_coo(src, index, None, None, reduce)[0] == want)


@pytest.mark.parametrize("reduce", REDUCTIONS)
def test_zero_elements(oracle, reduce):
    # test/test_zero_tensors.py:12-36
    x = torch.randn(0, 0, 0, 16)
    index = torch.tensor([], dtype=torch.long)
    got = oracle.op_scatter(x, index, 0, None, 0, reduce)
    got = got[0] if isinstance(got, tuple) else got
    assert got.size() == (0, 0, 0, 16)
    assert oracle.segment_coo(x, index, None, 0, reduce)[0].size() == (0, 0, 0, 16)
    assert oracle.gather_coo(x, index).size() == (0, 0, 0, 16)
    assert oracle.segment_csr(x, index, None, reduce)[0].size() == (0, 0, 0, 16)
    assert oracle.gather_csr(x, index).size() == (0, 0, 0, 16)
