"""The fixed-pattern cross-lane helpers of csrc/dpp.h (DPP row shifts, wave_shr:1, v_permlane16_swap /
v_permlane32_swap) against their definition in terms of lane numbers: ts_selftest_lane_ops applies each of them to
x = 3 * lane + 1 in one wavefront."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_lane_ops_match_their_definition():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from pytorch_scatter_amd import capi
    rows = 17
    out = torch.full((rows, 64), -1, dtype=torch.int32, device="cuda:0")
    capi._check(capi.lib().ts_selftest_lane_ops(capi._p(out), capi._stream(out)))
    got = out.cpu().numpy()
    lane = np.arange(64)
    x = 3 * lane + 1
    r = 0
    want_up1 = np.where(lane == 0, x, x[np.maximum(lane - 1, 0)])
    assert (got[r] == want_up1).all(), ("lane_up1", got[r]); r += 1
    for off in (1, 2, 4, 8, 16, 32):
        assert (got[r] == x[lane ^ off]).all(), ("lane_xor", off, got[r]); r += 1
    for off in (1, 2, 4, 8, 16, 32):
        recv = (lane & off) == 0          # the lanes a reduction tree reads at this step
        assert (got[r][recv] == x[(lane + off)[recv]]).all(), ("lane_down", off, got[r]); r += 1
    assert (got[r] == np.cumsum(x)).all(), ("wave_inclusive_sum", got[r]); r += 1
    assert (got[r] == want_up1 + 7).all(), ("lane_up1_64 low word", got[r]); r += 1
    assert (got[r] == want_up1).all(), ("lane_up1_64 high word", got[r]); r += 1
    assert (got[r] == x[lane ^ 16]).all(), ("lane_xor<16> on a float", got[r]); r += 1
    assert r == rows
