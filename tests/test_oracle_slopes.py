"""Pins oracle.build_slope_tensor and the package's _build_slope_tensor against
known answers (lightning_attn/utils/utils.py:6-31) and the plain-C restatement."""
import numpy as np
import pytest
import torch

import oracle
from oracle import c_oracle
from lightning_attn.utils import _build_slope_tensor


@pytest.mark.parametrize("fn", [oracle.build_slope_tensor, _build_slope_tensor])
def test_known_answers(fn):
    s8 = fn(8)
    assert s8.dtype == torch.float32 and s8.shape == (8, 1, 1) and s8.device.type == "cpu"
    assert torch.equal(s8.flatten(), torch.tensor([2.0 ** -(i + 1) for i in range(8)]))
    s12 = fn(12).flatten().double()
    want = [2.0 ** -(i + 1) for i in range(8)] + [2.0 ** -0.5, 2.0 ** -1.5, 2.0 ** -2.5, 2.0 ** -3.5]
    assert torch.allclose(s12, torch.tensor(want, dtype=torch.float64), rtol=1e-7, atol=0)
    s32 = fn(32).flatten().double()
    want32 = torch.tensor([2.0 ** (-(i + 1) / 4) for i in range(32)], dtype=torch.float64)
    assert torch.allclose(s32, want32, rtol=1e-6, atol=0)
    assert abs(s32[0].item() - 0.84089643) < 1e-7 and s32[-1].item() == 0.00390625
    assert fn(1).flatten().tolist() == [2.0 ** -8]


@pytest.mark.parametrize("h", [1, 2, 3, 5, 8, 12, 16, 20, 24, 32, 40, 64, 96])
def test_matches_c_and_package(h):
    a = oracle.build_slope_tensor(h)
    assert torch.equal(a, _build_slope_tensor(h))
    c = c_oracle.slopes(h)
    assert np.allclose(a.flatten().double().numpy(), c, rtol=1e-6, atol=0)
    # all rates positive, at most 1, first half (power-of-two part) strictly decreasing
    assert (a > 0).all() and (a < 1).all()


def test_interleave_rule():
    # non power of two: slopes(p) ++ slopes(2p)[0::2][:h-p]
    for h, p in ((12, 8), (20, 16), (40, 32)):
        s = oracle.build_slope_tensor(h).flatten()
        assert torch.equal(s[:p], oracle.build_slope_tensor(p).flatten())
        assert torch.equal(s[p:], oracle.build_slope_tensor(2 * p).flatten()[0::2][: h - p])
