"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py):
the oracle must reproduce them on any box, and the HIP kernels must match them."""
import glob
import os

import numpy as np
import pytest
import torch

import oracle
from util import assert_close_scaled, rel_norm

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ATTN = sorted(glob.glob(os.path.join(GOLD, "attn_*.npz")))
SRMS = sorted(glob.glob(os.path.join(GOLD, "srms_*.npz")))


def _load(path):
    with np.load(path, allow_pickle=False) as z:
        return {k: torch.from_numpy(z[k]) for k in z.files}


def test_fixtures_present():
    assert len(ATTN) == 3 and len(SRMS) == 2


@pytest.mark.parametrize("path", ATTN, ids=os.path.basename)
def test_oracle_reproduces_attention_fixture(path):
    f = _load(path)
    s = f["s"].reshape(-1, 1, 1) if "s" in f else None
    o, dq, dk, dv = oracle.linear_attn_fwd_bwd(f["q"], f["k"], f["v"], s, f["do"], torch.float64)
    for got, key in ((o, "o"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
        assert torch.allclose(got, f[key], rtol=1e-10, atol=1e-10), key
    bq, bk, bv = oracle.block_recurrence_bwd(f["q"], f["k"], f["v"], s, f["do"], 64)
    assert torch.allclose(bq, f["dq"], rtol=1e-9, atol=1e-9)
    assert torch.allclose(bk, f["dk"], rtol=1e-9, atol=1e-9)
    assert torch.allclose(bv, f["dv"], rtol=1e-9, atol=1e-9)


@pytest.mark.parametrize("path", SRMS, ids=os.path.basename)
def test_oracle_reproduces_srms_fixture(path):
    f = _load(path)
    y, dx = oracle.srmsnorm_fwd_bwd(f["x"], f["dy"], float(f["eps"]), torch.float64)
    assert torch.allclose(y, f["y"], rtol=1e-11, atol=1e-12)
    assert torch.allclose(dx, f["dx"], rtol=1e-9, atol=1e-11)


@pytest.mark.gpu
@pytest.mark.parametrize("path", ATTN, ids=os.path.basename)
def test_hip_matches_attention_fixture(path):
    from lightning_attn.ops import lightning_attn_func

    f = _load(path)
    dev = torch.device("cuda")
    q, k, v = (f[n].bfloat16().to(dev).requires_grad_() for n in ("q", "k", "v"))
    s = f["s"].reshape(-1, 1, 1).to(dev) if "s" in f else None
    o = lightning_attn_func(q, k, v, s)
    o.backward(f["do"].bfloat16().to(dev))
    # bf16 tolerance of this path: rtol = atol = 2e-2 (absolute term scaled by rms(ref))
    for got, key in ((o, "o"), (q.grad, "dq"), (k.grad, "dk"), (v.grad, "dv")):
        assert_close_scaled(got, f[key], 2e-2, 2e-2, key)
        assert rel_norm(got, f[key]) < 1e-2, key


@pytest.mark.gpu
@pytest.mark.parametrize("path", SRMS, ids=os.path.basename)
def test_hip_matches_srms_fixture(path):
    from lightning_attn.ops import SimpleRMSNorm

    f = _load(path)
    dev = torch.device("cuda")
    x = f["x"].bfloat16().to(dev).requires_grad_()
    y = SimpleRMSNorm(x.shape[-1], float(f["eps"]))(x)
    y.backward(f["dy"].bfloat16().to(dev))
    # tolerance of the reference's own test: atol 5e-2, rtol 1e-2 (tests/ops/test_srmsnorm.py:22-23)
    torch.testing.assert_close(y.double().cpu(), f["y"], atol=5e-2, rtol=1e-2)
    torch.testing.assert_close(x.grad.double().cpu(), f["dx"], atol=5e-2, rtol=1e-2)
