"""lightning_attn_silu_func: the attention block's SiLU on q, k, v (examples/module/tnl_attn.py:51-54 of the reference)
applied inside the forward kernel's tile load when no gradient is wanted.  Checked against the unfused chain
(three F.silu calls, then lightning_attn_func) on the device and against the naive oracle on SiLU-ed inputs:
same tolerance as the other bf16 / fp16 parity tests (util.assert_close_scaled with rtol = atol = 2e-2 scaled by the
sequence RMS, relative Frobenius error < 1e-2)."""
import pytest
import torch
import torch.nn.functional as F

import oracle
from util import assert_close_scaled, rel_norm

pytestmark = pytest.mark.gpu

from lightning_attn.ops import lightning_attn_func, lightning_attn_silu_func  # noqa: E402
from lightning_attn.ops.hip import silu_fused_ok  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402

DEV = "cuda"


def _inputs(b, h, n, d, e, dtype, seed, token_major):
    g = torch.Generator().manual_seed(seed)

    def mk(c):
        if token_major:  # a (b, n, h*c) projection output viewed as (b, h, n, c)
            return (1.5 * torch.randn(b, n, h, c, generator=g)).to(dtype).transpose(1, 2)
        return (1.5 * torch.randn(b, h, n, c, generator=g)).to(dtype)

    return mk(d), mk(d), mk(e)


@pytest.mark.parametrize("b, h, n, d, e, dtype, decay, token_major", [
    (2, 8, 700, 128, 128, torch.bfloat16, True, False),
    (1, 4, 333, 64, 96, torch.float16, False, False),
    (4, 32, 1024, 128, 128, torch.bfloat16, True, True),    # the block's layout at the benchmark's b*h
    (1, 2, 4096, 128, 128, torch.bfloat16, True, True),     # few sequences: chunks from scanned states
    (8, 32, 300, 128, 128, torch.bfloat16, True, False),    # many sequences: 128-column workgroups
    (1, 3, 500, 72, 40, torch.bfloat16, True, False),
])
def test_silu_in_the_tile_load_matches_the_unfused_chain(b, h, n, d, e, dtype, decay, token_major):
    q, k, v = _inputs(b, h, n, d, e, dtype, 7 + n, token_major)
    s = _build_slope_tensor(h) if decay else None
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    sd = s.to(DEV) if decay else None
    assert silu_fused_ok(qd, kd, vd)
    print("silu case", (b, h, n, d, e, dtype, decay, token_major), flush=True)
    got = lightning_attn_silu_func(qd, kd, vd, sd)
    with torch.no_grad():
        chain = lightning_attn_func(F.silu(qd), F.silu(kd), F.silu(vd), sd)
    torch.cuda.synchronize()
    assert got.shape == chain.shape and got.dtype == dtype and not got.requires_grad
    # same kernels on (nearly always bit-) equal operands: the fast exp / reciprocal may flip a rounding here and there
    assert rel_norm(got, chain.float()) < 2e-3
    sel = slice(0, min(h, 3))
    want = oracle.linear_attn(F.silu(q[-1:, sel]).float(), F.silu(k[-1:, sel]).float(), F.silu(v[-1:, sel]).float(),
                              s[sel] if decay else None)
    assert_close_scaled(got[-1:, sel], want, 2e-2, 2e-2, "silu o")
    assert rel_norm(got[-1:, sel], want) < 1e-2


def test_silu_func_falls_back_where_the_fused_forward_does_not_apply():
    b, h, n, d = 1, 4, 300, 128
    q, k, v = (t.to(DEV) for t in _inputs(b, h, n, d, d, torch.bfloat16, 3, False))
    s = _build_slope_tensor(h).to(DEV)
    # a gradient is wanted: the differentiable chain
    qg, kg, vg = (t.clone().requires_grad_() for t in (q, k, v))
    assert not silu_fused_ok(qg, kg, vg)
    o = lightning_attn_silu_func(qg, kg, vg, s)
    do = torch.randn_like(o)
    o.backward(do)
    qr, kr, vr = (t.clone().requires_grad_() for t in (q, k, v))
    lightning_attn_func(F.silu(qr), F.silu(kr), F.silu(vr), s).backward(do)
    torch.cuda.synchronize()
    for a, r in ((qg.grad, qr.grad), (kg.grad, kr.grad), (vg.grad, vr.grad)):
        assert torch.equal(a, r)
    with torch.no_grad():
        assert silu_fused_ok(qg, kg, vg)  # no gradient recorded: fused
        assert rel_norm(lightning_attn_silu_func(qg, kg, vg, s), o.detach().float()) < 2e-3
    # feature dims the fused forward does not take, float32
    q2, k2, v2 = (t.to(DEV) for t in _inputs(1, 2, 200, 192, 192, torch.bfloat16, 4, False))
    assert not silu_fused_ok(q2, k2, v2)
    s2 = _build_slope_tensor(2).to(DEV)
    with torch.no_grad():
        a = lightning_attn_silu_func(q2, k2, v2, s2)
        r = lightning_attn_func(F.silu(q2), F.silu(k2), F.silu(v2), s2)
    assert torch.equal(a, r)
    assert not silu_fused_ok(q.float(), k.float(), v.float())
