"""Seeded random walk over shapes, dtypes, layouts and launch modes (sequence chunks from scanned states or
with warm-up blocks, 64- / 128-column / all-column workgroups, paired / separate dK + dV launches, states saved
by the forward pass or not), each case against the naive oracle."""
import os
import random
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "lightning-attention_amd"))
sys.path.insert(0, ROOT)

from lightning_attn.ops import lightning_attn_func  # noqa: E402
from lightning_attn.ops.hip import launch_opts  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402
from oracle import linear_attn_oracle as oracle  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rel(a, r):
    return ((a.float().cpu() - r.float()).norm() / (r.float().norm() + 1e-30)).item()


def _walk(seed, cases, dims, widths, max_b, max_h):
    rnd = random.Random(seed)
    for case in range(cases):
        b, h = rnd.randint(1, max_b), rnd.randint(1, max_h)
        n = rnd.choice([1, 2, 63, 64, 65, 127, 128, 129, 300, 513, 777, 1000, rnd.randint(1, 1200)])
        d = 8 * rnd.randint(*dims)
        e = d if rnd.random() < 0.6 else 8 * rnd.randint(*dims)
        dtype = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        if dtype == torch.float32:  # the float32 kernel takes feature dims up to 128
            d, e = min(d, 8 * rnd.randint(1, 16)), min(e, 8 * rnd.randint(1, 16))
        decay = rnd.random() < 0.75
        token_major = rnd.random() < 0.4
        env = {}  # launch options of this case
        if rnd.random() < 0.6:
            env["wide"] = rnd.choice(widths)
        if rnd.random() < 0.6:
            env["chunks"] = rnd.choice([1, 2, 3, 4, 5, 9, 17, 40, 64])
        if rnd.random() < 0.3:
            env["scan"] = False
        if rnd.random() < 0.2:
            env["paired"] = False
        if rnd.random() < 0.5:
            env["once"] = rnd.choice([False, True])
        if rnd.random() < 0.3:
            env["save_states"] = False
        g = torch.Generator().manual_seed(1000 * seed + case)

        def make(cols, scale):
            t = (torch.randn(b, n, h, cols, generator=g) * scale).to(dtype)
            return t.to(DEV).transpose(1, 2) if token_major else t.transpose(1, 2).contiguous().to(DEV)

        q, k, v, do = make(d, 0.6), make(d, 0.6), make(e, 1.0), make(e, 1.0)
        s = _build_slope_tensor(h) if decay else None
        what = (seed, case, (b, h, n, d, e), dtype, decay, token_major, env)
        print(what, flush=True)  # names the case should a launch go wrong
        qg, kg, vg = (t.detach().requires_grad_() for t in (q, k, v))
        with launch_opts(**env):
            o = lightning_attn_func(qg, kg, vg, None if s is None else s.to(DEV))
            o.backward(do)
        torch.cuda.synchronize()
        want = oracle.linear_attn_fwd_bwd(q.cpu(), k.cpu(), v.cpu(), s, do.cpu(),
                                          torch.float64 if dtype == torch.float32 else torch.float32)
        limit = {torch.bfloat16: 1e-2, torch.float16: 2e-3, torch.float32: 1e-4}[dtype]
        for name, a, r in zip(("o", "dq", "dk", "dv"), (o.detach(), qg.grad, kg.grad, vg.grad), want):
            assert a.dtype == dtype and _rel(a, r) < limit, (what, name, _rel(a, r))


@pytest.mark.parametrize("seed", [101, 202, 303, 404, 505])
def test_random_cases_match_the_oracle(seed):
    _walk(seed, 20, (1, 32), [False, True], 3, 9)


@pytest.mark.parametrize("seed", [11, 22, 33])
def test_random_cases_at_feature_dims_129_to_192_match_the_oracle(seed):
    """Where a workgroup can take all columns of a sequence (three accumulator slabs per state wave), and where the
    forward pass of many sequences leaves states for dQ in that form."""
    _walk(seed, 16, (17, 24), [False, True, "all", "all"], 5, 30)
