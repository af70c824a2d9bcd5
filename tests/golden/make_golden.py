"""Writes the committed fixtures of tests/golden/ (run from the repo root:
``python tests/golden/make_golden.py``).

The reference ships no golden vectors for this path, so these come from this
repository's own oracle: inputs are seeded, rounded to bfloat16 (stored as
float32, which holds them exactly) and the expected outputs are the plain-C
double-precision brute force of oracle/la_oracle.c.  The fixtures let the GPU
box check both its oracle build and the HIP kernels against numbers produced in
a different container."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402
from oracle import c_oracle  # noqa: E402


def attention_case(name, b, h, n, d, e, decay, seed):
    g = torch.Generator().manual_seed(seed)
    q, k, v, do = (torch.randn(b, h, n, x, generator=g).bfloat16().float().numpy() for x in (d, d, e, e))
    s = oracle.build_slope_tensor(h).flatten().numpy() if decay else None
    sd = None if s is None else s.astype(np.float64)
    o = c_oracle.naive_fwd(q, k, v, sd)
    dq, dk, dv = c_oracle.naive_bwd(q, k, v, sd, do)
    out = dict(q=q, k=k, v=v, do=do, o=o, dq=dq, dk=dk, dv=dv)
    if s is not None:
        out["s"] = s
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)


def srms_case(name, rows, cols, seed, eps):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g)
    x = torch.where(torch.rand(rows, cols, generator=g) < 0.01, x * 50, x).bfloat16().float().numpy()
    dy = torch.randn(rows, cols, generator=g).bfloat16().float().numpy()
    y, rstd = c_oracle.srms_fwd(x, eps)
    dx = c_oracle.srms_bwd(x, dy, eps)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), x=x, dy=dy, y=y, rstd=rstd, dx=dx, eps=np.float64(eps))


if __name__ == "__main__":
    attention_case("attn_decay_h3_n70_d8_e16", 1, 3, 70, 8, 16, True, 11)
    attention_case("attn_nodecay_h2_n130_d16_e8", 1, 2, 130, 16, 8, False, 12)
    attention_case("attn_decay_h4_n64_d16_e16", 1, 4, 64, 16, 16, True, 13)
    srms_case("srms_r6_c264", 6, 264, 21, 1e-6)
    srms_case("srms_r3_c1000", 3, 1000, 22, 1e-6)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
