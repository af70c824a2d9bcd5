"""Pins the attention oracle (oracle/linear_attn_oracle.py) on the CPU:
plain-C brute force, special cases, invariants, gradcheck, block recurrence."""
import numpy as np
import pytest
import torch

import oracle
from oracle import c_oracle
from lightning_attn.ops import linear_attn as pkg_linear_attn

torch.manual_seed(0)


def _rand(b, h, n, d, e, dtype=torch.float64, seed=0):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(b, h, n, x, generator=g, dtype=torch.float64).to(dtype) for x in (d, d, e, e))


@pytest.mark.parametrize("shape", [(1, 1, 1, 4, 4), (2, 3, 7, 4, 5), (1, 5, 33, 8, 3), (1, 2, 64, 16, 16)])
@pytest.mark.parametrize("decay", [True, False])
def test_naive_vs_c_bruteforce(shape, decay):
    b, h, n, d, e = shape
    q, k, v, do = _rand(*shape)
    s = oracle.build_slope_tensor(h) if decay else None
    sn = None if s is None else s.double().numpy()
    o, dq, dk, dv = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float64)
    oc = c_oracle.naive_fwd(q.numpy(), k.numpy(), v.numpy(), sn)
    cq, ck, cv = c_oracle.naive_bwd(q.numpy(), k.numpy(), v.numpy(), sn, do.numpy())
    for a, c in ((o, oc), (dq, cq), (dk, ck), (dv, cv)):
        assert np.allclose(a.numpy(), c, rtol=1e-11, atol=1e-11)


def test_fp32_dataflow_and_package_mirror():
    q, k, v, _ = _rand(2, 4, 50, 16, 8, torch.float32)
    s = oracle.build_slope_tensor(4)
    o32 = oracle.linear_attn(q, k, v, s)
    assert o32.dtype == torch.float32
    assert torch.allclose(o32.double(), oracle.linear_attn_f64(q, k, v, s), rtol=1e-4, atol=1e-4)
    # the package's public linear_attn is an independent restatement of the same dataflow
    assert torch.equal(pkg_linear_attn(q, k, v, s), o32)
    assert torch.equal(pkg_linear_attn(q, k, v), oracle.linear_attn(q, k, v))
    qb, kb, vb = (t.bfloat16() for t in (q, k, v))
    ob = oracle.linear_attn(qb, kb, vb, s)
    assert ob.dtype == torch.bfloat16 and torch.equal(ob, pkg_linear_attn(qb, kb, vb, s))


def test_mask_definition():
    m = oracle.decay_mask(6, 0.5)
    assert m.dtype == torch.float32 and m.shape == (6, 6)
    assert torch.equal(torch.triu(m, 1), torch.zeros(6, 6))
    assert torch.equal(torch.diagonal(m), torch.ones(6))
    assert abs(m[5, 2].item() - np.exp(-1.5)) < 1e-7
    full = oracle.full_mask(5, oracle.build_slope_tensor(3))
    assert full.shape == (3, 5, 5)
    assert torch.equal(oracle.full_mask(5, None), torch.tril(torch.ones(5, 5)))


def test_special_cases():
    q, k, v, _ = _rand(1, 2, 9, 4, 3)
    # no decay == plain causal linear attention; zero rates agree with None
    o_none = oracle.linear_attn_f64(q, k, v, None)
    o_zero = oracle.linear_attn_f64(q, k, v, torch.zeros(2, 1, 1))
    assert torch.allclose(o_none, o_zero)
    want = torch.tril(q @ k.transpose(2, 3)) @ v
    assert torch.allclose(o_none, want)
    # huge rate: only the diagonal survives, o_i = (q_i . k_i) v_i
    o_big = oracle.linear_attn_f64(q, k, v, torch.full((2, 1, 1), 200.0))
    assert torch.allclose(o_big, (q * k).sum(-1, keepdim=True) * v, atol=1e-12)
    # n = 1
    q1, k1, v1, _ = _rand(1, 2, 1, 4, 3)
    assert torch.allclose(oracle.linear_attn_f64(q1, k1, v1, oracle.build_slope_tensor(2)),
                          (q1 * k1).sum(-1, keepdim=True) * v1)


def test_invariants():
    q, k, v, _ = _rand(1, 3, 20, 4, 4)
    s = oracle.build_slope_tensor(3)
    o = oracle.linear_attn_f64(q, k, v, s)
    # causality: changing tokens >= t leaves outputs < t alone
    q2, k2, v2 = q.clone(), k.clone(), v.clone()
    q2[:, :, 12:] += 1.0
    k2[:, :, 12:] -= 2.0
    v2[:, :, 12:] *= 3.0
    o2 = oracle.linear_attn_f64(q2, k2, v2, s)
    assert torch.equal(o[:, :, :12], o2[:, :, :12]) and not torch.allclose(o[:, :, 12:], o2[:, :, 12:])
    # heads are independent and use their own rate
    for hh in range(3):
        oh = oracle.linear_attn_f64(q[:, hh:hh + 1], k[:, hh:hh + 1], v[:, hh:hh + 1], s[hh:hh + 1])
        assert torch.allclose(oh, o[:, hh:hh + 1])
    # linear in v, additive over feature slices of q/k
    assert torch.allclose(oracle.linear_attn_f64(q, k, 2 * v + v2, s),
                          2 * o + oracle.linear_attn_f64(q, k, v2, s))
    parts = oracle.linear_attn_f64(q[..., :2], k[..., :2], v, s) + oracle.linear_attn_f64(q[..., 2:], k[..., 2:], v, s)
    assert torch.allclose(parts, o)


def test_gradcheck_fp64():
    q, k, v, _ = _rand(1, 2, 6, 3, 2)
    s = oracle.build_slope_tensor(2)
    q, k, v = (t.requires_grad_() for t in (q, k, v))
    assert torch.autograd.gradcheck(lambda a, b, c: oracle.linear_attn_f64(a, b, c, s), (q, k, v), eps=1e-6, atol=1e-6)


@pytest.mark.parametrize("n", [1, 63, 64, 65, 200, 513])
@pytest.mark.parametrize("block", [16, 64, 128])
@pytest.mark.parametrize("decay", [True, False])
def test_block_recurrence_identity(n, block, decay):
    q, k, v, do = _rand(1, 3, n, 8, 5, seed=n)
    s = oracle.build_slope_tensor(3) if decay else None
    o, dq, dk, dv = oracle.linear_attn_fwd_bwd(q, k, v, s, do, torch.float64)
    ob = oracle.block_recurrence_fwd(q, k, v, s, block)
    bq, bk, bv = oracle.block_recurrence_bwd(q, k, v, s, do, block)
    for a, c in ((ob, o), (bq, dq), (bk, dk), (bv, dv)):
        assert torch.allclose(a, c, rtol=1e-10, atol=1e-10)


def test_config1_plumbing():
    """b1 h8 n1024 d=e=64 fp32, slopes(8), loss = o.sum(): the CPU-runnable configuration."""
    q, k, v, _ = _rand(1, 8, 1024, 64, 64, torch.float32, seed=2024)
    s = oracle.build_slope_tensor(8)
    do = torch.ones(1, 8, 1024, 64)
    o, dq, dk, dv = oracle.linear_attn_fwd_bwd(q, k, v, s, do)
    ob = oracle.block_recurrence_fwd(q, k, v, s, 64)
    bq, bk, bv = oracle.block_recurrence_bwd(q, k, v, s, do, 64)
    for a, c in ((o, ob), (dq, bq), (dk, bk), (dv, bv)):
        assert ((a.double() - c).norm() / c.norm()).item() < 1e-5


@pytest.mark.parametrize("decay", [True, False])
def test_kv_state_read_out_by_the_naive_path(decay):
    """kv_state against the naive path: with k, v zeroed from token T on, o_i = exp(-s (i - T)) q_i KV_T
    for i >= T; unit-vector queries read KV_T out row by row.  Plus the split rule of the recurrence."""
    b, h, n, d, e, T = 2, 3, 40, 5, 4, 23
    _, k, v, _ = _rand(b, h, n, d, e, seed=11)
    s = oracle.build_slope_tensor(h) if decay else None
    rate = s.reshape(-1).double() if decay else torch.zeros(h, dtype=torch.float64)
    S = oracle.kv_state(k, v, s, T)
    assert S.shape == (b, h, d, e)
    k0, v0 = k.clone(), v.clone()
    k0[:, :, T:] = 0
    v0[:, :, T:] = 0
    for row in range(d):
        q = torch.zeros(b, h, n, d, dtype=torch.float64)
        q[..., row] = 1.0
        o = oracle.linear_attn_f64(q, k0, v0, s)
        for i in (T, T + 1, n - 1):
            want = torch.exp(-rate * (i - T)).view(1, h, 1) * S[:, :, row, :]
            assert torch.allclose(o[:, :, i, :], want, rtol=1e-12, atol=1e-12)
    T1 = 9
    tail = oracle.kv_state(k[:, :, T1:], v[:, :, T1:], s, T - T1)
    joined = torch.exp(-rate * (T - T1)).view(1, h, 1, 1) * oracle.kv_state(k, v, s, T1) + tail
    assert torch.allclose(S, joined, rtol=1e-12, atol=1e-12)
