"""Oracle for decayed linear attention (Lightning Attention) -- test infrastructure.

Restates, without importing it, the reference's naive O(n^2) PyTorch path:

* ``build_slope_tensor``  <- lightning_attn/utils/utils.py:6-31
* ``decay_mask``/``full_mask`` <- lightning_attn/ops/torch/linear_attention.py:4-24
* ``linear_attn``         <- lightning_attn/ops/torch/linear_attention.py:27-34
* ``block_recurrence_*``  <- the recurrence the reference's device kernels
  implement, lightning_attn/ops/triton/lightning_attn2.py:41-85 (forward),
  :135-166 (intra-block backward), :234-395 (inter-block backward)

What pins each function (see tests/test_oracle_*.py):

* build_slope_tensor : known answers for h = 8, 12, 32 (closed form
  2^(-8(i+1)/h) and the published ALiBi interleave rule), dtype/shape.
* decay_mask / linear_attn : brute-force fp64 triple loop in plain C
  (oracle/la_oracle.c, an independent code path), special cases
  (s=None -> tril, huge s -> o_i=(q_i.k_i)v_i, n=1), causality, per-head
  independence, and the committed fixtures under tests/golden/.
* gradients : torch.autograd through linear_attn against the closed-form
  gradient sums evaluated by the C brute force, plus gradcheck in fp64.
* block_recurrence_* : identity with linear_attn_f64 for ragged n and for
  block sizes 16/64/128, concatenation property, linearity.
* kv_state : with k, v zeroed from token T on, the naive output at i >= T is
  exp(-s (i - T)) q_i KV_T (checked against linear_attn_f64 with unit-vector
  queries, which reads the matrix out row by row); KV_T over a split sequence
  obeys KV_T = exp(-s (T - T1)) KV_T1 + (state of the tokens T1..T alone).

No function here is "parity unpinned".
"""
import math

import torch


def build_slope_tensor(n_heads: int) -> torch.Tensor:
    """ALiBi-style per-head decay rates, float32, shape (h, 1, 1), on CPU.

    Follows lightning_attn/utils/utils.py:6-31.  For h a power of two the
    reference builds start = 2^(-2^-(log2 h - 3)) = 2^(-8/h) and returns
    start * start^i, i.e. (2^(-8/h))^(i+1) evaluated by repeated float
    multiplication in Python doubles, then rounds to float32.  Otherwise it
    takes the slopes of the largest power of two below h and appends every
    other slope of the next power of two.
    """

    def pow2_slopes(m):
        start = 2.0 ** (-(2.0 ** -(math.log2(m) - 3)))
        return [start * start**i for i in range(m)]

    def slopes(m):
        if math.log2(m).is_integer():
            return pow2_slopes(m)
        p = 2 ** math.floor(math.log2(m))
        return pow2_slopes(p) + slopes(2 * p)[0::2][: m - p]

    return torch.tensor(slopes(n_heads), dtype=torch.float32).reshape(n_heads, 1, 1)


def decay_mask(n: int, slope: float, dtype=torch.float32) -> torch.Tensor:
    """M[i,j] = exp(-slope*(i-j)) for i>=j, else 0.

    Follows linear_attention.py:4-12: the reference fills row i with
    -(slope * arange(i+1)) reversed (a float32 product of an integer and the
    slope), -inf above the diagonal, then exponentiates in float32.
    """
    idx = torch.arange(n)
    diff = (idx[:, None] - idx[None, :])  # i - j
    y = diff.clamp(min=0).to(dtype) * slope  # fl(k * slope) like the reference
    m = torch.exp(-y)
    return torch.where(diff >= 0, m, torch.zeros((), dtype=dtype))


def full_mask(n: int, slopes, dtype=torch.float32) -> torch.Tensor:
    """(h,n,n) mask, or (n,n) lower-triangular ones when slopes is None
    (linear_attention.py:15-24)."""
    if slopes is None:
        return torch.tril(torch.ones(n, n, dtype=dtype))
    return torch.stack([decay_mask(n, float(s), dtype) for s in slopes.reshape(-1)], 0)


def linear_attn(q, k, v, s=None):
    """Naive path with the reference's rounding order (linear_attention.py:27-34):
    scores in q.dtype, fp32 mask multiply, cast back to q.dtype, matmul with v."""
    n = q.shape[2]
    mask = full_mask(n, s).to(q.device)
    qk = torch.matmul(q, k.transpose(2, 3))
    qk = (qk.to(torch.float32) * mask).to(q.dtype)
    return torch.matmul(qk, v)


def linear_attn_f64(q, k, v, s=None):
    """Exact-arithmetic variant: everything in float64 (inputs up-cast)."""
    n = q.shape[2]
    sd = None if s is None else s.double()
    mask = full_mask(n, sd, torch.float64)
    qk = torch.matmul(q.double(), k.double().transpose(2, 3)) * mask
    return torch.matmul(qk, v.double())


def linear_attn_fwd_bwd(q, k, v, s, do, compute_dtype=None):
    """o, dq, dk, dv of the naive path through autograd.

    compute_dtype=None keeps the input dtype (the reference's own dataflow);
    torch.float32 / torch.float64 evaluate the same formula at that precision
    on the given (already rounded) inputs -- the target the device kernels are
    compared against.
    """
    dt = compute_dtype or q.dtype
    qq = q.detach().to(dt).requires_grad_()
    kk = k.detach().to(dt).requires_grad_()
    vv = v.detach().to(dt).requires_grad_()
    if dt == torch.float64:
        o = linear_attn_f64(qq, kk, vv, s)
    else:
        o = linear_attn(qq, kk, vv, s)
    o.backward(do.to(dt))
    return o.detach(), qq.grad, kk.grad, vv.grad


def _lam(s, h, dtype):
    if s is None:
        return torch.zeros(h, dtype=dtype)
    return s.reshape(-1).to(dtype)


def block_recurrence_fwd(q, k, v, s=None, block=64, dtype=torch.float64):
    """Forward by the block recurrence of lightning_attn2.py:41-85.

    O_t = ((Q_t K_t^T) * D) V_t + Lq * (Q_t KV);  KV <- lam^B KV + (K_t * Lk)^T V_t
    with Lq[r]=exp(-s r), Lk[r]=exp(-s (B-r)), D[r,c]=exp(-s (r-c)) [r>=c].
    Rows past n are zero-padded and dropped, as the kernel's tail masks do.
    """
    b, h, n, d = q.shape
    e = v.shape[-1]
    B = block
    T = (n + B - 1) // B
    pad = T * B - n
    rate = _lam(s, h, dtype).view(1, h, 1, 1)
    qf, kf, vf = (torch.nn.functional.pad(t.to(dtype), (0, 0, 0, pad)) for t in (q, k, v))
    r = torch.arange(B, dtype=dtype).view(1, 1, B, 1)
    lq = torch.exp(-rate * r)
    lk = torch.exp(-rate * (B - r))
    lb = torch.exp(-rate * B)
    diff = r - r.transpose(2, 3)
    D = torch.where(diff >= 0, torch.exp(-rate * diff.clamp(min=0)), torch.zeros((), dtype=dtype))
    kv = torch.zeros(b, h, d, e, dtype=dtype)
    out = torch.zeros(b, h, T * B, e, dtype=dtype)
    for t in range(T):
        sl = slice(t * B, (t + 1) * B)
        Q, K, V = qf[:, :, sl], kf[:, :, sl], vf[:, :, sl]
        out[:, :, sl] = ((Q @ K.transpose(2, 3)) * D) @ V + lq * (Q @ kv)
        kv = lb * kv + (K * lk).transpose(2, 3) @ V
    return out[:, :, :n]


def kv_state(k, v, s, T, dtype=torch.float64):
    """The d x e state the forward recurrence holds after the first T tokens,
    KV_T = sum_{t<T} exp(-s (T - t)) k_t^T v_t: the `kv` accumulator of
    lightning_attn2.py:55, 78-84 after T / BLOCK iterations, written as the closed-form sum.
    k: (b,h,n,d), v: (b,h,n,e) -> (b,h,d,e)."""
    b, h, n, d = k.shape
    rate = _lam(s, h, dtype).view(1, h, 1, 1)
    t = torch.arange(T, dtype=dtype).view(1, 1, T, 1)
    w = torch.exp(-rate * (T - t))
    return (k[:, :, :T].to(dtype) * w).transpose(2, 3) @ v[:, :, :T].to(dtype)


def block_recurrence_bwd(q, k, v, s, do, block=64, dtype=torch.float64):
    """dq, dk, dv by the recurrences of lightning_attn2.py:135-166, 234-395.

    dQ: forward sweep over the KV state; dK, dV: reverse sweep over the dKV
    state.  Written by hand (no autograd) so that it is an independent check of
    the formulas the device kernels implement.
    """
    b, h, n, d = q.shape
    e = v.shape[-1]
    B = block
    T = (n + B - 1) // B
    pad = T * B - n
    rate = _lam(s, h, dtype).view(1, h, 1, 1)
    qf, kf, vf, gf = (torch.nn.functional.pad(t.to(dtype), (0, 0, 0, pad)) for t in (q, k, v, do))
    r = torch.arange(B, dtype=dtype).view(1, 1, B, 1)
    lq = torch.exp(-rate * r)
    lk = torch.exp(-rate * (B - r))
    lb = torch.exp(-rate * B)
    diff = r - r.transpose(2, 3)
    D = torch.where(diff >= 0, torch.exp(-rate * diff.clamp(min=0)), torch.zeros((), dtype=dtype))
    dq = torch.zeros_like(qf)
    dk = torch.zeros_like(kf)
    dv = torch.zeros_like(vf)
    kv = torch.zeros(b, h, d, e, dtype=dtype)
    for t in range(T):
        sl = slice(t * B, (t + 1) * B)
        Q, K, V, G = qf[:, :, sl], kf[:, :, sl], vf[:, :, sl], gf[:, :, sl]
        A = (G @ V.transpose(2, 3)) * D
        dq[:, :, sl] = A @ K + lq * (G @ kv.transpose(2, 3))
        kv = lb * kv + (K * lk).transpose(2, 3) @ V
    dkv = torch.zeros(b, h, d, e, dtype=dtype)
    for t in reversed(range(T)):
        sl = slice(t * B, (t + 1) * B)
        Q, K, V, G = qf[:, :, sl], kf[:, :, sl], vf[:, :, sl], gf[:, :, sl]
        A = (G @ V.transpose(2, 3)) * D
        P = (Q @ K.transpose(2, 3)) * D
        dk[:, :, sl] = A.transpose(2, 3) @ Q + lk * (V @ dkv.transpose(2, 3))
        dv[:, :, sl] = P.transpose(2, 3) @ G + lk * (K @ dkv)
        dkv = lb * dkv + (Q * lq).transpose(2, 3) @ G
    return dq[:, :, :n], dk[:, :, :n], dv[:, :, :n]
