"""autograd operators over the HIP sweep kernels.

Same names and call conventions as lightning_attn/ops/triton/lightning_attn2.py:398-507
and lightning_attn2_no_decay.py:367-471: ``lightning_attn2(q, k, v, s)`` and
``lightning_attn2_no_decay(q, k, v)`` with q,k (b,h,n,d), v (b,h,n,e), s holding
h float32 rates; inputs are made contiguous, outputs come from torch.empty,
kernels go on the current stream, and only the inputs are saved for backward."""
import torch

from . import _lib


def _fwd(q, k, v, s):
    _lib.require_gpu(q, "lightning_attn2")
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("q, k, v must share a dtype")
    b, h, n, d = q.shape
    e = v.shape[-1]
    if k.shape != q.shape or v.shape[:3] != q.shape[:3]:
        raise ValueError("shape mismatch: q %s k %s v %s" % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    if s is not None:
        s = s.to(device=q.device, dtype=torch.float32).contiguous()
        if s.numel() != h:
            raise ValueError("s must hold one rate per head (%d), got %d" % (h, s.numel()))
    L = _lib.lib()
    code = _lib.dtype_code(q.dtype)
    o = torch.empty((b, h, n, e), dtype=q.dtype, device=q.device)
    ws_bytes = L.la_workspace_bytes(0, b, h, n, d, e, code)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    with torch.cuda.device(q.device):
        rc = L.la_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr() if s is not None else None,
                      o.data_ptr(), b, h, n, d, e, code, ws.data_ptr() if ws is not None else None, ws_bytes,
                      _lib.stream_ptr(q.device))
    _lib.check(rc, "la_fwd")
    return o, q, k, v, s


def _bwd(q, k, v, s, do):
    do = do.contiguous()
    b, h, n, d = q.shape
    e = v.shape[-1]
    L = _lib.lib()
    code = _lib.dtype_code(q.dtype)
    if do.dtype != q.dtype:
        do = do.to(q.dtype)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    ws_bytes = L.la_workspace_bytes(1, b, h, n, d, e, code)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    with torch.cuda.device(q.device):
        rc = L.la_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr() if s is not None else None,
                      do.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), b, h, n, d, e, code,
                      ws.data_ptr() if ws is not None else None, ws_bytes, _lib.stream_ptr(q.device))
    _lib.check(rc, "la_bwd")
    return dq, dk, dv


class LightningAttention2(torch.autograd.Function):
    """Decayed variant (lightning_attn2.py:398-504)."""

    @staticmethod
    def forward(ctx, q, k, v, s):
        if s is None:
            raise ValueError("lightning_attn2 needs decay rates s; use lightning_attn2_no_decay")
        o, q, k, v, s = _fwd(q, k, v, s)
        ctx.save_for_backward(q, k, v, s)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, s = ctx.saved_tensors
        dq, dk, dv = _bwd(q, k, v, s, do)
        return dq, dk, dv, None


class LightningAttention2NoDecay(torch.autograd.Function):
    """lam = 1 variant (lightning_attn2_no_decay.py:367-468)."""

    @staticmethod
    def forward(ctx, q, k, v):
        o, q, k, v, _ = _fwd(q, k, v, None)
        ctx.save_for_backward(q, k, v)
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v = ctx.saved_tensors
        return _bwd(q, k, v, None, do)


lightning_attn2 = LightningAttention2.apply
lightning_attn2_no_decay = LightningAttention2NoDecay.apply
# the chunk-parallel variant of the reference (lightning_attn2_parallel.py:835-1072)
# computes the same function; the sweep kernels serve it as well
lightning_attn2_parallel = LightningAttention2.apply
