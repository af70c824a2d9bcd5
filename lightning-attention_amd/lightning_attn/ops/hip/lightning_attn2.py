"""autograd operators over the HIP sweep kernels.

Same names and call conventions as lightning_attn/ops/triton/lightning_attn2.py:398-507
and lightning_attn2_no_decay.py:367-471: ``lightning_attn2(q, k, v, s)`` and
``lightning_attn2_no_decay(q, k, v)`` with q,k (b,h,n,d), v (b,h,n,e), s holding
h float32 rates; outputs come from torch.empty, kernels go on the current stream,
and the inputs are saved for backward - plus, for shapes where the library asks for
them (la_saved_state_bytes in the header), a few float32 states of the forward walk that let
the dQ sweep of the backward pass start mid-sequence (8 MiB at b4 h32 n8192 d=e=128).

Where the reference copies (``.contiguous()`` on q, k, v, do, lightning_attn2.py:402-405,
439-442), bf16 / fp16 tensors whose feature dim is contiguous and whose other strides are
16-byte multiples are used in place: a projection output ``(b, n, h*d)`` viewed as
``(b, h, n, d)`` needs no copy, and o, dq, dk, dv are allocated in the memory order of
v, q, k, v, so ``rearrange(o, "b h n d -> b n (h d)")`` is a view as well."""
import ctypes

import torch

from . import _lib


def _norm_strides(t):
    """Strides of a 4-d tensor with those of size-1 dims (never used for addressing, may be
    anything) replaced by the dense value."""
    st = list(t.stride())
    for i in (2, 1, 0):
        if t.shape[i] == 1:
            st[i] = t.shape[i + 1] * st[i + 1]
    return st


def _in_place_ok(t):
    """True when the kernels can address `t` (b,h,n,c) through its own strides."""
    if t.dtype == torch.float32 or t.dim() != 4 or t.stride(3) != 1:
        return False
    elt = t.element_size()
    if t.data_ptr() % 16:
        return False
    st = _norm_strides(t)
    if any(x <= 0 or (x * elt) % 16 for x in st[:3]):
        return False
    if st[2] < t.shape[3]:
        return False
    return ((t.shape[2] - 1) * st[2] + t.shape[3]) * elt < 2 ** 31


def _usable(t):
    """`t` itself where the kernels can address it, else a dense, 16-byte aligned copy."""
    if t.is_contiguous():
        # (a dense view into a larger buffer may start off the 16-byte grid)
        return t if t.data_ptr() % 16 == 0 else t.clone(memory_format=torch.contiguous_format)
    return t if _in_place_ok(t) else t.contiguous()


def _strides(*tensors):
    """(batch, head, token) strides of each tensor, in argument order."""
    vals = []
    for t in tensors:
        vals += _norm_strides(t)[:3]
    return (ctypes.c_int64 * len(vals))(*vals)


def _fwd(q, k, v, s, for_backward=False, silu=False):
    """Runs the forward pass; returns o, the tensors as the kernels used them and - `for_backward`, where the
    library has a use for them - the states the backward pass starts its dQ chunks from (else None).
    `silu`: q, k, v are pre-activations, the kernel applies SiLU as it loads them (forward only)."""
    _lib.require_same_device("lightning_attn2", q=q, k=k, v=v)
    if not (q.dtype == k.dtype == v.dtype):
        raise TypeError("q, k, v must share a dtype")
    if q.dim() != 4 or k.shape != q.shape or v.dim() != 4 or v.shape[:3] != q.shape[:3]:
        raise ValueError("shape mismatch: q %s k %s v %s" % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    q, k, v = _usable(q), _usable(k), _usable(v)
    b, h, n, d = q.shape
    e = v.shape[-1]
    if s is not None:
        if s.dtype != torch.float32 or s.device != q.device or not s.is_contiguous():
            s = s.to(device=q.device, dtype=torch.float32).contiguous()
        if s.numel() != h:
            raise ValueError("s must hold one rate per head (%d), got %d" % (h, s.numel()))
    L = _lib.lib()
    code = _lib.dtype_code(q.dtype)
    o = torch.empty_like(v)  # same sizes as v; dense, in v's memory order
    opts = _lib.current_opts()
    with _lib.on_device(q.device):
        ws_bytes = _lib.workspace_bytes(0, b, h, n, d, e, code, opts)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        sp = s.data_ptr() if s is not None else None
        wp = ws.data_ptr() if ws is not None else None
        strides = None if all(t.is_contiguous() for t in (q, k, v, o)) else _strides(q, k, v, o)
        op = ctypes.byref(opts) if opts is not None else None
        if silu:
            saved = None
            rc = L.la_fwd_silu(q.data_ptr(), k.data_ptr(), v.data_ptr(), sp, o.data_ptr(), strides, b, h, n, d, e, code,
                               wp, ws_bytes, op, _lib.stream_ptr(q.device))
        else:
            sv_bytes = _lib.saved_state_bytes(b, h, n, d, e, code, opts) if for_backward else 0
            saved = torch.empty(sv_bytes // 4, dtype=torch.float32, device=q.device) if sv_bytes else None
            rc = L.la_fwd_save(q.data_ptr(), k.data_ptr(), v.data_ptr(), sp, o.data_ptr(), strides, b, h, n, d, e, code,
                               wp, ws_bytes, op, saved.data_ptr() if saved is not None else None, sv_bytes,
                               _lib.stream_ptr(q.device))
    _lib.check(rc, "la_fwd")
    return o, q, k, v, s, saved


def _bwd(q, k, v, s, do, opts=None, saved=None):
    b, h, n, d = q.shape
    e = v.shape[-1]
    L = _lib.lib()
    code = _lib.dtype_code(q.dtype)
    if do.device != q.device:
        raise RuntimeError("lightning_attn2 backward: the upstream gradient is on %s, the inputs on %s" % (do.device, q.device))
    if do.dtype != q.dtype:
        do = do.to(q.dtype)
    do = _usable(do)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    with _lib.on_device(q.device):
        ws_bytes = _lib.workspace_bytes(1, b, h, n, d, e, code, opts)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        sp = s.data_ptr() if s is not None else None
        wp = ws.data_ptr() if ws is not None else None
        dense = all(t.is_contiguous() for t in (q, k, v, do, dq, dk, dv))
        strides = None if dense else _strides(q, k, v, do, dq, dk, dv)
        rc = L.la_bwd_saved(q.data_ptr(), k.data_ptr(), v.data_ptr(), sp, do.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                            dv.data_ptr(), strides, b, h, n, d, e, code, wp, ws_bytes,
                            ctypes.byref(opts) if opts is not None else None,
                            saved.data_ptr() if saved is not None else None, saved.numel() * 4 if saved is not None else 0,
                            _lib.stream_ptr(q.device))
    _lib.check(rc, "la_bwd")
    return dq, dk, dv


class LightningAttention2(torch.autograd.Function):
    """Decayed variant (lightning_attn2.py:398-504)."""

    @staticmethod
    def forward(ctx, q, k, v, s):
        if s is None:
            raise ValueError("lightning_attn2 needs decay rates s; use lightning_attn2_no_decay")
        o, q, k, v, s, saved = _fwd(q, k, v, s, any(ctx.needs_input_grad[:3]))
        ctx.save_for_backward(q, k, v, s, saved)
        # autograd runs backward on a thread of its own: the launch options in force now go with the node
        ctx.la_opts = _lib.current_opts()
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, s, saved = ctx.saved_tensors
        dq, dk, dv = _bwd(q, k, v, s, do, ctx.la_opts, saved)
        return dq, dk, dv, None


class LightningAttention2NoDecay(torch.autograd.Function):
    """lam = 1 variant (lightning_attn2_no_decay.py:367-468)."""

    @staticmethod
    def forward(ctx, q, k, v):
        o, q, k, v, _, saved = _fwd(q, k, v, None, any(ctx.needs_input_grad))
        ctx.save_for_backward(q, k, v, saved)
        ctx.la_opts = _lib.current_opts()
        return o

    @staticmethod
    def backward(ctx, do):
        q, k, v, saved = ctx.saved_tensors
        return _bwd(q, k, v, None, do, ctx.la_opts, saved)


def _native_ok(q, k, v, s):
    """Arguments the C++ autograd path takes as they are; anything else goes through the Python operators,
    which convert what can be converted and raise the documented errors."""
    if not (q.is_cuda and k.is_cuda and v.is_cuda and q.dtype in _lib._DTYPES and q.dtype == k.dtype == v.dtype):
        return False
    if q.dim() != 4 or v.dim() != 4 or k.shape != q.shape or v.shape[:3] != q.shape[:3] or k.device != q.device or v.device != q.device:
        return False
    return s is None or (torch.is_tensor(s) and s.numel() == q.shape[1])


def _run(q, k, v, s, function):
    ops = _lib.native_ops()
    if ops is not None and _native_ok(q, k, v, s):
        o = _lib.current_opts()
        if o is None:
            return ops.attn(q, k, v, s, 0, 0, 0, 0, 0, True)
        return ops.attn(q, k, v, s, o.chunks, o.scan, o.wide, o.paired, o.once, getattr(o, "save_states", True))
    return function.apply(q, k, v, s) if function is LightningAttention2 else function.apply(q, k, v)


def lightning_attn2(q, k, v, s):
    """Decayed lightning attention (lightning_attn2.py:398-507): q, k (b,h,n,d), v (b,h,n,e), s h float32 rates.
    Runs LightningAttention2, as a C++ autograd node where that library is built."""
    if s is None:
        raise ValueError("lightning_attn2 needs decay rates s; use lightning_attn2_no_decay")
    return _run(q, k, v, s, LightningAttention2)


def lightning_attn2_no_decay(q, k, v):
    """lam = 1 variant (lightning_attn2_no_decay.py:367-471)."""
    return _run(q, k, v, None, LightningAttention2NoDecay)


# the chunk-parallel variant of the reference (lightning_attn2_parallel.py:835-1072)
# computes the same function; the sweep kernels serve it as well
lightning_attn2_parallel = lightning_attn2


def silu_fused_ok(q, k, v):
    """True when lightning_attn_silu can run as one kernel: HIP tensors of one 16-bit dtype with feature dims
    the fused forward takes, and no gradient wanted (there is no fused backward pass)."""
    if not (q.is_cuda and q.dtype in (torch.bfloat16, torch.float16) and q.dtype == k.dtype == v.dtype):
        return False
    if torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad):
        return False
    return bool(_lib.lib().la_fwd_silu_supported(q.shape[-1], v.shape[-1], _lib.dtype_code(q.dtype)))


def lightning_attn_silu(q, k, v, s):
    """lightning_attn2(silu(q), silu(k), silu(v), s) (s None: no decay) as ONE forward kernel, the activation
    applied where the tiles are loaded: the forward pass of the attention block (examples/module/tnl_attn.py:51-56)
    without its three activation passes.  Only where silu_fused_ok(q, k, v); not differentiable."""
    ops = _lib.native_ops()
    if ops is not None and _native_ok(q, k, v, s):
        o = _lib.current_opts()
        if o is None:
            return ops.attn_silu(q, k, v, s, 0, 0, 0, 0, 0)
        return ops.attn_silu(q, k, v, s, o.chunks, o.scan, o.wide, o.paired, o.once)
    with torch.no_grad():
        return _fwd(q, k, v, s, False, True)[0]
