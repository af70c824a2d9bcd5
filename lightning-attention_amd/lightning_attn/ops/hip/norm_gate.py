"""Gated output norm of the TNL attention block over the HIP row kernels:
``norm_gate(o, g, weight, bias, eps) = layer_norm(o, weight, bias, eps) * sigmoid(g)``,
the arithmetic of the reference's examples/module/tnl_attn.py:66-69 in one pass forward and
one backward."""
import torch

from . import _lib


_supported = {}
_ws_bytes = {}


def norm_gate_supported(cols, dtype):
    """True when the kernels take rows of `cols` elements of `dtype` (the answer depends on these two alone
    and is remembered)."""
    key = (cols, dtype)
    got = _supported.get(key)
    if got is None:
        try:
            got = bool(_lib.lib().norm_gate_supported(cols, _lib.dtype_code(dtype)))
        except TypeError:
            got = False
        if len(_supported) > 1024:
            _supported.clear()
        _supported[key] = got
    return got


def _workspace_bytes(rows, cols, code):
    key = (rows, cols, code)
    got = _ws_bytes.get(key)
    if got is None:
        got = _lib.lib().norm_gate_workspace_bytes(rows, cols, code)
        if len(_ws_bytes) > 1024:
            _ws_bytes.clear()
        _ws_bytes[key] = got
    return got


def _dense(t):
    """Row-major and 16-byte aligned (a dense view into a larger buffer may start off that grid)."""
    if not t.is_contiguous():
        t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


class _NormGate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, o, g, weight, bias, eps):
        _lib.require_same_device("norm_gate", o=o, g=g, weight=weight, bias=bias)
        if not (o.dtype == g.dtype == weight.dtype == bias.dtype):
            raise TypeError("o, g, weight and bias must share a dtype")
        cols = o.shape[-1]
        if g.shape != o.shape or weight.shape != (cols,) or bias.shape != (cols,):
            raise ValueError("shape mismatch: o %s g %s weight %s bias %s"
                             % (tuple(o.shape), tuple(g.shape), tuple(weight.shape), tuple(bias.shape)))
        code = _lib.dtype_code(o.dtype)
        o2, g2 = _dense(o.reshape(-1, cols)), _dense(g.reshape(-1, cols))
        weight, bias = _dense(weight), _dense(bias)
        rows = o2.shape[0]
        y = torch.empty_like(o2)
        mean = torch.empty((rows,), dtype=torch.float32, device=o.device)
        rstd = torch.empty((rows,), dtype=torch.float32, device=o.device)
        with _lib.on_device(o.device):
            rc = _lib.lib().norm_gate_fwd(o2.data_ptr(), g2.data_ptr(), weight.data_ptr(), bias.data_ptr(), y.data_ptr(),
                                          mean.data_ptr(), rstd.data_ptr(), rows, cols, float(eps), code,
                                          _lib.stream_ptr(o.device))
        _lib.check(rc, "norm_gate_fwd")
        ctx.save_for_backward(o2, g2, weight, bias, mean, rstd)
        ctx.shape = o.shape
        return y.reshape(o.shape)

    @staticmethod
    def backward(ctx, dy):
        o2, g2, weight, bias, mean, rstd = ctx.saved_tensors
        rows, cols = o2.shape
        if dy.device != o2.device:
            raise RuntimeError("norm_gate backward: the upstream gradient is on %s, the inputs on %s" % (dy.device, o2.device))
        dy2 = _dense(dy.to(o2.dtype).reshape(rows, cols))
        code = _lib.dtype_code(o2.dtype)
        d_o, d_g = torch.empty_like(o2), torch.empty_like(g2)
        dw, db = torch.empty_like(weight), torch.empty_like(bias)
        L = _lib.lib()
        with _lib.on_device(o2.device):
            ws_bytes = _workspace_bytes(rows, cols, code)
            ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=o2.device)
            rc = L.norm_gate_bwd(o2.data_ptr(), g2.data_ptr(), weight.data_ptr(), bias.data_ptr(), mean.data_ptr(),
                                 rstd.data_ptr(), dy2.data_ptr(), d_o.data_ptr(), d_g.data_ptr(), dw.data_ptr(), db.data_ptr(),
                                 ws.data_ptr(), ws_bytes, rows, cols, code, _lib.stream_ptr(o2.device))
        _lib.check(rc, "norm_gate_bwd")
        return d_o.reshape(ctx.shape), d_g.reshape(ctx.shape), dw, db, None


def norm_gate(o, g, weight, bias, eps=1e-5):
    """layer_norm(o, (C,), weight, bias, eps) * sigmoid(g) over the last dim; differentiable in
    o, g, weight and bias.  HIP tensors only; see norm_gate_supported for the row widths."""
    ops = _lib.native_ops()
    if (ops is not None and o.is_cuda and o.dtype in _lib._DTYPES and o.dtype == g.dtype == weight.dtype == bias.dtype
            and g.shape == o.shape and o.dim() >= 1 and weight.shape == bias.shape == o.shape[-1:]
            and g.device == o.device and weight.device == o.device and bias.device == o.device):
        return ops.norm_gate(o, g, weight, bias, eps)  # the same operator as a C++ autograd node
    return _NormGate.apply(o, g, weight, bias, eps)
