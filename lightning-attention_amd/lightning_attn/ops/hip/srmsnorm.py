"""SimpleRMSNorm over the HIP row kernels; interface of
lightning_attn/ops/triton/srmsnorm.py:76-185."""
import torch

from . import _lib


class _SrmsNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, eps):
        _lib.require_gpu(x, "SimpleRMSNorm")
        # eps too small for fp16 (srmsnorm.py:80-81)
        if x.dtype == torch.float16:
            eps = max(eps, 1.6e-5)
        x_arg = x.reshape(-1, x.shape[-1])
        if not x_arg.is_contiguous():
            x_arg = x_arg.contiguous()
        rows, cols = x_arg.shape
        # same bound as the reference: one row may not exceed 64 KB (srmsnorm.py:94-97)
        if cols > 65536 // x.element_size():
            raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
        y = torch.empty_like(x_arg)
        rstd = torch.empty((rows,), dtype=torch.float32, device=x.device)
        L = _lib.lib()
        with _lib.on_device(x.device):
            # (torch reports an arbitrary stride for a dim of size <= 1)
            rc = L.srmsnorm_fwd(x_arg.data_ptr(), y.data_ptr(), rstd.data_ptr(), rows, cols, x_arg.stride(0) if rows > 1 else cols,
                                float(eps), _lib.dtype_code(x.dtype), _lib.stream_ptr(x.device))
        _lib.check(rc, "srmsnorm_fwd")
        ctx.save_for_backward(x, rstd)
        return y.reshape(x.shape)

    @staticmethod
    def backward(ctx, dy):
        x, rstd = ctx.saved_tensors
        x_arg = x.reshape(-1, x.size(-1))
        if not x_arg.is_contiguous():
            x_arg = x_arg.contiguous()
        rows, cols = x_arg.shape
        if dy.device != x.device:
            raise RuntimeError("SimpleRMSNorm backward: the upstream gradient is on %s, x on %s" % (dy.device, x.device))
        dy = dy.contiguous()
        if dy.dtype != x.dtype:
            dy = dy.to(x.dtype)
        assert dy.numel() == x.numel(), (
            "Something is wrong in the backward graph, possibly because of an inplace operation after the layernorm"
        )
        dx = torch.empty_like(dy)
        L = _lib.lib()
        with _lib.on_device(x.device):
            rc = L.srmsnorm_bwd(x_arg.data_ptr(), dy.data_ptr(), rstd.data_ptr(), dx.data_ptr(), rows, cols,
                                x_arg.stride(0) if rows > 1 else cols, _lib.dtype_code(x.dtype), _lib.stream_ptr(x.device))
        _lib.check(rc, "srmsnorm_bwd")
        return dx.reshape(dy.shape), None


class SimpleRMSNorm(torch.nn.Module):
    """y = x / sqrt(mean(x^2, -1) + eps), no learnable scale (srmsnorm.py:178-185)."""

    def __init__(self, dim: int, eps: float = 1e-6):
        super().__init__()
        self.eps = eps
        self.dim = dim

    def forward(self, x):
        ops = _lib.native_ops()
        if ops is not None and x.is_cuda and x.dtype in _lib._DTYPES and x.dim() >= 1:
            return ops.srmsnorm(x, self.eps)  # the same operator as a C++ autograd node
        return _SrmsNorm.apply(x, self.eps)
