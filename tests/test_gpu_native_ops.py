"""The operators as C++ autograd nodes (csrc/torch_binding.cpp) against the Python autograd path over the same C ABI:
same launches, so outputs and gradients must agree bit for bit, for dense and projection-layout tensors, with and
without decay, under launch options, for float32, and for SimpleRMSNorm.  Arguments the C++ path does not take
(CPU tensors, mismatched shapes) still raise the Python operators' errors."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from lightning_attn.ops import SimpleRMSNorm, lightning_attn_func  # noqa: E402
from lightning_attn.ops.hip import _lib, launch_opts  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402

DEV = "cuda"


def _both_paths(fn):
    """fn() with the C++ nodes, then with the Python nodes."""
    assert _lib.native_ops() is not None, "liblightning_attn_torch.so is not built"
    res = []
    for native in (True, False):
        prev = _lib.use_native_ops(native)
        try:
            res.append(fn())
        finally:
            _lib.use_native_ops(prev)
    return res


@pytest.mark.parametrize("b, h, n, d, e, dtype, decay, token_major, opts", [
    (2, 8, 700, 128, 128, torch.bfloat16, True, False, {}),
    (4, 32, 1024, 128, 128, torch.bfloat16, True, True, {}),          # saved states, projection layout
    (1, 4, 3000, 192, 192, torch.bfloat16, False, False, {}),         # chunks from scanned states, no decay
    (1, 3, 333, 64, 96, torch.float16, True, False, dict(chunks=2)),
    (1, 8, 1024, 64, 64, torch.float32, True, False, {}),
    (4, 32, 1024, 128, 128, torch.bfloat16, True, False, dict(save_states=False)),
])
def test_native_attention_nodes_match_the_python_nodes(b, h, n, d, e, dtype, decay, token_major, opts):
    g = torch.Generator().manual_seed(n)

    def mk(c):
        if token_major:
            return torch.randn(b, n, h, c, generator=g).to(dtype).to(DEV).transpose(1, 2)
        return torch.randn(b, h, n, c, generator=g).to(dtype).to(DEV)

    q, k, v, do = mk(d), mk(d), mk(e), mk(e)
    s = _build_slope_tensor(h).to(DEV) if decay else None

    def run():
        qg, kg, vg = (t.clone().requires_grad_() if not token_major else t.detach().requires_grad_() for t in (q, k, v))
        with launch_opts(**opts):
            o = lightning_attn_func(qg, kg, vg, s)
            o.backward(do)
        torch.cuda.synchronize()
        return o.detach(), qg.grad, kg.grad, vg.grad, o.stride()

    print("native case", (b, h, n, d, e, dtype, decay, token_major, opts), flush=True)
    native, python = _both_paths(run)
    assert native[4] == python[4]  # o in the same memory order
    for name, a, c in zip(("o", "dq", "dk", "dv"), native, python):
        assert torch.equal(a, c), name
    # without gradients
    with torch.no_grad():
        a, c = _both_paths(lambda: lightning_attn_func(q, k, v, s))
    assert torch.equal(a, c) and torch.equal(a, native[0])


@pytest.mark.parametrize("shape, dtype", [((37, 1024), torch.bfloat16), ((2, 50, 2048), torch.float16), ((5, 333), torch.float32)])
def test_native_srmsnorm_node_matches_the_python_node(shape, dtype):
    x = torch.randn(*shape).to(dtype).to(DEV)
    dy = torch.randn(*shape).to(dtype).to(DEV)
    norm = SimpleRMSNorm(shape[-1])

    def run():
        xg = x.clone().requires_grad_()
        y = norm(xg)
        y.backward(dy)
        torch.cuda.synchronize()
        return y.detach(), xg.grad

    (y1, g1), (y0, g0) = _both_paths(run)
    assert torch.equal(y1, y0) and torch.equal(g1, g0)


def test_arguments_the_native_path_does_not_take_raise_as_before():
    q = torch.randn(1, 2, 64, 64, device=DEV).bfloat16()
    s = _build_slope_tensor(2).to(DEV)
    with pytest.raises(RuntimeError, match="HIP device"):
        lightning_attn_func(q.cpu(), q.cpu(), q.cpu(), s.cpu())
    with pytest.raises(ValueError, match="shape mismatch"):
        lightning_attn_func(q, q[:, :, :32], q, s)
    with pytest.raises(TypeError):
        lightning_attn_func(q, q.half(), q, s)
    with pytest.raises(ValueError, match="one rate per head"):
        lightning_attn_func(q, q, q, _build_slope_tensor(4).to(DEV))
    with pytest.raises(RuntimeError, match="64KB"):
        SimpleRMSNorm(40000)(torch.randn(2, 40000, device=DEV).bfloat16())


def test_native_norm_gate_and_silu_forward_match_the_python_paths():
    from lightning_attn.ops import lightning_attn_silu_func
    from lightning_attn.ops.hip import norm_gate

    g = torch.Generator().manual_seed(8)
    rows, cols = 300, 1024
    o, gate, dy = (torch.randn(2, rows // 2, cols, generator=g).bfloat16().to(DEV) for _ in range(3))
    w = (1 + 0.1 * torch.randn(cols, generator=g)).bfloat16().to(DEV)
    b = (0.1 * torch.randn(cols, generator=g)).bfloat16().to(DEV)

    def run():
        leaves = [t.clone().requires_grad_() for t in (o, gate, w, b)]
        y = norm_gate(*leaves, 1e-5)
        y.backward(dy)
        torch.cuda.synchronize()
        return [y.detach()] + [t.grad for t in leaves]

    native, python = _both_paths(run)
    for a, c in zip(native, python):
        assert torch.equal(a, c)
    q, k, v = (torch.randn(2, 6, 500, 128, generator=g).bfloat16().to(DEV) for _ in range(3))
    s = _build_slope_tensor(6).to(DEV)
    a, c = _both_paths(lambda: lightning_attn_silu_func(q, k, v, s))
    assert torch.equal(a, c) and not a.requires_grad
