"""Pins of the gated-norm oracle (CPU): the library-routine form against the written-out formulas the
device kernel evaluates, autograd against the hand-derived gradients, gradcheck in float64, and the
special cases that reduce it to something simpler."""
import torch

import oracle


def _inputs(rows, cols, seed=0, dtype=torch.float64):
    g_ = torch.Generator().manual_seed(seed)
    o = torch.randn(rows, cols, generator=g_, dtype=dtype) * 3 + 0.7
    g = torch.randn(rows, cols, generator=g_, dtype=dtype) * 2
    w = torch.randn(cols, generator=g_, dtype=dtype)
    b = torch.randn(cols, generator=g_, dtype=dtype)
    dy = torch.randn(rows, cols, generator=g_, dtype=dtype)
    return o, g, w, b, dy


def test_library_form_equals_written_out_formulas():
    o, g, w, b, dy = _inputs(37, 96)
    auto = oracle.norm_gate_fwd_bwd(o, g, w, b, dy, eps=1e-5, dtype=torch.float64)
    closed = oracle.norm_gate_closed_form(o, g, w, b, dy, eps=1e-5)
    for name, a, c in zip(("y", "d_o", "d_g", "d_weight", "d_bias"), auto, closed):
        torch.testing.assert_close(a, c, rtol=1e-10, atol=1e-10, msg=name)


def test_gradcheck_float64():
    o, g, w, b, _ = _inputs(5, 8, seed=1)
    leaves = [t.clone().requires_grad_() for t in (o, g, w, b)]
    assert torch.autograd.gradcheck(lambda *a: oracle.norm_gate_ref(*a, eps=1e-5, dtype=torch.float64), leaves)


def test_special_cases():
    o, g, w, b, _ = _inputs(9, 64, seed=2)
    # a wide-open gate leaves the plain LayerNorm; a shut one leaves zero
    y_open = oracle.norm_gate_ref(o, torch.full_like(g, 40.0), w, b, dtype=torch.float64)
    torch.testing.assert_close(y_open, torch.nn.functional.layer_norm(o, (64,), w, b, 1e-5))
    assert oracle.norm_gate_ref(o, torch.full_like(g, -800.0), w, b, dtype=torch.float64).abs().max() == 0
    # g = 0 halves; weight 1 / bias 0 gives rows of mean 0 and variance 1 - eps * rstd^2
    y = oracle.norm_gate_ref(o, torch.zeros_like(g), torch.ones_like(w), torch.zeros_like(b), eps=1e-5, dtype=torch.float64) * 2
    assert y.mean(-1).abs().max() < 1e-12
    var = o.var(-1, unbiased=False)
    torch.testing.assert_close(y.pow(2).mean(-1), var / (var + 1e-5))
    # shifting or scaling a row of o changes nothing (up to eps)
    y0 = oracle.norm_gate_ref(o, g, w, b, eps=0.0, dtype=torch.float64)
    y1 = oracle.norm_gate_ref(o * 7.5 + 3.0, g, w, b, eps=0.0, dtype=torch.float64)
    torch.testing.assert_close(y0, y1, rtol=1e-9, atol=1e-9)


def test_row_gradient_is_orthogonal_to_constants_and_to_the_row():
    """d_o of a LayerNorm sums to zero over a row and is orthogonal to the normalised row."""
    o, g, w, b, dy = _inputs(11, 40, seed=3)
    _, d_o, _, _, _ = oracle.norm_gate_closed_form(o, g, w, b, dy, eps=0.0)
    assert d_o.sum(-1).abs().max() < 1e-10
    xh = (o - o.mean(-1, keepdim=True))
    assert (d_o * xh).sum(-1).abs().max() < 1e-9
