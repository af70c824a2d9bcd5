"""la_fwd_static: the forward entry point that allocates nothing (its chunk states live in a static
device array inside the library) against la_fwd with a caller-supplied workspace, through the C ABI.

Both run the same plan on the same kernels, so the outputs must agree bit for bit.  Two calls in a
row share the array; the second one is smaller, so whatever the first left behind in the part it
does not overwrite must not matter."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from lightning_attn.ops.hip import _lib  # noqa: E402
from lightning_attn.utils import _build_slope_tensor  # noqa: E402

DEV = "cuda"


def _inputs(b, h, n, d, e, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    q, k = ((torch.randn(b, h, n, d, generator=g, device=DEV) * 0.5).bfloat16() for _ in range(2))
    v = torch.randn(b, h, n, e, generator=g, device=DEV).bfloat16()
    return q, k, v


def _la_fwd(L, q, k, v, s, ws_bytes):
    b, h, n, d = q.shape
    e = v.shape[-1]
    o = torch.full_like(v, float("nan"))
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    rc = L.la_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr() if s is not None else None, o.data_ptr(),
                  b, h, n, d, e, 0, ws.data_ptr() if ws_bytes else None, ws_bytes, st)
    assert rc == 0, L.la_error_string(rc)
    return o


def _la_fwd_static(L, q, k, v, s):
    b, h, n, d = q.shape
    e = v.shape[-1]
    o = torch.full_like(v, float("nan"))
    st = torch.cuda.current_stream().cuda_stream
    rc = L.la_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr() if s is not None else None,
                         o.data_ptr(), b, h, n, d, e, 0, st)
    assert rc == 0, L.la_error_string(rc)
    return o


def test_static_scratch_forward_matches_workspace_forward():
    L = _lib.lib()
    # (b, h, n, d, e): few long sequences, so that the walk is cut into chunks from scanned states;
    # the second call is smaller than the first and uses less of the array
    shapes = [(1, 8, 8192, 128, 128), (1, 4, 4101, 128, 64), (1, 2, 6000, 192, 192)]
    results = []
    for i, (b, h, n, d, e) in enumerate(shapes):
        need = L.la_workspace_bytes(0, b, h, n, d, e, 0)
        assert 0 < need <= 48 << 20, (b, h, n, d, e, need)
        q, k, v = _inputs(b, h, n, d, e, 100 + i)
        s = _build_slope_tensor(h).to(DEV).float().contiguous() if i != 1 else None
        print("la_fwd_static case", (b, h, n, d, e), "workspace bytes", need, flush=True)
        got = _la_fwd_static(L, q, k, v, s)
        results.append((q, k, v, s, need, got))
    torch.cuda.synchronize()
    # the property the entry point exists for: a call allocates no device memory (the outputs are
    # made first; the first calls above have looked the array's address up already)
    outs = [torch.full_like(v, float("nan")) for (_, _, v, _, _, _) in results]
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    reserved0 = torch.cuda.memory_reserved()
    st = torch.cuda.current_stream().cuda_stream
    for (q, k, v, s, _, _), o in zip(results, outs):
        b, h, n, d = q.shape
        rc = L.la_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), s.data_ptr() if s is not None else None,
                             o.data_ptr(), b, h, n, d, v.shape[-1], 0, st)
        assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_reserved() == reserved0
    for (_, _, _, _, _, got), o in zip(results, outs):
        assert torch.equal(got, o)
    for q, k, v, s, need, got in results:
        want = _la_fwd(L, q, k, v, s, need)
        torch.cuda.synchronize()
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got, want), tuple(q.shape)


def test_static_scratch_forward_without_chunks_and_argument_errors():
    """A shape whose plan uses no scratch at all, and the host-side argument checks of la_fwd."""
    L = _lib.lib()
    b, h, n, d, e = 2, 40, 300, 64, 64
    assert L.la_workspace_bytes(0, b, h, n, d, e, 0) == 0
    q, k, v = _inputs(b, h, n, d, e, 7)
    s = _build_slope_tensor(h).to(DEV).float().contiguous()
    got = _la_fwd_static(L, q, k, v, s)
    want = _la_fwd(L, q, k, v, s, 0)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    assert L.la_fwd_static(None, k.data_ptr(), v.data_ptr(), None, got.data_ptr(), b, h, n, d, e, 0, None) == -1
    assert L.la_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), None, got.data_ptr(), b, h, n, 100, e, 0, None) == -3
