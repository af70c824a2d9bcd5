"""Host-side behaviour that needs no GPU: the C-ABI library loads and exports
what include/lightning_attn_hip.h declares, argument validation, error paths."""
import ctypes
import os
import re

import pytest
import torch

from lightning_attn.ops import SimpleRMSNorm, lightning_attn_func, lightning_attn2, lightning_attn2_no_decay
from lightning_attn.ops.hip import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "lightning_attn_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:la|srmsnorm|norm_gate)_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert set(names) == set(_lib.SYMBOLS), names
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python lightning-attention_amd/build.py"
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), n


def test_host_only_entry_points():
    L = _lib.lib()
    assert b"gfx950" in L.la_version()
    for d, e, dt, want in ((128, 128, 0, 1), (192, 192, 0, 1), (16, 64, 1, 1), (8, 256, 0, 1), (128, 128, 2, 1),
                           (4, 64, 0, 0), (100, 64, 0, 0), (264, 64, 0, 0), (64, 0, 0, 0), (64, 64, 7, 0)):
        assert L.la_supported(d, e, dt) == want, (d, e, dt)
    assert L.la_error_string(0) == b"success"
    assert b"NULL" in L.la_error_string(-1)
    # scratch for the chunked walk: none when the sequences fill the chip, for short walks or float32;
    # otherwise one d x e (padded) float state per chunk but the last, per sequence and column slice
    assert L.la_workspace_bytes(0, 4, 32, 8192, 128, 128, 0) == 0
    assert L.la_workspace_bytes(1, 4, 32, 8192, 128, 128, 0) == 0
    assert L.la_workspace_bytes(0, 1, 8, 2048, 128, 128, 0) == 0
    assert L.la_workspace_bytes(0, 2, 12, 2048, 192, 192, 0) == 0
    wide_dims = L.la_workspace_bytes(0, 1, 8, 8192, 192, 192, 0)
    assert wide_dims > 0 and wide_dims % (8 * 3 * 192 * 64 * 4) == 0
    assert L.la_workspace_bytes(0, 1, 8, 8192, 128, 128, 2) == 0
    need = L.la_workspace_bytes(0, 1, 8, 8192, 128, 128, 0)
    assert need > 0 and need % (128 * 64 * 4) == 0 and need <= 8 * 2 * 63 * 128 * 64 * 4
    assert L.la_workspace_bytes(1, 1, 8, 8192, 128, 128, 0) >= need
    # argument errors are reported before any launch, so they are testable without a device
    assert L.la_fwd(None, None, None, None, None, 1, 1, 64, 64, 64, 0, None, 0, None) == -1
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    p16 = (p + 15) & ~15
    assert L.la_fwd(p16, p16, p16, None, p16, 1, 1, 64, 100, 64, 0, None, 0, None) == -3
    assert L.la_fwd(p16, p16, p16, None, p16, 1, 0, 64, 64, 64, 0, None, 0, None) == -2
    assert L.la_fwd(p16 + 2, p16, p16, None, p16, 1, 1, 64, 64, 64, 0, None, 0, None) == -5
    assert L.la_bwd(p16, p16, p16, None, None, p16, p16, p16, 1, 1, 64, 64, 64, 0, None, 0, None) == -1
    assert L.srmsnorm_fwd(None, None, None, 4, 64, 64, 1e-6, 0, None) == -1
    assert L.srmsnorm_fwd(p16, p16, p16, 4, 0, 64, 1e-6, 0, None) == -2
    assert L.srmsnorm_fwd(p16, p16, p16, 4, 64, 32, 1e-6, 0, None) == -2
    assert L.srmsnorm_fwd(p16, p16, p16, 4, 64, 64, 1e-6, 9, None) == -3
    # strided entry points: strides in elements, (batch, head, token) per tensor
    dense = [64 * 64, 64 * 64, 64] * 4
    def st(vals):
        return (ctypes.c_int64 * len(vals))(*vals)
    assert L.la_fwd_strided(p16, p16, p16, None, p16, None, 1, 1, 64, 64, 64, 0, None, 0, None) == -1
    assert L.la_fwd_strided(None, p16, p16, None, p16, st(dense), 1, 1, 64, 64, 64, 0, None, 0, None) == -1
    bad = list(dense); bad[2] = 68  # token stride not a multiple of 16 bytes
    assert L.la_fwd_strided(p16, p16, p16, None, p16, st(bad), 1, 1, 64, 64, 64, 0, None, 0, None) == -5
    bad = list(dense); bad[5] = 32  # token stride below the feature dim
    assert L.la_fwd_strided(p16, p16, p16, None, p16, st(bad), 1, 1, 64, 64, 64, 0, None, 0, None) == -2
    bad = list(dense); bad[11] = 1 << 26  # one sequence would span more than 2 GiB
    assert L.la_fwd_strided(p16, p16, p16, None, p16, st(bad), 1, 1, 64, 64, 64, 0, None, 0, None) == -2
    bad = list(dense); bad[2] = 128  # float32 tensors must be plain
    assert L.la_fwd_strided(p16, p16, p16, None, p16, st(bad), 1, 1, 64, 64, 64, 2, None, 0, None) == -3
    assert L.la_bwd_strided(p16, p16, p16, None, p16, p16, p16, p16, None, 1, 1, 64, 64, 64, 0, None, 0, None) == -1
    assert L.la_fwd_strided(p16, p16, p16, None, p16, st(dense), 0, 4, 64, 64, 64, 0, None, 0, None) == 0
    # empty problems succeed without touching the device
    assert L.la_fwd(p16, p16, p16, None, p16, 0, 4, 64, 64, 64, 0, None, 0, None) == 0
    assert L.srmsnorm_bwd(p16, p16, p16, p16, 0, 64, 64, 0, None) == 0


def test_workspace_query_is_consistent():
    """Properties of the scratch size over a grid of shapes (host logic only; without a device the library
    plans for 256 CUs): a whole number of state slots, never more than 63 of them per sequence, sweep and
    column slice, nothing for float32 or when the sequences fill the chip by themselves, nothing when
    scanned chunk states are switched off, and the backward pass never asks for less than the forward."""
    L = _lib.lib()
    seen_some = False
    for b, h in ((1, 1), (1, 8), (2, 12), (1, 32), (4, 32), (8, 64)):
        for n in (64, 1000, 4096, 65536):
            for d in (8, 64, 128, 192, 256):
                for e in (d, 64):
                    fwd = L.la_workspace_bytes(0, b, h, n, d, e, 0)
                    bwd = L.la_workspace_bytes(1, b, h, n, d, e, 0)
                    assert L.la_workspace_bytes(0, b, h, n, min(d, 128), min(e, 128), 2) == 0  # float32
                    assert fwd % 16 == 0 and bwd % 16 == 0 and bwd >= fwd
                    # one slot: (feature dim padded to 64 / 128 / 192 / 256) x (64 or 128 columns) floats
                    cap = lambda dk, dv: b * h * 2 * ((dv + 63) // 64) * 63 * max(128, -(-dk // 64) * 64) * 128 * 4
                    assert fwd <= cap(d, e) and bwd <= max(cap(e, d), cap(d, e))
                    if b * h >= 256 or n <= 64:
                        assert fwd == 0 and bwd == 0
                    seen_some = seen_some or fwd > 0
    assert seen_some
    assert L.la_workspace_bytes(0, 1, 8, 65536, 128, 128, 0) > 0
    no_scan = _lib.LaunchOpts(0, _lib.LA_OPT_OFF, 0, 0, 0)
    assert L.la_workspace_bytes_opts(0, 1, 8, 65536, 128, 128, 0, ctypes.byref(no_scan)) == 0
    assert L.la_workspace_bytes_opts(1, 1, 8, 65536, 192, 192, 0, ctypes.byref(no_scan)) == 0
    # NULL options = the plain query; a forced chunk count sizes the workspace for that count
    assert L.la_workspace_bytes_opts(0, 1, 8, 65536, 128, 128, 0, None) == L.la_workspace_bytes(0, 1, 8, 65536, 128, 128, 0)
    forced = _lib.LaunchOpts(5, 0, _lib.LA_OPT_OFF, 0, 0)
    assert L.la_workspace_bytes_opts(0, 4, 32, 8192, 128, 128, 0, ctypes.byref(forced)) == 128 * 2 * 4 * 128 * 64 * 4
    # shapes the entry points reject need no workspace; neither do malformed options
    assert L.la_workspace_bytes(0, 1, 8, 1 << 22, 128, 128, 0) == 0
    assert L.la_workspace_bytes(0, 1, 8, 8192, 100, 128, 0) == 0
    bad = _lib.LaunchOpts(0, 7, 0, 0, 0)
    assert L.la_workspace_bytes_opts(0, 1, 8, 65536, 128, 128, 0, ctypes.byref(bad)) == 0


def test_saved_state_query_is_consistent():
    """Properties of la_saved_state_bytes / la_saved_state_interval over a grid of shapes (host logic only; 256 CUs
    assumed without a device): a whole number m of d x e float matrices per sequence, boundaries a multiple of 64
    tokens apart and all inside the sequence, m + 1 chunks that give every CU at most one workgroup; nothing for
    float32, for feature dims the pair has no kernel forms for, for shapes whose sequences fill the chip or leave it
    to the chunked plans, and nothing when the launch options pin another form."""
    L = _lib.lib()
    used = set()
    for b, h in ((1, 8), (2, 12), (1, 64), (3, 24), (4, 20), (4, 32), (5, 32), (8, 32)):
        for n in (64, 512, 1000, 1536, 4096, 8192, 65536):
            for d, e in ((64, 64), (72, 128), (128, 128), (128, 96), (96, 160), (136, 136), (192, 192), (176, 144), (192, 128), (256, 256)):
                for dtype in (0, 1, 2):
                    if dtype == 2 and (d > 128 or e > 128):
                        continue
                    nbytes = L.la_saved_state_bytes(b, h, n, d, e, dtype, None)
                    step = L.la_saved_state_interval(b, h, n, d, e, dtype, None)
                    assert (nbytes == 0) == (step == 0)
                    small = 64 < d <= 128 and 96 < e <= 128  # (e <= 96: the forward pass takes one 128-column workgroup per sequence)
                    big = 128 < d <= 192 and 128 < e <= 192
                    units8 = (b * h + 7) // 8 * 8
                    if big and units8 * 3 <= 256:  # the forward pass then runs in 64-column workgroups: no form that saves
                        big = False
                    if dtype == 2 or not (small or big) or not 64 < b * h <= 128 or n < 1536:  # (short walks: not worth it)
                        assert nbytes == 0, (b, h, n, d, e, dtype)
                        continue
                    assert nbytes > 0, (b, h, n, d, e, dtype)
                    m, rest = divmod(nbytes, b * h * d * e * 4)
                    assert rest == 0 and m >= 1 and step % 64 == 0
                    assert m * step < n <= (m + 1) * step + 63
                    assert (b * h + 7) // 8 * 8 * (m + 1) <= 256
                    used.add((small, big))
                    for kw in (dict(chunks=2), dict(wide=_lib.LA_OPT_ON), dict(wide=_lib.LA_OPT_ALL), dict(scan=_lib.LA_OPT_ON)):
                        o = _lib.LaunchOpts(kw.get("chunks", 0), kw.get("scan", 0), kw.get("wide", 0), 0, 0)
                        assert L.la_saved_state_bytes(b, h, n, d, e, dtype, ctypes.byref(o)) == 0
    assert used == {(True, False), (False, True)}
    # the headline shape: one matrix of 128 x 128 floats per sequence, at the middle of the sequence
    assert L.la_saved_state_bytes(4, 32, 8192, 128, 128, 0, None) == 128 * 128 * 128 * 4
    assert L.la_saved_state_interval(4, 32, 8192, 128, 128, 0, None) == 4096
    assert L.la_saved_state_bytes(4, 32, 8192, 192, 192, 0, None) == 128 * 192 * 192 * 4


def test_static_scratch_holds_every_plan_of_the_forward():
    """la_fwd_static rejects shapes whose plan needs more than its static array (LA_E_WORKSPACE): over a
    grid of shapes, on a chip of 256 compute units (what the library plans for without a device), no
    forward plan does, so nothing that la_fwd accepts is turned away there."""
    L = _lib.lib()
    text = open(HEADER).read()
    cap = re.search(r"#define LA_STATIC_SCRATCH_BYTES \((\d+)u << (\d+)\)", text)
    cap = int(cap.group(1)) << int(cap.group(2))
    assert cap == 48 << 20
    worst = 0
    for b, h in ((1, 1), (1, 2), (1, 3), (1, 4), (1, 8), (2, 12), (1, 16), (1, 32), (3, 5), (1, 64), (1, 120)):
        for n in (1000, 4096, 8192, 65536, 1 << 20):
            for d in (64, 128, 192, 256):
                for e in (64, 128, 192, 256):
                    worst = max(worst, L.la_workspace_bytes(0, b, h, n, d, e, 0))
    assert 0 < worst <= cap
    assert b"workspace" in L.la_error_string(-4)
    # its argument checks are la_fwd's and run before the device is touched
    buf = ctypes.create_string_buffer(64)
    p16 = (ctypes.addressof(buf) + 15) & ~15
    assert L.la_fwd_static(None, p16, p16, None, p16, 1, 1, 64, 64, 64, 0, None) == -1
    assert L.la_fwd_static(p16, p16, p16, None, p16, 1, 1, 64, 100, 64, 0, None) == -3
    assert L.la_fwd_static(p16, p16, p16, None, p16, 0, 1, 64, 64, 64, 0, None) == 0


def test_launch_options():
    """la_launch_opts is validated on the host before anything is launched, and the Python context
    that carries it restores the previous options on exit (also when nested)."""
    L = _lib.lib()
    buf = ctypes.create_string_buffer(64)
    p16 = (ctypes.addressof(buf) + 15) & ~15
    bad = _lib.LaunchOpts(0, 0, 5, 0, 0)
    assert L.la_fwd_opts(p16, p16, p16, None, p16, None, 1, 1, 64, 64, 64, 0, None, 0, ctypes.byref(bad), None) == -2
    neg = _lib.LaunchOpts(-1, 0, 0, 0, 0)
    assert L.la_bwd_opts(p16, p16, p16, None, p16, p16, p16, p16, None, 1, 1, 64, 64, 64, 0, None, 0, ctypes.byref(neg), None) == -2
    assert L.la_fwd_opts(None, p16, p16, None, p16, None, 1, 1, 64, 64, 64, 0, None, 0, None, None) == -1
    from lightning_attn.ops.hip import launch_opts
    assert _lib.current_opts() is None
    with launch_opts(chunks=3, wide=True) as outer:
        assert outer.key() == (3, 0, 2, 0, 0) and _lib.current_opts() is outer
        with launch_opts(scan=False, paired=False, once=True) as inner:
            assert inner.key() == (0, 1, 0, 1, 2) and _lib.current_opts() is inner
        assert _lib.current_opts() is outer
    assert _lib.current_opts() is None


class _FakeTensor:
    def __init__(self, device):
        self.device = torch.device(device)
        self.is_cuda = self.device.type == "cuda"


def test_tensors_must_share_a_device():
    """A host pointer (or one of another GPU) must never reach a launch: the check that stops it
    runs on the host, so stand-in objects with a device are enough to exercise it."""
    ok = _FakeTensor("cuda:0")
    _lib.require_same_device("op", q=ok, k=_FakeTensor("cuda:0"), v=ok)
    with pytest.raises(RuntimeError, match="same HIP device"):
        _lib.require_same_device("op", q=ok, k=_FakeTensor("cpu"), v=ok)
    with pytest.raises(RuntimeError, match="same HIP device"):
        _lib.require_same_device("op", q=ok, k=ok, v=_FakeTensor("cuda:1"))
    with pytest.raises(RuntimeError, match="HIP device"):
        _lib.require_same_device("op", q=_FakeTensor("cpu"), k=ok, v=ok)


def test_no_cpu_fallback():
    q = torch.randn(1, 2, 16, 16)
    with pytest.raises(RuntimeError, match="HIP device"):
        lightning_attn_func(q, q, q, torch.ones(2, 1, 1))
    with pytest.raises(RuntimeError, match="HIP device"):
        lightning_attn2_no_decay(q, q, q)
    with pytest.raises(RuntimeError, match="HIP device"):
        SimpleRMSNorm(16)(q)
    with pytest.raises(ValueError):
        lightning_attn2(q, q, q, None)


def test_interface_validation():
    q = torch.randn(1, 2, 16, 0)
    with pytest.raises(AssertionError):
        lightning_attn_func(q, q, q)  # no features at all
    with pytest.raises(ValueError):
        lightning_attn_func(torch.randn(1, 2, 16, 16), torch.randn(1, 2, 16, 16), torch.randn(1, 2, 16, 16), None, "ring")


def test_missing_library_is_an_error(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/liblightning_attn_hip.so")
    with pytest.raises(RuntimeError, match="not built"):
        _lib.lib()


def test_triton_import_path_is_an_alias_of_the_hip_operators():
    """lightning_attn/ops/triton/__init__.py:1-4 of the reference exports its operators under
    lightning_attn.ops.triton; the same imports work here and name the HIP operators."""
    from lightning_attn.ops import hip
    from lightning_attn.ops.triton import SimpleRMSNorm as S1, lightning_attn2 as a1, lightning_attn2_no_decay as a2
    from lightning_attn.ops.triton import lightning_attn2_parallel as a3
    from lightning_attn.ops.triton.lightning_attn2 import LightningAttention2, lightning_attn2 as b1
    from lightning_attn.ops.triton.lightning_attn2_no_decay import lightning_attn2_no_decay as b2
    from lightning_attn.ops.triton.lightning_attn2_parallel import lightning_attn2_parallel as b3
    from lightning_attn.ops.triton.srmsnorm import SimpleRMSNorm as S2, _SrmsNorm
    assert S1 is hip.SimpleRMSNorm and S2 is S1 and _SrmsNorm is hip._SrmsNorm
    assert LightningAttention2 is hip.LightningAttention2
    for f in (a1, a2, a3, b1, b2, b3):
        assert callable(f)
    assert a1 is hip.lightning_attn2 and a2 is hip.lightning_attn2_no_decay and a3 is hip.lightning_attn2_parallel


def test_triton_package_names_stay_operators_after_submodule_imports():
    """Importing a submodule first (as `from lightning_attn.ops.triton.lightning_attn2 import ...` does) must not
    turn the package attribute of the same name into the module: checked in a fresh interpreter."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys; sys.path[:0] = %r\n"
        "import lightning_attn.ops.triton.lightning_attn2\n"
        "import lightning_attn.ops.triton.lightning_attn2_no_decay\n"
        "import lightning_attn.ops.triton.lightning_attn2_parallel\n"
        "import lightning_attn.ops.triton.srmsnorm\n"
        "import lightning_attn.ops.triton as t\n"
        "from lightning_attn.ops.triton import lightning_attn2, lightning_attn2_no_decay, lightning_attn2_parallel\n"
        "import types\n"
        "for f in (lightning_attn2, lightning_attn2_no_decay, lightning_attn2_parallel, t.lightning_attn2):\n"
        "    assert callable(f) and not isinstance(f, types.ModuleType), f\n"
        "assert isinstance(t.SimpleRMSNorm, type)\n"
    ) % ([os.path.join(root, "lightning-attention_amd"), root],)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
