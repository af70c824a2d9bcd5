"""ctypes binding of liblightning_attn_hip.so (declared in include/lightning_attn_hip.h).

The library is loaded on first use.  A missing library is a hard error: there is
no CPU or eager fallback behind these operators."""
import contextlib
import ctypes
import os
import threading

import torch

_PKG = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
LIB_PATH = os.path.join(_PKG, "_C", "liblightning_attn_hip.so")

LA_BF16, LA_FP16, LA_FP32 = 0, 1, 2
_DTYPES = {torch.bfloat16: LA_BF16, torch.float16: LA_FP16, torch.float32: LA_FP32}

SYMBOLS = (
    "la_init", "la_version", "la_error_string", "la_supported", "la_workspace_bytes",
    "la_fwd", "la_bwd", "la_fwd_strided", "la_bwd_strided", "la_workspace_bytes_opts", "la_fwd_opts", "la_bwd_opts",
    "la_fwd_static", "la_fwd_silu", "la_fwd_silu_supported", "la_saved_state_bytes", "la_saved_state_interval", "la_fwd_save", "la_bwd_saved",
    "srmsnorm_fwd", "srmsnorm_bwd", "norm_gate_supported", "norm_gate_workspace_bytes", "norm_gate_fwd", "norm_gate_bwd",
)

TORCH_LIB_PATH = os.path.join(_PKG, "_C", "liblightning_attn_torch.so")

_lib = None
_lock = threading.RLock()
_native = None          # torch.ops.lightning_attn_hip, False when the binding is absent or switched off
_native_enabled = True

_vp, _i64, _int, _sz, _f = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t, ctypes.c_float

LA_OPT_AUTO, LA_OPT_OFF, LA_OPT_ON, LA_OPT_ALL = 0, 1, 2, 3


class LaunchOpts(ctypes.Structure):
    """la_launch_opts of the header: all zero = the library's own choices."""
    _fields_ = [("chunks", ctypes.c_int32), ("scan", ctypes.c_int32), ("wide", ctypes.c_int32),
                ("paired", ctypes.c_int32), ("once", ctypes.c_int32)]

    def key(self):
        return (self.chunks, self.scan, self.wide, self.paired, self.once)


_tls = threading.local()


def current_opts():
    """The launch options in force on this thread (None: the library's own choices)."""
    return getattr(_tls, "opts", None)


def _tri(v):
    if v == "all":  # (wide only) every column of a sequence in one workgroup, LA_OPT_ALL
        return LA_OPT_ALL
    return LA_OPT_AUTO if v is None else (LA_OPT_ON if v else LA_OPT_OFF)


@contextlib.contextmanager
def launch_opts(chunks=0, scan=None, wide=None, paired=None, once=None, save_states=True):
    """Within the block, the attention operators called from this thread map their work onto
    launches as told (the backward pass of an operator follows the options its forward ran under): `chunks` sequence chunks (0 = library's choice); `scan`, `wide`, `paired`,
    `once` = None (library's choice) / False / True; `save_states` = False: a forward pass that will be
    differentiated keeps its inputs only, as the reference does, instead of also leaving a few states
    for its backward pass (la_fwd_save in the header).  For measurements and tests; the results do
    not depend on it beyond rounding (see la_launch_opts in the header)."""
    prev = current_opts()
    _tls.opts = LaunchOpts(int(chunks or 0), _tri(scan), _tri(wide), _tri(paired), _tri(once))
    _tls.opts.save_states = bool(save_states)
    try:
        yield _tls.opts
    finally:
        _tls.opts = prev


def lib():
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    "liblightning_attn_hip.so is not built (expected at %s); run "
                    "`python lightning-attention_amd/build.py`" % LIB_PATH
                )
            L = ctypes.CDLL(LIB_PATH)
            L.la_init.restype = _int
            L.la_init.argtypes = []
            L.la_version.restype = ctypes.c_char_p
            L.la_version.argtypes = []
            L.la_error_string.restype = ctypes.c_char_p
            L.la_error_string.argtypes = [_int]
            L.la_supported.restype = _int
            L.la_supported.argtypes = [_i64, _i64, _int]
            L.la_workspace_bytes.restype = _sz
            L.la_workspace_bytes.argtypes = [_int, _i64, _i64, _i64, _i64, _i64, _int]
            L.la_fwd.restype = _int
            L.la_fwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]
            L.la_bwd.restype = _int
            L.la_bwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int,
                                 _vp, _sz, _vp]
            L.la_fwd_strided.restype = _int
            L.la_fwd_strided.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]
            L.la_bwd_strided.restype = _int
            L.la_bwd_strided.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64,
                                         _int, _vp, _sz, _vp]
            _op = ctypes.POINTER(LaunchOpts)
            L.la_workspace_bytes_opts.restype = _sz
            L.la_workspace_bytes_opts.argtypes = [_int, _i64, _i64, _i64, _i64, _i64, _int, _op]
            L.la_fwd_opts.restype = _int
            L.la_fwd_opts.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _sz, _op, _vp]
            L.la_bwd_opts.restype = _int
            L.la_bwd_opts.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int,
                                      _vp, _sz, _op, _vp]
            L.la_saved_state_bytes.restype = _sz
            L.la_saved_state_bytes.argtypes = [_i64, _i64, _i64, _i64, _i64, _int, _op]
            L.la_saved_state_interval.restype = _i64
            L.la_saved_state_interval.argtypes = [_i64, _i64, _i64, _i64, _i64, _int, _op]
            L.la_fwd_save.restype = _int
            L.la_fwd_save.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp, _sz, _op,
                                      _vp, _sz, _vp]
            L.la_bwd_saved.restype = _int
            L.la_bwd_saved.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int,
                                       _vp, _sz, _op, _vp, _sz, _vp]
            L.la_fwd_silu_supported.restype = _int
            L.la_fwd_silu_supported.argtypes = [_i64, _i64, _int]
            L.la_fwd_silu.restype = _int
            L.la_fwd_silu.argtypes = L.la_fwd_opts.argtypes
            L.la_fwd_static.restype = _int
            L.la_fwd_static.argtypes = [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _vp]
            L.srmsnorm_fwd.restype = _int
            L.srmsnorm_fwd.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _f, _int, _vp]
            L.srmsnorm_bwd.restype = _int
            L.srmsnorm_bwd.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]
            L.norm_gate_supported.restype = _int
            L.norm_gate_supported.argtypes = [_i64, _int]
            L.norm_gate_workspace_bytes.restype = _sz
            L.norm_gate_workspace_bytes.argtypes = [_i64, _i64, _int]
            L.norm_gate_fwd.restype = _int
            L.norm_gate_fwd.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f, _int, _vp]
            L.norm_gate_bwd.restype = _int
            L.norm_gate_bwd.argtypes = [_vp] * 11 + [_vp, _sz, _i64, _i64, _int, _vp]
            _lib = L
    return _lib


def native_ops():
    """torch.ops.lightning_attn_hip - the operators as C++ autograd functions over the same C ABI
    (csrc/torch_binding.cpp), which cost the host a fraction of what the Python autograd nodes do - or None
    when that library is not built or has been switched off; the Python operators then do the work themselves."""
    global _native
    if not _native_enabled:
        return None
    if _native is None:
        with _lock:
            if _native is None:
                ops = False
                if os.path.exists(TORCH_LIB_PATH) and os.path.exists(LIB_PATH):
                    try:
                        lib()  # the kernel library first: the binding links against it
                        torch.ops.load_library(TORCH_LIB_PATH)
                        ops = torch.ops.lightning_attn_hip
                        ops.attn, ops.srmsnorm, ops.attn_silu, ops.norm_gate  # resolve now
                    except (OSError, RuntimeError, AttributeError):
                        ops = False
                _native = ops
    return _native or None


def use_native_ops(on):
    """Switches the C++ autograd path on or off for this process (tests compare the two paths); returns the
    previous setting."""
    global _native_enabled
    prev, _native_enabled = _native_enabled, bool(on)
    return prev


def dtype_code(dtype):
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError("unsupported dtype %s (bfloat16, float16 or float32)" % dtype) from None


def check(rc, what):
    if rc != 0:
        raise RuntimeError("%s failed: %s (code %d)" % (what, lib().la_error_string(rc).decode(), rc))


def require_gpu(t, what):
    if not t.is_cuda:
        raise RuntimeError(
            "%s runs only on a HIP device: got a %s tensor (there is no CPU fallback; "
            "use lightning_attn.ops.linear_attn / SimpleRMSNormTorch for plain PyTorch)" % (what, t.device)
        )


def require_same_device(what, **tensors):
    """Every tensor whose pointer goes to a kernel must live on one HIP device: a host pointer, or
    one of another GPU, handed to a launch is a memory fault, not a Python error."""
    it = iter(tensors.items())
    name0, t0 = next(it)
    require_gpu(t0, what)
    for name, t in it:
        if t.device != t0.device:
            raise RuntimeError("%s: %s is on %s but %s is on %s; all tensors must be on the same HIP device"
                               % (what, name, t.device, name0, t0.device))


_ws_cache = {}


def workspace_bytes(which, b, h, n, d, e, code, opts):
    """la_workspace_bytes_opts, remembered per shape: the answer depends on the arguments alone."""
    key = (which, b, h, n, d, e, code, opts.key() if opts is not None else None, torch.cuda.current_device())
    got = _ws_cache.get(key)
    if got is None:
        got = lib().la_workspace_bytes_opts(which, b, h, n, d, e, code, ctypes.byref(opts) if opts is not None else None)
        if len(_ws_cache) > 4096:
            _ws_cache.clear()
        _ws_cache[key] = got
    return got


def saved_state_bytes(b, h, n, d, e, code, opts):
    """la_saved_state_bytes, remembered per shape like workspace_bytes; 0 where `opts` turn the states off."""
    if opts is not None and not getattr(opts, "save_states", True):
        return 0
    key = ("saved", b, h, n, d, e, code, opts.key() if opts is not None else None, torch.cuda.current_device())
    got = _ws_cache.get(key)
    if got is None:
        got = lib().la_saved_state_bytes(b, h, n, d, e, code, ctypes.byref(opts) if opts is not None else None)
        if len(_ws_cache) > 4096:
            _ws_cache.clear()
        _ws_cache[key] = got
    return got


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device):
    """hipStream_t of torch's current stream on `device`, as an integer."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)  # no Stream object in between
    return torch.cuda.current_stream(device).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def on_device(device):
    """Context in which `device` is the current HIP device (the library launches on the current one):
    nothing to do, and nothing done, when it already is."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)
