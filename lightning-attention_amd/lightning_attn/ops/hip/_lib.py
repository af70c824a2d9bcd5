"""ctypes binding of liblightning_attn_hip.so (declared in include/lightning_attn_hip.h).

The library is loaded on first use.  A missing library is a hard error: there is
no CPU or eager fallback behind these operators."""
import ctypes
import os
import threading

import torch

_PKG = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
LIB_PATH = os.path.join(_PKG, "_C", "liblightning_attn_hip.so")

LA_BF16, LA_FP16, LA_FP32 = 0, 1, 2
_DTYPES = {torch.bfloat16: LA_BF16, torch.float16: LA_FP16, torch.float32: LA_FP32}

SYMBOLS = (
    "la_version", "la_error_string", "la_supported", "la_workspace_bytes",
    "la_fwd", "la_bwd", "la_fwd_strided", "la_bwd_strided", "srmsnorm_fwd", "srmsnorm_bwd",
)

_lib = None
_lock = threading.Lock()

_vp, _i64, _int, _sz, _f = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t, ctypes.c_float


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
            L.srmsnorm_fwd.restype = _int
            L.srmsnorm_fwd.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _f, _int, _vp]
            L.srmsnorm_bwd.restype = _int
            L.srmsnorm_bwd.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]
            _lib = L
    return _lib


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
