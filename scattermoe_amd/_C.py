"""ctypes binding of libscattermoe_amd.so — the C ABI declared in include/scattermoe_amd.h.

The library is the product: if it is missing it is built once with hipcc; if that is impossible the
import raises.  There is no PyTorch/CPU fallback behind these calls.
"""
import ctypes
import os
import threading

import torch

from . import _build

_lib = None
_lock = threading.Lock()

F32, BF16, F16 = 0, 1, 2
I64, I32, I16, U8 = 0, 1, 2, 3

_FLOAT_CODES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}
_INDEX_CODES = {torch.int64: I64, torch.int32: I32, torch.int16: I16, torch.uint8: U8}

_p, _i64, _int, _sz, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t, ctypes.c_float

_SIGNATURES = {
    "smoe_version": (_int, []),
    "smoe_last_error": (ctypes.c_char_p, []),
    "smoe_source_hash": (ctypes.c_char_p, []),
    "smoe_route_workspace_bytes": (_sz, [_i64, _int]),
    "smoe_route": (_int, [_p, _int, _i64, _int, _p, _p, _p, _p, _sz, _p]),
    "smoe_route_static_init": (_int, []),
    "smoe_route_static": (_int, [_p, _int, _i64, _int, _p, _p, _p, _p]),
    "smoe_offsets_from_sorted": (_int, [_p, _i64, _int, _p, _p]),
    "smoe_scatter2scatter": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64,
                                    _p, _p, _p, _i64, _i64, _i64, _int, _int, _int, _int, _int, _p]),
    "smoe_scatter2scatter_workspace_bytes": (_sz, [_i64, _i64, _i64, _int, _int]),
    "smoe_scatter2scatter_ws": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64,
                                       _p, _p, _p, _i64, _i64, _i64, _int, _int, _int, _int, _int, _p, _sz, _p]),
    "smoe_group": (_int, [_p, _i64, _i64, _p, _p, _i64, _i64, _p, _i64, _i64, _int, _int, _p]),
    "smoe_group_by_source": (_int, [_p, _i64, _i64, _p, _p, _i64, _i64, _p, _p, _i64, _i64, _int, _int, _p]),
    "smoe_groupXtY": (_int, [_p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _i64,
                             _p, _i64, _i64, _i64, _int, _int, _p]),
    "smoe_groupXtY_gathered": (_int, [_p, _i64, _i64, _p, _i64, _i64, _p, _int, _p, _i64, _i64, _i64, _p, _i64, _i64,
                                      _p, _i64, _i64, _i64, _int, _int, _p]),
    "smoe_combine": (_int, [_p, _i64, _p, _i64, _i64, _p, _i64, _i64, _int, _i64, _int, _p]),
    "smoe_gate_grad": (_int, [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _int, _i64, _int, _p]),
    "smoe_gate_grad_group": (_int, [_p, _i64, _p, _i64, _p, _i64, _i64, _p, _p, _p, _i64, _p, _i64, _i64,
                                    _i64, _int, _i64, _int, _p]),
    "smoe_glu_fwd": (_int, [_p, _i64, _p, _i64, _i64, _i64, _int, _int, _p]),
    "smoe_glu_bwd": (_int, [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _int, _int, _p]),
    "smoe_scatter2scatter_glu": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _i64, _p, _i64, _p, _i64,
                                        _p, _p, _p, _i64, _i64, _i64, _int, _int, _int, _int, _int, _p]),
    "smoe_scatter2scatter_glu_bwd": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _p, _i64,
                                            _p, _p, _p, _i64, _i64, _i64, _int, _int, _int, _p]),
    "smoe_scatter2scatter_oss_glu": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _i64, _p, _i64, _p, _i64,
                                            _p, _p, _p, _i64, _i64, _i64, _int, _int, _int, _f32, _f32, _int, _p]),
    "smoe_scatter2scatter_oss_glu_bwd": (_int, [_p, _i64, _i64, _p, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _p, _p,
                                                _i64, _i64, _i64, _int, _f32, _f32, _int, _p]),
    "smoe_gpt_oss_glu_fwd": (_int, [_p, _i64, _p, _i64, _i64, _i64, _f32, _f32, _int, _p]),
    "smoe_gpt_oss_glu_bwd": (_int, [_p, _i64, _p, _i64, _p, _i64, _i64, _i64, _f32, _f32, _int, _p]),
    "smoe_decode_glu_mlp": (_int, [_p, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _i64,
                                   _p, _i64, _i64, _p, _i64, _i64, _p, _i64, _p, _i64, _i64, _int, _i64, _i64,
                                   _int, _int, _int, _p]),
    "smoe_topk_softmax": (_int, [_p, _i64, _i64, _i64, _int, _int, _int, _p, _i64, _i64, _p, _i64, _i64, _int, _p]),
}

ERR_UNSUPPORTED = -6

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def lib_path():
    return _build.LIB_PATH


def source_hash():
    """Digest of the sources the loaded library was compiled from."""
    return load().smoe_source_hash().decode()


def load():
    """Return the loaded library, building it first if the .so is absent."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(_build.LIB_PATH):
                _build.build()
            lib = ctypes.CDLL(_build.LIB_PATH)
            for name, (res, args) in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = res
                fn.argtypes = args
            if lib.smoe_version() != 1:
                raise RuntimeError("libscattermoe_amd.so ABI version mismatch: %d" % lib.smoe_version())
            built_from = lib.smoe_source_hash().decode()
            if os.path.isdir(_build.CSRC) and built_from != _build.source_hash():
                raise RuntimeError(
                    "libscattermoe_amd.so is stale: built from sources %s, the sources beside it are %s; "
                    "rebuild with `python -m scattermoe_amd._build`" % (built_from, _build.source_hash()))
            _lib = lib
    return _lib


def float_code(dtype):
    try:
        return _FLOAT_CODES[dtype]
    except KeyError:
        raise TypeError("scattermoe_amd kernels support float32/bfloat16/float16, got %s" % dtype)


def index_code(dtype):
    try:
        return _INDEX_CODES[dtype]
    except KeyError:
        raise TypeError("expert indices must be int64/int32/int16/uint8, got %s" % dtype)


def check(rc, what):
    if rc != 0:
        msg = load().smoe_last_error().decode("utf-8", "replace")
        raise RuntimeError("%s failed (code %d): %s" % (what, rc, msg))


def require_gpu(t, what):
    if not t.is_cuda:
        raise RuntimeError(
            "%s: tensor is on %s; the scattermoe_amd kernels run on a ROCm GPU only (no CPU path exists)"
            % (what, t.device))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device):
    """hipStream_t of torch's current stream on `device`, as an integer."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class _NoSwitch:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def on_device(device):
    """Context that makes `device` the current HIP device for a launch; free when it already is (the usual case:
    switching costs several microseconds of host time per launch, which a decode step cannot hide)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_SWITCH
    return torch.cuda.device(device)


def ptr(t):
    return None if t is None else t.data_ptr()
