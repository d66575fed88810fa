"""ctypes binding of libstreaming_attention.so (the C ABI in include/streaming_attention.h).

The library is the only compute path: if it cannot be loaded the operator raises, it
never falls back to a PyTorch implementation.
"""
from __future__ import annotations

import ctypes
import os
import threading

_LIB_NAME = "libstreaming_attention.so"
_lock = threading.Lock()
_lib = None

DTYPE_IDS = {"torch.float32": 0, "torch.float16": 1, "torch.bfloat16": 2}

_vp, _i32, _i64, _f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_pi64 = ctypes.POINTER(ctypes.c_int64)

# name -> argument types, in the order of include/streaming_attention.h
SIGNATURES = {
    "sa_forward": [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _pi64, _pi64, _pi64,
                   _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp],
    "sa_bwd_delta": [_vp, _vp, _vp, _pi64, _pi64, _i32, _i32, _i32, _i32, _i32, _vp],
    "sa_bwd_dq": [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _pi64, _pi64, _pi64, _pi64,
                  _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp],
    "sa_bwd_dkdv": [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _pi64, _pi64, _pi64, _pi64,
                    _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp],
    "sa_backward": [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                    _pi64, _pi64, _pi64, _pi64, _pi64,
                    _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp],
    "sa_backward_static": [_vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp,
                           _pi64, _pi64, _pi64, _pi64, _pi64,
                           _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp],
    "sa_query": [_i32],
    "sa_launch_choice": [_i32, _i32, _i32, _i32],
    "sa_tune_override": [_i32, _i32],
    "sa_error_string": [_i32],
}


def library_path() -> str:
    return os.environ.get(
        "STREAMING_ATTENTION_LIB",
        os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME),
    )


def load() -> ctypes.CDLL:
    """Load the shared library once and attach argument types to its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not os.path.exists(path):
            raise RuntimeError(
                f"{_LIB_NAME} not found at {path}: build it with `make -C kernels_amd/csrc` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'`). "
                "There is no fallback implementation."
            )
        lib = ctypes.CDLL(path)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_char_p if name == "sa_error_string" else ctypes.c_int
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().sa_error_string(rc).decode()
        raise RuntimeError(f"{what} failed with code {rc}: {msg}")


_stride_cache: dict = {}


def strides4(t) -> ctypes.Array:
    """The four element strides of ``t`` as an int64[4]; arrays are cached per stride tuple (the
    library only reads them)."""
    key = t.stride()
    arr = _stride_cache.get(key)
    if arr is None:
        if len(_stride_cache) > 4096:
            _stride_cache.clear()
        arr = _stride_cache[key] = (ctypes.c_int64 * 4)(*key)
    return arr
