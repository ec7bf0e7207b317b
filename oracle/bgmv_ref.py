"""ctypes front end of ``oracle/bgmv_ref.c`` (index-literal C restatement of the reference
BGMV kernels).  TEST INFRASTRUCTURE ONLY -- see the header of ``bgmv_ref.c``."""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libbgmv_ref.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "_build/libbgmv_ref.so"], check=True, capture_output=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.bgmv_ref_to_float.restype = ctypes.c_float
        _lib.bgmv_ref_to_float.argtypes = [ctypes.c_uint16, ctypes.c_int]
        _lib.bgmv_ref_from_float.restype = ctypes.c_uint16
        _lib.bgmv_ref_from_float.argtypes = [ctypes.c_float, ctypes.c_int]
    return _lib


def _p(t: torch.Tensor):
    assert t.device.type == "cpu" and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _dt(t: torch.Tensor) -> int:
    return {torch.float16: 0, torch.bfloat16: 1}[t.dtype]


def _i64(t):
    return t.to("cpu").to(torch.int64).contiguous()


def shrink(y, x, w, a_start, a_len, a_loc, ids, qkvo):
    """Returns a new y; arguments as in ``dispatch_bgmv`` with ``h_in > h_out``."""
    out = y.clone().contiguous()
    x = x.contiguous(); w = w.contiguous()
    a_start, a_len, a_loc, ids = map(_i64, (a_start, a_len, a_loc, ids))
    rc = lib().bgmv_ref_shrink(_p(out), _p(x), _p(w), _p(a_start), _p(a_len), _p(a_loc), _p(ids),
                               ctypes.c_int64(qkvo), ctypes.c_int64(x.shape[0]),
                               ctypes.c_int64(x.shape[1]), ctypes.c_int64(out.shape[1]), _dt(x))
    assert rc == 0
    return out


def expand(y, x, w, a_start, a_len, a_loc, ids, qkvo, scales):
    out = y.clone().contiguous()
    x = x.contiguous(); w = w.contiguous(); scales = scales.to(x.dtype).contiguous()
    a_start, a_len, a_loc, ids = map(_i64, (a_start, a_len, a_loc, ids))
    rc = lib().bgmv_ref_expand(_p(out), _p(x), _p(w), _p(a_start), _p(a_len), _p(a_loc), _p(ids),
                               ctypes.c_int64(qkvo), _p(scales), ctypes.c_int64(x.shape[0]),
                               ctypes.c_int64(x.shape[1]), ctypes.c_int64(out.shape[1]), _dt(x))
    assert rc == 0
    return out
