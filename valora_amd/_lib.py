"""ctypes binding of ``libmlora.so`` (declared in ``include/mlora.h``).

There is no CPU fallback: if the library is missing or a call fails, a ``RuntimeError`` is
raised -- the same exception type the reference's extensions surface through ``TORCH_CHECK``
(valora/csrc/lora_ops.cc:27-34,124-125).
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_int, c_int32, c_int64, c_size_t, c_void_p

import torch  # imported first so the process uses torch's HIP runtime (same soname)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmlora.so")

MLORA_F16, MLORA_BF16 = 0, 1
SHRINK_OVERWRITE, SHRINK_ZERO_PAD, SHRINK_ACCUMULATE = 0, 1, 2
REDUCE_IN_EXPAND, ONE_LAUNCH, ONE_LAUNCH_NO_WAIT, SHRINK_RECOMPUTE, EXPAND_COLUMN_LOOP, ONE_LAUNCH_NEVER_READY = 1, 2, 4, 8, 16, 32

# every symbol include/mlora.h declares
SYMBOLS = [
    "mlora_last_error", "mlora_version", "mlora_plan_bytes", "mlora_scratch_bytes", "mlora_one_launch_scratch_bytes",
    "mlora_workspace_bytes", "mlora_tile_lookup", "mlora_tile_fallback", "mlora_build_plan", "mlora_count_consecutive",
    "mlora_ids_from_segments", "mlora_ids_from_requests", "mlora_shrink", "mlora_expand", "mlora_lora_apply",
    "mlora_lora_apply_multi", "mlora_dispatch_bgmv", "mlora_dispatch_bgmv_static",
    "mlora_dispatch_sgmm", "mlora_prefill_shrink", "mlora_prefill_expand",
    "mlora_pool_alloc", "mlora_pool_alloc_contiguous", "mlora_pool_free", "mlora_pool_fill",
    "mlora_pool_scatter_rows", "mlora_pool_gather_rows", "mlora_index_compact", "mlora_merge_adapter",
]


class Pool(ctypes.Structure):
    _fields_ = [("w", c_void_p), ("w_rows", c_int64), ("a_start", c_void_p), ("a_len", c_void_p),
                ("a_loc", c_void_p), ("n_adapters", c_int64), ("a_loc_len", c_int64),
                ("n_slots", c_int32)]


class Target(ctypes.Structure):
    _fields_ = [("y", c_void_p), ("w_b", c_void_p), ("w_b_rows", c_int64), ("slot", c_int32)]


MAX_TARGETS = 4


class Plan(ctypes.Structure):
    _fields_ = [("dev", c_void_p), ("bytes", c_size_t), ("T", c_int64), ("n_adapters", c_int64),
                ("bm_shrink", c_int32), ("bm_expand", c_int32), ("n_slots", c_int32)]


class TileConfig(ctypes.Structure):
    _fields_ = [("bm_shrink", c_int32), ("ksplit", c_int32), ("bm_expand", c_int32), ("flags", c_int32)]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m valora_amd._build` "
            "(hipcc --offload-arch=gfx950); there is no fallback path")
    L = ctypes.CDLL(LIB_PATH)
    L.mlora_last_error.restype = c_char_p
    L.mlora_version.restype = c_int
    for n in ("mlora_plan_bytes", "mlora_scratch_bytes", "mlora_workspace_bytes", "mlora_one_launch_scratch_bytes"):
        getattr(L, n).restype = c_size_t
    L.mlora_plan_bytes.argtypes = [c_int64, c_int64]
    L.mlora_scratch_bytes.argtypes = [c_int64, c_int64, c_int32]
    L.mlora_workspace_bytes.argtypes = [c_int64, c_int64, c_int64]
    L.mlora_one_launch_scratch_bytes.argtypes = [c_int64, c_int64, c_int64, c_int32, c_int32]
    for n in ("mlora_tile_lookup", "mlora_tile_fallback"):
        getattr(L, n).argtypes = [c_int64, c_int64, c_int64, c_int64, POINTER(TileConfig)]
    L.mlora_build_plan.argtypes = [c_void_p, POINTER(Plan), c_void_p, c_int64, c_void_p, c_void_p,
                                   c_int64, c_int32, c_int32, c_int32]
    L.mlora_count_consecutive.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p,
                                          c_void_p, c_void_p, c_void_p, c_void_p]
    L.mlora_ids_from_segments.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64]
    L.mlora_ids_from_requests.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                          c_int64, c_int64]
    L.mlora_shrink.argtypes = [c_void_p, POINTER(Plan), c_void_p, c_size_t, c_void_p, c_int64, c_int64,
                               c_int64, POINTER(Pool), c_int32, c_int32, c_void_p, c_int64, c_int32, c_int32,
                               c_int32, c_int]
    L.mlora_expand.argtypes = [c_void_p, POINTER(Plan), c_void_p, c_int64, c_int64, c_void_p, c_void_p,
                               c_int64, c_int64, POINTER(Pool), c_int32, c_void_p, c_int32, c_int32, c_int]
    L.mlora_lora_apply.argtypes = [c_void_p, POINTER(Plan), c_void_p, c_size_t, c_void_p, c_void_p,
                                   c_int64, c_int64, c_int64, c_int64, POINTER(Pool), POINTER(Pool),
                                   c_int32, c_void_p, c_int32, c_int32, c_int]
    L.mlora_lora_apply_multi.argtypes = [c_void_p, POINTER(Plan), c_void_p, c_size_t, c_void_p, c_int64, c_int64,
                                         c_int64, c_int64, POINTER(Pool), c_int32, POINTER(Target), c_void_p,
                                         c_int32, c_int32, c_int]
    L.mlora_dispatch_bgmv.argtypes = [c_void_p, c_void_p, c_void_p, POINTER(Pool), c_void_p, c_int64,
                                      c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_size_t, POINTER(Plan)]
    L.mlora_dispatch_bgmv_static.argtypes = [c_void_p, c_void_p, c_void_p, POINTER(Pool), c_void_p, c_int64,
                                             c_void_p, c_int64, c_int64, c_int64, c_int]
    L.mlora_dispatch_sgmm.argtypes = [c_void_p, c_void_p, c_void_p, POINTER(Pool), c_void_p, c_int64,
                                      c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                      c_int, c_int32, c_void_p, c_size_t, POINTER(Plan)]
    L.mlora_prefill_shrink.argtypes = [c_void_p, c_void_p, c_void_p, POINTER(Pool), c_void_p, c_void_p,
                                       c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                       c_int64, c_int, c_void_p, c_size_t, POINTER(Plan)]
    L.mlora_prefill_expand.argtypes = [c_void_p, c_void_p, c_void_p, POINTER(Pool), c_void_p, c_void_p,
                                       c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                       c_int64, c_int64, c_int, c_void_p, c_size_t, POINTER(Plan)]
    L.mlora_pool_alloc.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p]
    L.mlora_pool_alloc_contiguous.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p]
    L.mlora_pool_free.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_int64]
    L.mlora_pool_fill.argtypes = [c_void_p, c_void_p, c_int64, c_int32]
    for n in ("mlora_pool_scatter_rows", "mlora_pool_gather_rows"):
        getattr(L, n).argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                  c_int64, c_int32]
    L.mlora_index_compact.argtypes = [c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                                      c_void_p]
    L.mlora_merge_adapter.argtypes = [c_void_p, POINTER(c_void_p), POINTER(c_int32), c_int32, c_int64, c_int64, c_int64,
                                      POINTER(Pool), POINTER(Pool), c_int64, c_int64, ctypes.c_float, c_int32, c_int]
    for n in SYMBOLS[6:]:  # everything after the size queries returns a status
        getattr(L, n).restype = c_int
    _lib = L
    return L


def check(rc: int) -> None:
    if rc != 0:
        msg = lib().mlora_last_error().decode("utf-8", "replace")
        raise RuntimeError(msg or f"libmlora call failed with status {rc}")


def dtype_code(dt: torch.dtype) -> int:
    """Half -> 0, BFloat16 -> 1; anything else has no kernel (valora/csrc/lora_ops.cc:99-125)."""
    if dt == torch.float16:
        return MLORA_F16
    if dt == torch.bfloat16:
        return MLORA_BF16
    return -1


def ptr(t) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device) -> c_void_p:
    """Handle of PyTorch's current stream on ``device`` (the raw getter saves ~4 us per call over building a
    ``torch.cuda.Stream`` object; both name the same stream)."""
    if _raw_stream is not None and device.index is not None:
        return c_void_p(_raw_stream(device.index))
    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


def make_pool(w: torch.Tensor, a_start: torch.Tensor, a_len: torch.Tensor, a_loc: torch.Tensor,
              row_width: int, n_slots: int = 4) -> Pool:
    """``w`` is the pool viewed as rows of ``row_width`` elements (any shape whose trailing dims
    multiply to it -- the reference passes ``[rows, heads, head_dim]``)."""
    n_rows = w.numel() // row_width if row_width > 0 else 0
    return Pool(ptr(w), n_rows, ptr(a_start), ptr(a_len), ptr(a_loc), a_start.numel(), a_loc.numel(),
                n_slots)
