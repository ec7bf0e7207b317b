"""Drop-in for the reference's BGMV extension ``valora._kernels``.

``dispatch_bgmv`` keeps the reference's positional signature, argument meaning, in-place
behaviour and error behaviour (valora/csrc/lora_ops.cc:76-126); the work is done by the gfx950
kernels behind ``libmlora.so``.  Call sites it serves:
valora/models/peft/lora_unordered_batch_infer.py:632-638,1141-1148,1521-1527.
"""
from __future__ import annotations

import torch

from . import _lib, _plan_cache


def _check_input(t: torch.Tensor, name: str) -> None:
    # CHECK_INPUT = CHECK_CUDA + CHECK_CONTIGUOUS (valora/csrc/lora_ops.cc:27-34)
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


_NAMES = ("y", "x", "w", "start_indicies", "lora_ranks", "loc_indicies", "indicies")


def _check_common(y, x, w, start_indicies, lora_ranks, loc_indicies, indicies):
    ts = (y, x, w, start_indicies, lora_ranks, loc_indicies, indicies)
    for t in ts:
        if not (t.is_cuda and t.is_contiguous()):     # the common case costs one pass; name the culprit below
            for t2, n in zip(ts, _NAMES):
                _check_input(t2, n)
    if y.dim() != 2:
        raise RuntimeError("y must be a 2D tensor")
    if x.dim() != 2:
        raise RuntimeError("x must be a 2D tensor")
    if w.dim() != 3:
        raise RuntimeError("w must be a 3D tensor")
    if indicies.dim() != 1:
        raise RuntimeError("indicies must be a 1D tensor")
    if indicies.size(0) != x.size(0):
        raise RuntimeError(f"CHECK_EQ(indicies.size(0), x.size(0)) failed. {indicies.size(0)} vs {x.size(0)}")
    if y.size(0) != x.size(0):
        raise RuntimeError(f"CHECK_EQ(y.size(0), x.size(0)) failed. {y.size(0)} vs {x.size(0)}")
    long = torch.long
    if not (start_indicies.dtype is long and lora_ranks.dtype is long and loc_indicies.dtype is long
            and indicies.dtype is long):
        for t, n in zip(ts[3:], _NAMES[3:]):
            if t.dtype != torch.long:  # data_ptr<int64_t>() throws on any other type
                raise RuntimeError(f"expected scalar type Long but found {t.dtype} ({n})")


def _no_kernel(h_in, h_out, dtype):
    return RuntimeError(f"No suitable kernel. h_in={h_in} h_out={h_out} dtype={dtype}")


def _workspace(T: int, n_adapters: int, narrow: int, device) -> torch.Tensor:
    n = _lib.lib().mlora_workspace_bytes(T, n_adapters, narrow)
    return torch.empty(max(int(n), 256), dtype=torch.uint8, device=device)


def dispatch_bgmv(y, x, w, start_indicies, lora_ranks, loc_indicies, indicies, qkvo, lora_scales) -> None:
    """In place on ``y``.  ``h_in > h_out``: shrink ``y[t, :r] = x[t] @ A_a.T`` (columns >= r keep
    their value); ``h_in < h_out``: expand ``y[t] += scale_a * x[t, :r] @ B_a``.  ``lora_ranks``
    holds ``4 * r``; ``w`` is the pool ``[rows, heads, head_dim]`` whose row width is the wide
    dimension of the call."""
    _check_common(y, x, w, start_indicies, lora_ranks, loc_indicies, indicies)
    T, h_in, h_out = x.size(0), x.size(1), y.size(1)
    code = _lib.dtype_code(x.dtype)
    if code < 0 or y.dtype != x.dtype or w.dtype != x.dtype:
        raise _no_kernel(h_in, h_out, x.dtype)
    if not (h_in < 65536 and h_out < 65536):
        raise _no_kernel(h_in, h_out, x.dtype)
    wide = max(h_in, h_out)
    if lora_scales is not None and lora_scales.dtype != x.dtype:
        lora_scales = lora_scales.to(x.dtype)  # the kernel reads scales as T (bgmv_impl.cuh:180)
    pool = _lib.make_pool(w, start_indicies, lora_ranks, loc_indicies, wide, 4)
    narrow = min(h_in, h_out)
    plan = _cached_plan(indicies, start_indicies, lora_ranks, T, narrow, wide)
    stream = _lib.current_stream(x.device)
    if plan is not None:
        _planned_call(plan, stream, y, x, pool, qkvo, lora_scales, T, h_in, h_out, code)
        return
    ws = _workspace(T, start_indicies.numel(), narrow, x.device)
    _lib.check(_lib.lib().mlora_dispatch_bgmv(
        stream, _lib.ptr(y), _lib.ptr(x), pool, _lib.ptr(indicies), int(qkvo),
        _lib.ptr(lora_scales), T, h_in, h_out, code, _lib.ptr(ws), ws.numel(), None))


def _planned_call(plan, stream, y, x, pool, qkvo, scales, T, h_in, h_out, code, shrink_mode=_lib.SHRINK_OVERWRITE,
                  shrink_width=0, y_stride=None, x_stride=None) -> None:
    """One shrink or one expand launch on a plan that already exists: the argument mapping of the one-call
    entry points (direction by ``h_in < h_out``, valora/csrc/bgmv/bgmv_impl.cuh:221) minus the plan build."""
    narrow = min(h_in, h_out)
    if h_in < h_out:
        if scales is None:
            raise RuntimeError("lora_scales is null")
        _lib.check(_lib.lib().mlora_expand(stream, plan.handle, _lib.ptr(y), T, h_out, None, _lib.ptr(x),
                                           h_in if x_stride is None else x_stride, narrow, pool, int(qkvo),
                                           _lib.ptr(scales), 1, 0, code))
    else:
        _lib.check(_lib.lib().mlora_shrink(stream, plan.handle, _lib.ptr(plan.scratch), plan.scratch.numel(),
                                           _lib.ptr(x), T, h_in, narrow, pool, int(qkvo), int(plan.ksplit), _lib.ptr(y),
                                           h_out if y_stride is None else y_stride, shrink_mode, shrink_width, 0, code))


def _cached_plan(ids, a_start, a_len, T, narrow, wide, n_slots=4, extra_tensors=(), extra_scalars=(), make_ids=None):
    """The plan of this batch from the cache (built on a miss), or None when the shapes are ones only
    the one-call entry point reports properly (it raises the reference's errors).  ``make_ids`` builds the
    per-token ids the plan is cut from when the entry point does not get them directly (segment or
    per-request operands); the result lives as long as the cache entry."""
    if not _plan_cache.enabled() or T == 0 or narrow <= 0 or narrow > 128 or narrow % 8 or narrow >= wide:
        return None
    def build():
        from .plan import LoraPlan
        eff = ids if make_ids is None else make_ids()
        plan = LoraPlan(eff, a_start, a_len, narrow, n_slots=n_slots, hidden=wide)
        plan.ids_keepalive = eff
        return plan

    return _plan_cache.lookup((ids, a_start, a_len) + tuple(extra_tensors),
                              (T, narrow, wide, n_slots, ids.device.index) + tuple(extra_scalars), build)
