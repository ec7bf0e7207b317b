"""Merging the dominant adapter into the base weights ("deLoRA" mode) and the op that compensates
the requests of the other adapters.

Host mirror of the reference's merged single-adapter path: ``merge_adapter`` / ``unmerge_adapter``
(valora/models/peft/lora_single_batch_infer.py:103-149) and of the compensation branch of
``_lora_get_qkv`` (valora/models/peft/lora_unordered_batch_infer.py:991-1063).

The reference densifies the adapter out of the pool (lora_single_batch_infer.py:81-98), forms
``bmm(A, B * scaling)`` for the four slots in a ``[4, H, H]`` temporary and adds it to the weights;
here one launch of ``libmlora.so`` reads the pool rows in place and updates the four weights, each
weight element read once and written once.  For the compensation the reference duplicates the
activations (``cat([x, x])``), runs shrink and expand over ``own adapter | merged adapter`` and adds
``first half - second half``; here the same tokens go through two planned LoRA ops, the second with
negated scales, without copies.
"""
from __future__ import annotations

import ctypes
from typing import Sequence

import torch

from . import _lib
from .plan import LoraPlan


def _merge(weights: Sequence[torch.Tensor], key_buffer: torch.Tensor, value_buffer: torch.Tensor,
           a_start: torch.Tensor, a_len: torch.Tensor, a_loc: torch.Tensor, adapter_idx: int, scaling: float,
           max_rank: int, slots: Sequence[int], n_slots: int, sign: int) -> None:
    n = len(weights)
    if not 1 <= n <= _lib.MAX_TARGETS or len(slots) != n:
        raise RuntimeError(f"merge takes 1..{_lib.MAX_TARGETS} weights with one slot each")
    w0 = weights[0]
    h_in, h_out = w0.shape
    for w in weights:
        if w.dim() != 2 or w.shape != w0.shape or w.dtype != w0.dtype or w.stride(1) != 1 or w.stride(0) != w0.stride(0):
            raise RuntimeError("merge: weights must be 2-D [H_in, H_out] of one shape, dtype and row stride")
        if w.device != key_buffer.device:
            raise RuntimeError("merge: weights and pool must be on the same device")
    if key_buffer.dtype != w0.dtype or value_buffer.dtype != w0.dtype:
        raise RuntimeError("merge: pool and weights must have the same dtype")
    pa = _lib.make_pool(key_buffer, a_start, a_len, a_loc, h_in, n_slots)
    pb = _lib.make_pool(value_buffer, a_start, a_len, a_loc, h_out, n_slots)
    wp = (ctypes.c_void_p * n)(*[w.data_ptr() for w in weights])
    sl = (ctypes.c_int32 * n)(*[int(s) for s in slots])
    _lib.check(_lib.lib().mlora_merge_adapter(
        _lib.current_stream(w0.device), wp, sl, n, w0.stride(0), h_in, h_out, pa, pb, int(adapter_idx), int(max_rank),
        float(scaling), sign, _lib.dtype_code(w0.dtype)))


def merge_adapter(weights, key_buffer, value_buffer, a_start, a_len, a_loc, adapter_idx, scaling, max_rank,
                  slots=(0, 1, 2, 3), n_slots=4) -> None:
    """``weights[k] += A_k @ (B_k * scaling)`` in place for the slots of one layer
    (lora_single_batch_infer.py:103-125).  ``weights[k]`` is the ``[H_in, H_out]`` matrix the base
    model multiplies with (``x @ W``); ``key_buffer`` / ``value_buffer`` are the layer's pool."""
    _merge(weights, key_buffer, value_buffer, a_start, a_len, a_loc, adapter_idx, scaling, max_rank, slots, n_slots, 1)


def unmerge_adapter(weights, key_buffer, value_buffer, a_start, a_len, a_loc, adapter_idx, scaling, max_rank,
                    slots=(0, 1, 2, 3), n_slots=4) -> None:
    """``weights[k] -= A_k @ (B_k * scaling)`` (lora_single_batch_infer.py:127-149)."""
    _merge(weights, key_buffer, value_buffer, a_start, a_len, a_loc, adapter_idx, scaling, max_rank, slots, n_slots, -1)


class DeLoraPlan:
    """Per-batch plan of the compensation op while adapter ``merged_idx`` sits in the base weights:
    tokens of every other adapter get ``+ LoRA(own adapter) - LoRA(merged adapter)``, tokens of the
    merged adapter and tokens without adapter get nothing
    (lora_unordered_batch_infer.py:991-1063: ``q[delora_tk_index:] += qA_delora[:n] - qA_delora[n:]``)."""

    def __init__(self, ids: torch.Tensor, merged_idx: int, a_start: torch.Tensor, a_len: torch.Tensor,
                 max_rank: int, hidden: int, n_slots: int = 4, **kw):
        other = (ids != merged_idx) & (ids >= 0) & (ids < a_start.numel())
        minus_one = torch.full_like(ids, -1)
        self.own = LoraPlan(torch.where(other, ids, minus_one), a_start, a_len, max_rank, hidden=hidden,
                            n_slots=n_slots, **kw)
        self.merged = LoraPlan(torch.where(other, torch.full_like(ids, merged_idx), minus_one), a_start, a_len,
                               max_rank, hidden=hidden, n_slots=n_slots, **kw)

    def apply(self, y, x, key_buffer, value_buffer, a_start, a_len, a_loc, slot, scales) -> None:
        self.own.apply(y, x, key_buffer, value_buffer, a_start, a_len, a_loc, slot, scales)
        self.merged.apply(y, x, key_buffer, value_buffer, a_start, a_len, a_loc, slot, -scales)
