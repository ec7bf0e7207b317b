"""Drop-in for the reference's Triton prefill ops
``valora.models.peft.triton_kernel.lora.lora_prefill`` (lora_prefill.py:105-163): same names,
argument order and meaning, per-request operands; the kernels are the gfx950 ones.
Call sites: valora/models/peft/lora_unordered_batch_infer.py:1127-1139.
"""
from __future__ import annotations

import torch

from . import _lib
from .kernels import _cached_plan, _no_kernel, _planned_call, _workspace


def _request_plan(x, b_start_loc, b_seq_len, b_indicies, b_lora_start, b_lora_ranks, T, max_rank, wide, max_input_len):
    """The cached plan of this batch; the per-token ids come from the per-request operands (rows past
    ``max_input_len`` rounded up to 32 are left out, lora_prefill.py:147)."""
    narrow = max(8, -(-int(max_rank) // 8) * 8)
    if int(max_rank) <= 0 or narrow >= wide:
        return None      # shapes the one-call entry point rejects with the proper message
    max_rows = (int(max_input_len) + 31) // 32 * 32

    def ids_of_requests():
        s, n, idx = _req_operands(b_start_loc, b_seq_len, b_indicies)
        eff = torch.empty(T, dtype=torch.long, device=x.device)
        _lib.check(_lib.lib().mlora_ids_from_requests(_lib.current_stream(x.device), _lib.ptr(eff), _lib.ptr(s), _lib.ptr(n),
                                                      _lib.ptr(idx), n.numel(), T, max_rows))
        return eff

    return _cached_plan(b_indicies, b_lora_start, b_lora_ranks, T, narrow, wide,
                        extra_tensors=(b_start_loc, b_seq_len), extra_scalars=(max_rows,), make_ids=ids_of_requests)


def _req_operands(b_start_loc, b_seq_len, b_indicies):
    # infer_batch.py:77,106 builds these as int32; b_indicies is the int64 per-request req_bins
    return (b_start_loc.to(torch.int32).contiguous(), b_seq_len.to(torch.int32).contiguous(),
            b_indicies.to(torch.long).contiguous())


@torch.inference_mode()
def lora_get_qkvo_fwd_shrink(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len,
                             b_indicies, hidden_size, qkvo, max_rank, max_input_len) -> None:
    """``o[t, :max_rank] = x[t] @ A_a.T`` for the rows of every request (columns >= r are
    zero-filled, rows past ``max_input_len`` rounded up to 32 are not visited)."""
    code = _lib.dtype_code(x.dtype)
    if code < 0 or w.dtype != x.dtype or o.dtype != x.dtype:
        raise _no_kernel(hidden_size, max_rank, x.dtype)
    if x.stride(-1) != 1 or o.stride(-1) != 1 or x.stride(0) != hidden_size or not w.is_contiguous():
        raise RuntimeError("x rows must be dense, o and w must have unit inner stride")
    T = x.size(0)
    pool = _lib.make_pool(w, b_lora_start, b_lora_ranks, b_loc, hidden_size, 4)
    plan = _request_plan(x, b_start_loc, b_seq_len, b_indicies, b_lora_start, b_lora_ranks, T, max_rank, int(hidden_size),
                         max_input_len) if T > 0 and b_seq_len.numel() > 0 else None
    if plan is not None:
        # columns stored: cdiv(max_rank, BLOCK_N) blocks of BLOCK_N = 16 (or max_rank when <= 8), lora_prefill.py:142,147
        block_n = 16 if int(max_rank) > 8 else int(max_rank)
        width = min(-(-int(max_rank) // block_n) * block_n, o.stride(0))
        narrow = max(8, -(-int(max_rank) // 8) * 8)
        _planned_call(plan, _lib.current_stream(x.device), o, x, pool, qkvo, None, T, int(hidden_size), narrow, code,
                      shrink_mode=_lib.SHRINK_ZERO_PAD, shrink_width=width, y_stride=o.stride(0))
        return
    s, n, idx = _req_operands(b_start_loc, b_seq_len, b_indicies)
    ws = _workspace(T, b_lora_start.numel(), max(8, -(-int(max_rank) // 8) * 8), x.device)
    _lib.check(_lib.lib().mlora_prefill_shrink(
        _lib.current_stream(x.device), _lib.ptr(o), _lib.ptr(x), pool, _lib.ptr(s), _lib.ptr(n),
        _lib.ptr(idx), n.numel(), T, int(hidden_size), o.stride(0), int(qkvo), int(max_rank),
        int(max_input_len), code, _lib.ptr(ws), ws.numel(), None))


@torch.inference_mode()
def lora_get_qkvo_fwd_expand(x, w, o, scale, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len,
                             b_indicies, feat_out, qkvo, max_rank, max_input_len) -> None:
    """``o[t] += scale_a * x[t, :r] @ B_a`` for the rows of every request."""
    code = _lib.dtype_code(x.dtype)
    if code < 0 or w.dtype != x.dtype or o.dtype != x.dtype:
        raise _no_kernel(max_rank, feat_out, x.dtype)
    if x.stride(-1) != 1 or o.stride(-1) != 1 or o.stride(0) != feat_out or not w.is_contiguous():
        raise RuntimeError("o rows must be dense, x and w must have unit inner stride")
    T = o.size(0)
    if scale.dtype != x.dtype:
        scale = scale.to(x.dtype)
    pool = _lib.make_pool(w, b_lora_start, b_lora_ranks, b_loc, feat_out, 4)
    plan = _request_plan(x, b_start_loc, b_seq_len, b_indicies, b_lora_start, b_lora_ranks, T, max_rank, int(feat_out),
                         max_input_len) if T > 0 and b_seq_len.numel() > 0 else None
    if plan is not None:
        narrow = max(8, -(-int(max_rank) // 8) * 8)
        _planned_call(plan, _lib.current_stream(x.device), o, x, pool, qkvo, scale, T, narrow, int(feat_out), code,
                      x_stride=x.stride(0))
        return
    s, n, idx = _req_operands(b_start_loc, b_seq_len, b_indicies)
    ws = _workspace(T, b_lora_start.numel(), max(8, -(-int(max_rank) // 8) * 8), x.device)
    _lib.check(_lib.lib().mlora_prefill_expand(
        _lib.current_stream(x.device), _lib.ptr(o), _lib.ptr(x), pool, _lib.ptr(scale), _lib.ptr(s),
        _lib.ptr(n), _lib.ptr(idx), n.numel(), T, x.stride(0), int(feat_out), int(qkvo), int(max_rank),
        int(max_input_len), code, _lib.ptr(ws), ws.numel(), None))
