"""Drop-in for the reference's ATMM extension ``atmm_ops`` (imported there as
``from atmm_ops import dispatch_bgmv as dispatch_sgmm``,
valora/models/peft/lora_unordered_batch_infer.py:14).

Signature and checks: atmm/valora/csrc/lora_ops.cc:115-186.  Semantics chosen here ("canonical"):
rows of the first ``num_problems`` segments ``[start_ids[i], start_ids[i] + output_counts[i])``
are processed; each row uses the adapter named by its per-token id in ``indicies`` with that
adapter's own rank, the pool layouts of the BGMV path (B as ``[H_out, r]``) and ``lora_scales``.
Where the reference's launch differs -- adapter taken from ``lora_ids`` (all zeros in the
server), rank from ``rank_counts`` (all 64), B read as ``[r, H_out]``, scaling ignored, rows
assumed physically contiguous (atmm/valora/csrc/bgmv/bgmv_impl.cuh:85-123,174,236) -- it computes
a different function from every other path of the reference on real adapter weights, so it is
not reproduced.  ``rank_counts``, ``lora_ids`` and the six tile arguments are accepted and
ignored (tile selection is ``valora_amd.tile_table``); ``tmp_d`` is used as scratch when large
enough.  ``shrink_accumulate(True)`` restores the reference's ``beta = 1`` on the shrink.
"""
from __future__ import annotations

import torch

from . import _lib
from .kernels import _cached_plan, _check_common, _no_kernel, _planned_call, _workspace

_SHRINK_MODE = _lib.SHRINK_OVERWRITE


def shrink_accumulate(enabled: bool) -> None:
    """``True``: shrink adds into ``y`` (``D = X*W + C``, atmm/.../bgmv_impl.cuh:174) instead of
    overwriting it."""
    global _SHRINK_MODE
    _SHRINK_MODE = _lib.SHRINK_ACCUMULATE if enabled else _lib.SHRINK_OVERWRITE


def dispatch_bgmv(y, x, w, start_indicies, lora_ranks, loc_indicies, indicies, qkvo, lora_scales,
                  output_counts, rank_counts, lora_ids, start_ids, tmp_d, num_problems,
                  tb_x=0, tb_y=0, tb_z=0, wp_x=0, wp_y=0, wp_z=0) -> None:
    _check_common(y, x, w, start_indicies, lora_ranks, loc_indicies, indicies)
    T, h_in, h_out = x.size(0), x.size(1), y.size(1)
    code = _lib.dtype_code(x.dtype)
    if code < 0 or y.dtype != x.dtype or w.dtype != x.dtype or not (h_in < 65536 and h_out < 65536):
        raise _no_kernel(h_in, h_out, x.dtype)
    for t, n in ((output_counts, "output_counts"), (start_ids, "start_ids")):
        if not t.is_cuda or t.dtype != torch.long:
            raise RuntimeError(f"expected a CUDA Long tensor ({n})")
    P = int(num_problems)
    if P > output_counts.numel() or P > start_ids.numel():
        raise RuntimeError(f"num_problems={P} exceeds the segment tensors")
    if lora_scales is not None and lora_scales.dtype != x.dtype:
        lora_scales = lora_scales.to(x.dtype)
    pool = _lib.make_pool(w, start_indicies, lora_ranks, loc_indicies, max(h_in, h_out), 4)
    narrow = min(h_in, h_out)
    oc, st = output_counts.contiguous(), start_ids.contiguous()

    def ids_of_segments():
        eff = torch.empty(T, dtype=torch.long, device=x.device)
        _lib.check(_lib.lib().mlora_ids_from_segments(_lib.current_stream(x.device), _lib.ptr(eff), _lib.ptr(indicies),
                                                      _lib.ptr(st), _lib.ptr(oc), P, T))
        return eff

    plan = _cached_plan(indicies, start_indicies, lora_ranks, T, narrow, max(h_in, h_out),
                        extra_tensors=(output_counts, start_ids), extra_scalars=(P,), make_ids=ids_of_segments)
    if plan is not None:
        _planned_call(plan, _lib.current_stream(x.device), y, x, pool, qkvo, lora_scales, T, h_in, h_out, code,
                      shrink_mode=_SHRINK_MODE)
        return
    need = int(_lib.lib().mlora_workspace_bytes(T, start_indicies.numel(), min(h_in, h_out)))
    if (tmp_d is not None and tmp_d.is_cuda and tmp_d.is_contiguous() and tmp_d.element_size() == 1
            and tmp_d.numel() >= need and tmp_d.data_ptr() % 16 == 0):
        ws = tmp_d
    else:
        ws = _workspace(T, start_indicies.numel(), min(h_in, h_out), x.device)
    _lib.check(_lib.lib().mlora_dispatch_sgmm(
        _lib.current_stream(x.device), _lib.ptr(y), _lib.ptr(x), pool, _lib.ptr(indicies), int(qkvo),
        _lib.ptr(lora_scales), _lib.ptr(output_counts.contiguous()), _lib.ptr(start_ids.contiguous()), P,
        T, h_in, h_out, code, _SHRINK_MODE, _lib.ptr(ws), ws.numel(), None))


dispatch_sgmm = dispatch_bgmv
