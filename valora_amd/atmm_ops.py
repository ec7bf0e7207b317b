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
ignored (tile selection is the library's table, ``mlora_tile_lookup``); ``tmp_d`` is used as scratch
when large enough.  ``shrink_accumulate(True)`` restores the reference's ``beta = 1`` on the shrink
(``D = X*W + C``, atmm/valora/csrc/bgmv/bgmv_impl.cuh:174) instead of overwriting ``y``.

    dispatch_bgmv(y, x, w, start_indicies, lora_ranks, loc_indicies, indicies, qkvo, lora_scales,
                  output_counts, rank_counts, lora_ids, start_ids, tmp_d, num_problems,
                  tb_x=0, tb_y=0, tb_z=0, wp_x=0, wp_y=0, wp_z=0)

The function lives in the compiled torch extension module (``csrc/binding.cpp``).
"""
from __future__ import annotations

from ._ext import binding as _b

dispatch_bgmv = _b.dispatch_sgmm
dispatch_sgmm = dispatch_bgmv
shrink_accumulate = _b.shrink_accumulate
