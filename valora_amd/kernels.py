"""Drop-in for the reference's BGMV extension ``valora._kernels``.

``dispatch_bgmv`` keeps the reference's positional signature, argument meaning, in-place
behaviour and error behaviour (valora/csrc/lora_ops.cc:76-126); like the reference's, it is a
function of a compiled torch extension module (``csrc/binding.cpp``), which checks the operands,
finds the plan of the batch and makes one call into ``libmlora.so``.  Call sites it serves:
valora/models/peft/lora_unordered_batch_infer.py:632-638,1141-1148,1521-1527.

    dispatch_bgmv(y, x, w, start_indicies, lora_ranks, loc_indicies, indicies, qkvo, lora_scales)

In place on ``y``.  ``h_in > h_out``: shrink ``y[t, :r] = x[t] @ A_a.T`` (columns >= r keep their
value); ``h_in < h_out``: expand ``y[t] += scale_a * x[t, :r] @ B_a``.  ``lora_ranks`` holds
``4 * r``; ``w`` is the pool ``[rows, heads, head_dim]`` whose row width is the wide dimension of
the call.
"""
from __future__ import annotations

from ._ext import binding as _b

dispatch_bgmv = _b.dispatch_bgmv
