"""Drop-in for the reference's Triton prefill ops
``valora.models.peft.triton_kernel.lora.lora_prefill`` (lora_prefill.py:105-163): same names,
argument order and meaning, per-request operands; the kernels are the gfx950 ones, reached through
the compiled torch extension module (``csrc/binding.cpp``).
Call sites: valora/models/peft/lora_unordered_batch_infer.py:1127-1139.

    lora_get_qkvo_fwd_shrink(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len,
                             b_indicies, hidden_size, qkvo, max_rank, max_input_len)

``o[t, :max_rank] = x[t] @ A_a.T`` for the rows of every request (columns >= r are zero-filled, rows
past ``max_input_len`` rounded up to 32 are not visited, lora_prefill.py:142-147).

    lora_get_qkvo_fwd_expand(x, w, o, scale, b_loc, b_lora_start, b_lora_ranks, b_start_loc,
                             b_seq_len, b_indicies, feat_out, qkvo, max_rank, max_input_len)

``o[t] += scale_a * x[t, :r] @ B_a`` for the rows of every request.
"""
from __future__ import annotations

from ._ext import binding as _b

lora_get_qkvo_fwd_shrink = _b.lora_get_qkvo_fwd_shrink
lora_get_qkvo_fwd_expand = _b.lora_get_qkvo_fwd_expand
