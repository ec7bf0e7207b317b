"""One decoder layer with LoRA on all seven projections (q, k, v, o, gate, up, down).

The reference applies LoRA to the four attention projections only and leaves the FFN base-only
(valora/models/peft/lora_unordered_batch_infer.py:476,486 call the base FFN; its pool holds
``a_len = 4 * r`` rows per adapter, valora/server/router/model_infer/infer_adapter.py:144).  This module
is the wiring of the LoRA op into a forward pass with the FFN included, on a pool format that
extends the reference's: three (key, value) buffer pairs that share one row numbering and one
``a_start / a_len / a_loc`` index --

* ``attn``  rows of width H for A and for B; slots 0..3 = q, k, v, o   (the reference's buffers)
* ``up``    A rows of width H, B rows of width MLP; slots 0, 1 = gate, up
* ``down``  A rows of width MLP, B rows of width H; slot 0 = down

-- so an adapter still owns ``4 * r`` pool rows and every index tensor of the reference keeps its
meaning.  The base projections, normalisation, rotary embedding and attention are stock PyTorch
(`torch.mm`, `scaled_dot_product_attention`): they are the caller's side of the boundary; the LoRA
deltas go through ``LoraPlan``: q, k, v in one multi-target call, gate and up in another, o and
down in single calls -- four LoRA calls (8 to 12 launches) per layer for seven projections, where the
reference issues 8 calls (16 launches, each followed by a synchronize) for its four
(lora_unordered_batch_infer.py:946-1063,1611-1683).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Optional, Tuple

import torch
import torch.nn.functional as F

from .plan import LoraPlan


@dataclass
class LayerPools:
    """The three buffer pairs of ONE layer plus the shared index (all device tensors)."""
    attn: Tuple[torch.Tensor, torch.Tensor]     # (key_buffer, value_buffer), rows of width H / H
    up: Tuple[torch.Tensor, torch.Tensor]       # rows of width H / MLP
    down: Tuple[torch.Tensor, torch.Tensor]     # rows of width MLP / H
    a_start: torch.Tensor
    a_len: torch.Tensor
    a_loc: torch.Tensor
    a_scaling: torch.Tensor


@dataclass
class LayerWeights:
    """Base weights of one layer, stored ``[in, out]`` as the reference stores them (``x @ W``)."""
    wq: torch.Tensor
    wk: torch.Tensor
    wv: torch.Tensor
    wo: torch.Tensor
    w_gate: torch.Tensor
    w_up: torch.Tensor
    w_down: torch.Tensor
    ln1: torch.Tensor
    ln2: torch.Tensor


class LayerPlans:
    """Per-batch plans of a layer stack: one for the projections that read H-wide activations and one
    for ``down`` (MLP-wide input).  Built once per forward pass, reused by every layer."""

    def __init__(self, ids: torch.Tensor, a_start: torch.Tensor, a_len: torch.Tensor, max_rank: int, hidden: int,
                 mlp: int, n_slots: int = 4):
        self.h = LoraPlan(ids, a_start, a_len, max_rank, n_slots=n_slots, hidden=hidden)
        self.m = LoraPlan(ids, a_start, a_len, max_rank, n_slots=n_slots, hidden=mlp)


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * w


def rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, heads: int) -> torch.Tensor:
    """Rotate-half rotary embedding on ``x [T, heads * d]`` with ``cos / sin [T, d]``."""
    T = x.size(0)
    xh = x.view(T, heads, -1)
    d = xh.size(-1)
    x1, x2 = xh[..., : d // 2], xh[..., d // 2:]
    rot = torch.cat((-x2, x1), dim=-1)
    return (xh * cos[:, None, :] + rot * sin[:, None, :]).view(T, -1)


def layer_forward(x: torch.Tensor, w: LayerWeights, pools: Optional[LayerPools], plans: Optional[LayerPlans],
                  attention: Callable[[torch.Tensor, torch.Tensor, torch.Tensor], torch.Tensor], heads: int,
                  cos: Optional[torch.Tensor] = None, sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x [T, H]`` -> ``[T, H]``.  ``pools`` / ``plans`` None runs the base model only.  ``attention(q, k, v)``
    takes and returns ``[T, H]`` matrices (it owns the KV cache and the request boundaries)."""
    lora = pools is not None and plans is not None
    idx = (pools.a_start, pools.a_len, pools.a_loc) if lora else None
    h = rmsnorm(x, w.ln1)
    q, k, v = torch.mm(h, w.wq), torch.mm(h, w.wk), torch.mm(h, w.wv)
    if lora:
        plans.h.apply_multi([q, k, v], h, pools.attn[0], pools.attn[1], *idx, [0, 1, 2], pools.a_scaling)
    if cos is not None:
        q, k = rope(q, cos, sin, heads), rope(k, cos, sin, heads)
    a = attention(q, k, v)
    o = torch.mm(a, w.wo)
    if lora:
        plans.h.apply(o, a, pools.attn[0], pools.attn[1], *idx, 3, pools.a_scaling)
    x = x + o
    h2 = rmsnorm(x, w.ln2)
    g, u = torch.mm(h2, w.w_gate), torch.mm(h2, w.w_up)
    if lora:
        plans.h.apply_multi([g, u], h2, pools.up[0], pools.up[1], *idx, [0, 1], pools.a_scaling)
    m = F.silu(g) * u
    d = torch.mm(m, w.w_down)
    if lora:
        plans.m.apply(d, m, pools.down[0], pools.down[1], *idx, 0, pools.a_scaling)
    return x + d


def segment_attention(seq_lens, heads: int) -> Callable[[torch.Tensor, torch.Tensor, torch.Tensor], torch.Tensor]:
    """Causal self-attention inside each request of a packed batch (``seq_lens`` rows per request, no
    earlier context) with ``scaled_dot_product_attention``; enough for tests and for the prefill part
    of a benchmark step."""
    bounds, s = [], 0
    for n in seq_lens:
        bounds.append((s, s + int(n)))
        s += int(n)

    def attend(q, k, v):
        out = torch.empty_like(q)
        for (b, e) in bounds:
            n = e - b
            qq, kk, vv = (t[b:e].view(n, heads, -1).transpose(0, 1).unsqueeze(0) for t in (q, k, v))
            out[b:e] = F.scaled_dot_product_attention(qq, kk, vv, is_causal=True)[0].transpose(0, 1).reshape(n, -1)
        return out

    return attend
