"""Adapter pool index: the integer tensors and weight layout the LoRA op reads.

Mirrors the tensor contract of the reference's ``InferAdapter``
(valora/server/router/model_infer/infer_adapter.py:11-35,128-148) without its loading,
eviction or prefetch machinery:

* ``a_len[a]   = n_slots * r_a``          (int64; the reference fixes n_slots = 4: q, k, v, o)
* ``a_start[a]`` = offset of adapter a in ``a_loc``                       (int64)
* ``a_loc[a_start[a] + slot*r_a + j]`` = pool row of rank-row j of ``slot``  (int64)
* ``a_scaling[a] = alpha / r``            (stored in the op's 16-bit dtype)

Weight layout (valora/models/peft/layer_weights/lora_layer_weight.py:448-516,
infer_adapter.py:58-59,83-84):

* ``key_buffer`` row ``a_loc[base + j]`` holds ``A[:, j]`` -- A kept as ``[r, H_in]`` row-major;
* ``value_buffer`` rows ``a_loc[base : base + r]``, concatenated, hold ``B.T`` -- ``[H_out, r]``
  row-major, i.e. ``flat[o*r + j] = B[j, o]``.

A pool row is as wide as the wide dimension of the call that reads it (the kernels index
``row * feat``, valora/csrc/bgmv/bgmv_impl.cuh:48,191), so targets whose input and output
widths differ (MLP up / down) use a key buffer and a value buffer of different widths that
share one row numbering.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch


class AdapterPool:
    def __init__(self, n_rows: int, h_in: int, h_out: int, dtype: torch.dtype, device="cpu",
                 n_slots: int = 4, heads: int = 32):
        assert h_in % heads == 0 and h_out % heads == 0
        self.n_rows, self.h_in, self.h_out = n_rows, h_in, h_out
        self.dtype, self.device, self.n_slots, self.heads = dtype, torch.device(device), n_slots, heads
        # 3-D like the reference's pool (rows, heads, head_dim): dispatch_bgmv checks w.dim() == 3
        self.key_buffer = torch.zeros(n_rows, heads, h_in // heads, dtype=dtype, device=device)
        self.value_buffer = torch.zeros(n_rows, heads, h_out // heads, dtype=dtype, device=device)
        self.a_start = torch.empty(0, dtype=torch.long, device=device)
        self.a_len = torch.empty(0, dtype=torch.long, device=device)
        self.a_loc = torch.empty(0, dtype=torch.long, device=device)
        self.a_scaling = torch.empty(0, dtype=dtype, device=device)
        self._free = list(range(n_rows))
        self.ranks: List[int] = []

    @property
    def n_adapters(self) -> int:
        return int(self.a_start.numel())

    def alloc_rows(self, n: int, rows: Optional[Sequence[int]] = None) -> torch.Tensor:
        if rows is None:
            assert len(self._free) >= n, "adapter pool exhausted"
            rows = self._free[:n]
        taken = set(int(r) for r in rows)
        assert len(taken) == n
        self._free = [r for r in self._free if r not in taken]
        return torch.tensor(list(rows), dtype=torch.long, device=self.device)

    def load_adapter(self, A_slots: Sequence[torch.Tensor], B_slots: Sequence[torch.Tensor],
                     scaling: float, rows: Optional[Sequence[int]] = None) -> int:
        """``A_slots[s]`` is ``[H_in, r]``, ``B_slots[s]`` is ``[r, H_out]`` (dense, as PEFT's
        ``lora_A.weight.T`` / ``lora_B.weight.T``).  Returns the adapter index."""
        assert len(A_slots) == self.n_slots and len(B_slots) == self.n_slots
        r = A_slots[0].shape[1]
        loc = self.alloc_rows(self.n_slots * r, rows)
        kb = self.key_buffer.view(self.n_rows, self.h_in)
        vb = self.value_buffer.view(self.n_rows, self.h_out)
        for s in range(self.n_slots):
            A, B = A_slots[s], B_slots[s]
            assert A.shape == (self.h_in, r) and B.shape == (r, self.h_out)
            srows = loc[s * r:(s + 1) * r]
            kb[srows] = A.T.to(self.dtype).to(self.device)
            vb[srows] = B.T.contiguous().reshape(r, self.h_out).to(self.dtype).to(self.device)
        idx = self.n_adapters
        start = int(self.a_loc.numel())
        dev = self.device
        self.a_start = torch.cat((self.a_start, torch.tensor([start], dtype=torch.long, device=dev)))
        self.a_len = torch.cat((self.a_len, torch.tensor([self.n_slots * r], dtype=torch.long, device=dev)))
        self.a_loc = torch.cat((self.a_loc, loc))
        self.a_scaling = torch.cat((self.a_scaling, torch.tensor([scaling], dtype=self.dtype, device=dev)))
        self.ranks.append(r)
        return idx

    def to(self, device) -> "AdapterPool":
        p = AdapterPool.__new__(AdapterPool)
        p.__dict__.update(self.__dict__)
        p.device = torch.device(device)
        for name in ("key_buffer", "value_buffer", "a_start", "a_len", "a_loc", "a_scaling"):
            setattr(p, name, getattr(self, name).to(device))
        p._free = list(self._free)
        p.ranks = list(self.ranks)
        return p

    def dense(self, a: int, slot: int):
        """Dense ``(A [H_in, r], B [r, H_out])`` of one slot, re-read from the pool
        (valora/models/peft/lora_single_batch_infer.py:81-98)."""
        r = self.ranks[a]
        base = int(self.a_start[a]) + r * slot
        rows = self.a_loc[base: base + r]
        A = self.key_buffer.view(self.n_rows, self.h_in)[rows].T.contiguous()
        B = self.value_buffer.view(self.n_rows, self.h_out)[rows].reshape(self.h_out, r).T.contiguous()
        return A, B
