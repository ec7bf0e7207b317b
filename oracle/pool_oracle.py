"""CPU restatement of the reference's adapter residency code.  TEST INFRASTRUCTURE ONLY.

Nothing under ``valora_amd/`` may import this module; it is the checker for the HIP allocator,
row scatter / gather and re-indexing kernels.

Restated with CPU torch tensors, following the reference's own tensor formulation line by line:

* ``Allocator.alloc``             valora/common/mem_allocator.py:30-56
* ``Allocator.alloc_contiguous``  valora/common/mem_allocator.py:59-75
* ``Allocator.free / free_all``   valora/common/mem_allocator.py:203-221
* ``w_combined``                  valora/models/peft/layer_weights/lora_layer_weight.py:448-516
* ``Residency.load_adapters``     valora/server/router/model_infer/infer_adapter.py:45-173
* ``Residency.offload_adapters``  valora/server/router/model_infer/infer_adapter.py:176-256,263-284
* ``densify``                     valora/models/peft/lora_single_batch_infer.py:81-98

Pinning (tests/test_pool_oracle_pins.py): the allocator against plain Python loops ("scan the rows
in order, take the free ones") over exhaustive small states and random sequences; hand-derived
vectors in tests/golden/pool_index.json (worked out on paper from the cited lines); invariants
(alloc then free restores the state; rows handed out are free, distinct and ascending; re-indexing
keeps every survivor's rows, order and scaling; load then densify returns the PEFT matrices).  The
reference holds no test or fixture of its own for this code.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch


class Allocator:
    """mem_allocator.py:10-27,243-258 without the weight buffers."""

    def __init__(self, tot_size: int):
        self.tot_size = tot_size
        self.mem_state = torch.ones((tot_size,), dtype=torch.bool)
        self._mem_cum_sum = torch.empty((tot_size,), dtype=torch.int32)
        self.indexes = torch.arange(0, tot_size, dtype=torch.long)
        self.can_use_mem_size = tot_size

    def alloc(self, need_size: int) -> torch.Tensor:
        if need_size > self.can_use_mem_size:
            raise Exception(f'warn no enough pool space: need_size {need_size} left_size {self.can_use_mem_size}')
        torch.cumsum(self.mem_state, dim=0, dtype=torch.int32, out=self._mem_cum_sum)
        select_index = torch.logical_and(self._mem_cum_sum <= need_size, self.mem_state == 1)
        index = self.indexes[select_index]
        self.mem_state[index] = 0
        self.can_use_mem_size -= len(index)
        return index

    def alloc_contiguous(self, need_size: int):
        if need_size > self.can_use_mem_size:
            raise Exception(f'warn no enough pool space: need_size {need_size} left_size {self.can_use_mem_size}')
        torch.cumsum(self.mem_state, dim=0, dtype=torch.int32, out=self._mem_cum_sum)
        loc_sums = (self._mem_cum_sum[need_size - 1:self.tot_size]
                    - self._mem_cum_sum[0:self.tot_size - need_size + 1]
                    + self.mem_state[0:self.tot_size - need_size + 1])
        can_used_loc = self.indexes[0:self.tot_size - need_size + 1][loc_sums == need_size]
        if can_used_loc.shape[0] == 0:
            return None
        start_loc = can_used_loc[0]
        select_index = self.indexes[start_loc: start_loc + need_size]
        self.mem_state[select_index] = 0
        self.can_use_mem_size -= need_size
        start = start_loc.item()
        return select_index, start, start + need_size

    def free(self, free_index: torch.Tensor) -> None:
        self.can_use_mem_size += free_index.shape[0]
        self.mem_state[free_index] = 1

    def free_all(self) -> None:
        self.mem_state[:] = 1
        self.can_use_mem_size = self.tot_size


def w_combined(lora_A: Sequence[Optional[torch.Tensor]], lora_B: Sequence[Optional[torch.Tensor]], r: int,
               heads: int, H: int, dtype=torch.float16) -> torch.Tensor:
    """One layer's ``[2, n_slots*r, heads, H/heads]`` from PEFT ``lora_A.weight [r, H]`` and
    ``lora_B.weight [H, r]`` per slot, through the reference's own chain of transposes
    (lora_layer_weight.py:448-516): ``X_home = weight.transpose(0, 1).contiguous()``, then
    ``X_home.T.reshape(r, heads, H/heads)``; None -> zeros."""
    def safe_reshape(home):
        if home is not None:
            return home.T.reshape(r, heads, H // heads)
        return torch.zeros(r, heads, H // heads, dtype=dtype)
    a_home = [None if w is None else w.transpose(0, 1).contiguous().to(dtype) for w in lora_A]   # [H, r]
    b_home = [None if w is None else w.transpose(0, 1).contiguous().to(dtype) for w in lora_B]   # [r, H]
    blocks = [safe_reshape(h) for h in a_home] + [safe_reshape(h) for h in b_home]
    n = len(lora_A)
    return torch.concat(blocks).reshape(2, n * r, heads, H // heads).to(dtype)


class Residency:
    """InferAdapter on CPU tensors (infer_adapter.py:11-256).  ``adapters`` are dicts with keys
    ``lora_dir, r, scaling, w`` where ``w[layer]`` is that layer's ``w_combined``."""

    def __init__(self, alloc: Allocator, layers: int, heads: int, head_dim: int, dtype=torch.float16,
                 n_slots: int = 4):
        self.mem = alloc
        self.n_slots = n_slots
        self.dtype = dtype
        self.key_buffer = torch.zeros(layers, alloc.tot_size, heads, head_dim, dtype=dtype)
        self.value_buffer = torch.zeros(layers, alloc.tot_size, heads, head_dim, dtype=dtype)
        self.adapter_dirs: List[str] = []
        self.a_loc = torch.empty(0, dtype=torch.long)
        self.a_start = torch.empty(0, dtype=torch.long)
        self.a_len = torch.empty(0, dtype=torch.long)
        self.a_scaling = torch.empty(0, dtype=dtype)
        self.idx_map: Dict[str, int] = {}
        self.prefetch_tag: Dict[str, int] = {}
        self.cur_tag = 0

    def load_adapters(self, adapters, prefetch: bool = False) -> None:
        if len(adapters) == 0:
            return
        S = self.n_slots
        new_adapters, tot_size = [], 0
        if prefetch:
            self.cur_tag ^= 1
            capacity = self.mem.can_use_mem_size
            for adapter in adapters:
                self.prefetch_tag[adapter["lora_dir"]] = self.cur_tag
                if adapter is not None and adapter["lora_dir"] not in self.idx_map:
                    if tot_size + adapter["r"] * S > capacity:
                        break
                    new_adapters.append(adapter)
                    tot_size += adapter["r"] * S
        else:
            for adapter in adapters:
                if adapter is not None and adapter["lora_dir"] not in self.idx_map:
                    new_adapters.append(adapter)
                    tot_size += adapter["r"] * S
        new_loc = self.mem.alloc(tot_size)
        start_offset = self.a_start.shape[0]
        self.a_start = torch.cat((self.a_start, torch.empty(len(new_adapters), dtype=torch.long)))
        len_offset = self.a_len.shape[0]
        self.a_len = torch.cat((self.a_len, torch.empty(len(new_adapters), dtype=torch.long)))
        loc_offset = self.a_loc.shape[0]
        self.a_loc = torch.cat((self.a_loc, torch.empty(tot_size, dtype=torch.long)))
        cum_loc, cum_loc_list = 0, []
        for i, new_adapter in enumerate(new_adapters):
            cum_loc_list.append(cum_loc)
            self.idx_map[new_adapter["lora_dir"]] = len(self.adapter_dirs)
            self.adapter_dirs.append(new_adapter["lora_dir"])
            self.a_start[start_offset + i] = loc_offset + cum_loc
            self.a_len[len_offset + i] = new_adapter["r"] * S
            self.a_loc[loc_offset + cum_loc: loc_offset + cum_loc + new_adapter["r"] * S] = (
                new_loc[cum_loc: cum_loc + new_adapter["r"] * S])
            cum_loc += new_adapter["r"] * S
        self.a_scaling = torch.cat((self.a_scaling, torch.tensor([a["scaling"] for a in new_adapters],
                                                                 dtype=self.dtype)))
        for i, new_adapter in enumerate(new_adapters):
            loc = new_loc[cum_loc_list[i]: cum_loc_list[i] + new_adapter["r"] * S]
            for layer in range(self.key_buffer.shape[0]):
                wc = new_adapter["w"][layer]
                self.key_buffer[layer][loc] = wc[0]        # load_lora_A, infer_adapter.py:58-59
                self.value_buffer[layer][loc] = wc[1]      # load_lora_B, infer_adapter.py:83-84

    def offload_adapters(self, reserve_adapter_dirs) -> None:
        if len(reserve_adapter_dirs) == len(self.adapter_dirs):
            return
        if len(reserve_adapter_dirs) == 0:
            self.mem.free(self.a_loc)
            self.adapter_dirs = []
            self.a_loc = torch.empty(0, dtype=torch.long)
            self.a_start = torch.empty(0, dtype=torch.long)
            self.a_len = torch.empty(0, dtype=torch.long)
            self.a_scaling = torch.empty(0, dtype=self.dtype)
            self.idx_map = {}
            return
        remove_ind, left_ind, new_adapter_dirs = [], [], []
        self.idx_map = {}
        for i, adapter_dir in enumerate(self.adapter_dirs):
            if (adapter_dir not in reserve_adapter_dirs and
                    (adapter_dir not in self.prefetch_tag or self.prefetch_tag[adapter_dir] != self.cur_tag)):
                remove_ind.append(self.a_loc[self.a_start[i]:self.a_start[i] + self.a_len[i]])
            else:
                left_ind.append(i)
                self.idx_map[adapter_dir] = len(new_adapter_dirs)
                new_adapter_dirs.append(adapter_dir)
        if len(remove_ind) == 0:
            return
        self.adapter_dirs = new_adapter_dirs
        tot_size = torch.sum(self.a_len[left_ind]).item()
        self.mem.free(torch.cat(remove_ind))
        new_a_len = torch.empty(len(left_ind), dtype=torch.long)
        new_a_start = torch.empty(len(left_ind), dtype=torch.long)
        new_a_scaling = torch.empty(len(left_ind), dtype=self.dtype)
        new_a_loc = torch.empty(int(tot_size), dtype=torch.long)
        new_a_len[:] = self.a_len[left_ind]
        new_a_start[0] = 0
        new_a_start[1:] = torch.cumsum(new_a_len, dim=0)[:-1]
        new_a_scaling[:] = self.a_scaling[left_ind]
        # var_len_copy (infer_adapter.py:263-284): one program per surviving adapter
        old_start = self.a_start[left_ind]
        for a_id in range(len(left_ind)):
            length, o, n = int(new_a_len[a_id]), int(old_start[a_id]), int(new_a_start[a_id])
            new_a_loc[n:n + length] = self.a_loc[o:o + length]
        self.a_start, self.a_len, self.a_loc, self.a_scaling = new_a_start, new_a_len, new_a_loc, new_a_scaling

    def densify(self, adapter_idx: int, layer: int, slot: int):
        """``(A [H, r], B [r, H])`` re-read from the pool (lora_single_batch_infer.py:81-98)."""
        S = self.n_slots
        r = int(self.a_len[adapter_idx]) // S
        start = int(self.a_start[adapter_idx])
        loc = self.a_loc[start:start + r * S]
        H = self.key_buffer.shape[2] * self.key_buffer.shape[3]
        rows = loc[slot * r:(slot + 1) * r]
        A = self.key_buffer[layer][rows].reshape(r, H).transpose(0, 1)
        B = self.value_buffer[layer][rows].reshape(H, r).transpose(0, 1)
        return A, B
