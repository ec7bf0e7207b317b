"""Adapter residency on the GPU: the paged pool's row allocator, loading adapters into it and
dropping them again.

Mirrors the interface of the reference's ``MemoryAllocator`` (valora/common/mem_allocator.py:10-258:
``alloc``, ``alloc_contiguous``, ``free``, ``free_all``, ``can_use_mem_size``, ``key_buffer`` /
``value_buffer`` of shape ``[layers, rows, heads, head_dim]``) and ``InferAdapter``
(valora/server/router/model_infer/infer_adapter.py:11-256: ``init``, ``load_lora_A``, ``load_lora_B``,
``load_adapters``, ``offload_adapters`` and the tensors ``a_loc / a_start / a_len / a_scaling``), so the
op entry points of this package read exactly the tensors the reference's server would hand them.

What differs is how the work is issued.  The reference allocates with a chain of PyTorch ops
(cumsum, compare, masked select), copies an adapter with two indexed assignments per layer (64 for
a 32-layer model) and rebuilds the index with per-adapter slice writes plus a Triton kernel.  Here
each of these is one kernel launch of ``libmlora.so``: first-fit / contiguous allocation, one row
scatter per buffer for all layers, one re-index call.  The host keeps the row counts it already knows
(ranks, free rows) so nothing waits for the device except ``alloc_contiguous``, whose result the
reference reads back as well (mem_allocator.py:73).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence

import torch

from . import _lib


def _stream(device) -> Any:
    return _lib.current_stream(device)


class MemoryAllocator:
    """Row allocator + the two weight buffers (valora/common/mem_allocator.py:10-27,243-258)."""

    def __init__(self, tot_size: int, cache_size: int, dtype: torch.dtype, head_num: int, head_dim: int,
                 layer_num: int, device="cuda"):
        assert tot_size >= cache_size
        self.dtype = dtype
        self.head_num = head_num
        self.head_dim = head_dim
        self.layer_num = layer_num
        self.cell_size = head_num * head_dim
        self.tot_size = tot_size
        self.cache_size = cache_size
        self.device = torch.device(device)
        _lib.lib()   # fail here, not at the first allocation, when the library is missing
        self.reset_all_pool()

    def get_memory_size(self) -> int:
        dsize = torch.empty((), dtype=self.dtype).element_size()
        return 2 * self.layer_num * self.tot_size * self.cell_size * dsize

    def alloc(self, need_size: int) -> torch.Tensor:
        """The first ``need_size`` free rows, ascending (mem_allocator.py:30-56)."""
        if need_size > self.can_use_mem_size:
            raise Exception(f'warn no enough pool space: need_size {need_size} left_size {self.can_use_mem_size}')
        index = torch.empty(need_size, dtype=torch.long, device=self.device)
        _lib.check(_lib.lib().mlora_pool_alloc(_stream(self.device), _lib.ptr(self.mem_state), self.tot_size,
                                               need_size, _lib.ptr(index), _lib.ptr(self._status)))
        self.can_use_mem_size -= need_size
        return index

    def alloc_contiguous(self, need_size: int):
        """``(index, start, end)`` of the first run of ``need_size`` free rows, or None
        (mem_allocator.py:59-75).  Waits for the device: the caller gets ``start`` as an int."""
        if need_size > self.can_use_mem_size:
            raise Exception(f'warn no enough pool space: need_size {need_size} left_size {self.can_use_mem_size}')
        index = torch.empty(need_size, dtype=torch.long, device=self.device)
        _lib.check(_lib.lib().mlora_pool_alloc_contiguous(_stream(self.device), _lib.ptr(self.mem_state),
                                                          self.tot_size, need_size, _lib.ptr(index),
                                                          _lib.ptr(self._status)))
        start = int(self._status[0].item())
        if start < 0:
            return None
        self.can_use_mem_size -= need_size
        return index, start, start + need_size

    def free(self, free_index: torch.Tensor) -> None:
        """mem_allocator.py:203-217."""
        free_index = free_index.to(device=self.device, dtype=torch.long).contiguous()
        self.can_use_mem_size += free_index.shape[0]
        _lib.check(_lib.lib().mlora_pool_free(_stream(self.device), _lib.ptr(self.mem_state), self.tot_size,
                                              _lib.ptr(free_index), free_index.shape[0]))

    def free_all(self) -> None:
        _lib.check(_lib.lib().mlora_pool_fill(_stream(self.device), _lib.ptr(self.mem_state), self.tot_size, 1))
        self.can_use_mem_size = self.tot_size

    def delete_all_pool(self) -> None:
        self.mem_state = None
        self._status = None
        self.can_use_mem_size = 0
        self.key_buffer = None
        self.value_buffer = None

    def delete_all_cache(self) -> None:
        self.delete_all_pool()

    def reset_all_pool(self) -> None:
        dev = self.device
        self.mem_state = torch.ones((self.tot_size,), dtype=torch.bool, device=dev)
        self._status = torch.zeros(2, dtype=torch.int32, device=dev)
        self.can_use_mem_size = self.tot_size
        shape = (self.layer_num, self.tot_size, self.head_num, self.head_dim)
        self.key_buffer = torch.empty(shape, dtype=self.dtype, device=dev)
        self.value_buffer = torch.empty(shape, dtype=self.dtype, device=dev)

    def reset_all_cache(self) -> None:
        self.reset_all_pool()


class LoraAdapterWeights:
    """One adapter's weights in the packed form the pool takes: ``packed_home[layer, 0]`` = the A
    blocks of the slots stacked (``[n_slots*r, H]``, slot s rows = ``lora_A.weight`` of that slot),
    ``packed_home[layer, 1]`` = the B blocks (``lora_B.weight`` ``[H, r]`` of each slot read flat as
    ``[r, H]``) -- the per-layer ``w_combined[2, 4r, heads, head_dim]`` of the reference
    (valora/models/peft/layer_weights/lora_layer_weight.py:448-516) for all layers in one pinned host
    tensor, so an adapter is one host-to-device copy.  Exposes the fields ``InferAdapter`` reads from
    the reference's ``LoraTpPartAdapter`` (valora/models/peft/lora_adapter.py:20-47)."""

    def __init__(self, lora_dir: str, r: int, lora_alpha: float, network_config: Dict[str, int],
                 packed_home: torch.Tensor):
        L, H = network_config["num_hidden_layers"], network_config["hidden_size"]
        assert packed_home.dim() == 4 and packed_home.shape[0] == L and packed_home.shape[1] == 2
        assert packed_home.shape[3] == H and packed_home.shape[2] % r == 0
        self.lora_dir = lora_dir
        self.r = r
        self.lora_alpha = lora_alpha
        self.scaling = lora_alpha / r
        self.network_config = network_config
        self.n_slots = packed_home.shape[2] // r
        self.packed_home = packed_home
        self.packed: Optional[torch.Tensor] = None

    @classmethod
    def from_dense(cls, lora_dir: str, r: int, lora_alpha: float, network_config: Dict[str, int],
                   lora_A: Sequence[Sequence[torch.Tensor]], lora_B: Sequence[Sequence[torch.Tensor]],
                   dtype=torch.float16, pin: bool = True) -> "LoraAdapterWeights":
        """``lora_A[layer][slot]`` is PEFT's ``lora_A.weight`` ``[r, H]``, ``lora_B[layer][slot]`` its
        ``lora_B.weight`` ``[H, r]``; a missing slot (None) is zeros, as in the reference
        (lora_layer_weight.py:452-456)."""
        L, H = network_config["num_hidden_layers"], network_config["hidden_size"]
        n_slots = len(lora_A[0])
        packed = torch.zeros(L, 2, n_slots * r, H, dtype=dtype)
        for l in range(L):
            for s in range(n_slots):
                if lora_A[l][s] is not None:
                    assert lora_A[l][s].shape == (r, H)
                    packed[l, 0, s * r:(s + 1) * r] = lora_A[l][s].to(dtype)
                if lora_B[l][s] is not None:
                    assert lora_B[l][s].shape == (H, r)
                    packed[l, 1, s * r:(s + 1) * r] = lora_B[l][s].to(dtype).contiguous().reshape(r, H)
        if pin and torch.cuda.is_available():
            packed = packed.pin_memory()
        return cls(lora_dir, r, lora_alpha, network_config, packed)

    @classmethod
    def from_hf_weights(cls, lora_dir: str, weights: Dict[str, torch.Tensor], lora_config: Dict,
                        network_config: Dict[str, int], module_names: Sequence[str] = ("c_attn", "w1", "w2", "c_proj"),
                        dtype=torch.float16, pin: bool = True) -> "LoraAdapterWeights":
        """From a PEFT checkpoint's tensor dict, with the key scheme and the slicing of the reference's loader
        (valora/models/peft/layer_weights/lora_layer_weight.py:434-516): the key prefix is the first key up to
        ``layers``; layer ``l`` slot ``s`` reads ``{prefix}layers.{l}.self_attn.{module_names[s]}.lora_A.weight``
        (``[r, >=H]``, its first H columns are kept) and ``...lora_B.weight`` (``[>=H, r]``, its first H rows are
        kept -- the reference cuts a fused qkv or an MLP projection down to H the same way); a missing module is
        zeros.  ``module_names`` defaults to the reference's Qwen names; pass e.g.
        ``("q_proj", "k_proj", "v_proj", "o_proj")`` for Llama-style checkpoints."""
        if not weights:
            raise RuntimeError("empty adapter checkpoint")
        r, alpha = int(lora_config["r"]), float(lora_config["lora_alpha"])
        L, H = network_config["num_hidden_layers"], network_config["hidden_size"]
        first = next(iter(weights.keys()))
        cut = first.find("layers")
        if cut < 0:
            raise RuntimeError(f"cannot find 'layers' in checkpoint key {first!r}")
        lora_A, lora_B = [], []
        for l in range(L):
            prefix = first[:cut] + f"layers.{l}.self_attn"
            a_row, b_row = [], []
            for m in module_names:
                a = weights.get(f"{prefix}.{m}.lora_A.weight")
                b = weights.get(f"{prefix}.{m}.lora_B.weight")
                if a is not None and (a.dim() != 2 or a.shape[0] != r or a.shape[1] < H):
                    raise RuntimeError(f"{prefix}.{m}.lora_A.weight has shape {tuple(a.shape)}, expected [{r}, >={H}]")
                if b is not None and (b.dim() != 2 or b.shape[1] != r or b.shape[0] < H):
                    raise RuntimeError(f"{prefix}.{m}.lora_B.weight has shape {tuple(b.shape)}, expected [>={H}, {r}]")
                a_row.append(None if a is None else a[:, :H])
                b_row.append(None if b is None else b[:H, :])
            lora_A.append(a_row)
            lora_B.append(b_row)
        return cls.from_dense(lora_dir, r, alpha, network_config, lora_A, lora_B, dtype=dtype, pin=pin)

    @classmethod
    def dummy(cls, lora_dir: str, r: int, lora_alpha: float, network_config: Dict[str, int], n_slots: int = 4,
              dtype=torch.float16, seed: int = 0, pin: bool = True) -> "LoraAdapterWeights":
        """Uniform(-1e-3, 1e-3) weights, the reference's dummy adapters (lora_layer_weight.py:311-331)."""
        L, H = network_config["num_hidden_layers"], network_config["hidden_size"]
        g = torch.Generator(device="cpu").manual_seed(seed)
        packed = ((torch.rand(L, 2, n_slots * r, H, generator=g) * 2 - 1) * 1e-3).to(dtype)
        if pin and torch.cuda.is_available():
            packed = packed.pin_memory()
        return cls(lora_dir, r, lora_alpha, network_config, packed)

    def dense(self, layer: int, slot: int):
        """``(A [H, r], B [r, H])`` of one slot as the math uses them: ``delta = x @ A @ B * scaling``."""
        r = self.r
        A = self.packed_home[layer, 0, slot * r:(slot + 1) * r].T.contiguous()
        B = self.packed_home[layer, 1, slot * r:(slot + 1) * r].reshape(-1, r).T.contiguous()
        return A, B

    def is_on_gpu(self) -> bool:
        return self.packed is not None

    def load_to_gpu(self, device="cuda", prefetch: bool = False) -> None:
        if self.packed is None:
            self.packed = self.packed_home.to(device, non_blocking=True)

    def offload_from_gpu(self) -> None:
        self.packed = None


@dataclass
class InferAdapter:
    adapter_dirs: List[str]     # all adapters resident in the pool
    a_loc: torch.Tensor         # pool rows of all adapters, concatenated
    a_start: torch.Tensor       # a_start[i]: where adapter i's rows begin in a_loc
    a_len: torch.Tensor         # a_len[i] = n_slots * r_i
    a_scaling: torch.Tensor     # alpha / r, in the pool's dtype
    mem_manager: MemoryAllocator
    merged_adapter_dir: Any
    idx_map: Dict[str, int]
    prefetch_tag: Dict[str, int]
    cur_tag: int
    prefetch_stream: Any
    lens: List[int] = field(default_factory=list)   # host copy of a_len

    @classmethod
    def init(cls, mem_manager: MemoryAllocator, prefetch_stream=None) -> "InferAdapter":
        dev = mem_manager.device
        return cls(
            adapter_dirs=[],
            a_loc=torch.empty(0, dtype=torch.long, device=dev),
            a_start=torch.empty(0, dtype=torch.long, device=dev),
            a_len=torch.empty(0, dtype=torch.long, device=dev),
            a_scaling=torch.empty(0, dtype=mem_manager.dtype, device=dev),
            mem_manager=mem_manager,
            idx_map={},
            prefetch_tag={},
            cur_tag=0,
            prefetch_stream=prefetch_stream,
            merged_adapter_dir=None,
        )

    # ---- weights -> pool rows ------------------------------------------------------------------
    def _scatter(self, buffer: torch.Tensor, packed: torch.Tensor, which: int, loc: torch.Tensor) -> None:
        mm = self.mem_manager
        esz = buffer.element_size()
        n = loc.shape[0]
        assert packed.shape[2] == n and packed.shape[3] == mm.cell_size and packed.dtype == buffer.dtype
        assert packed.is_contiguous() and loc.is_contiguous() and loc.dtype == torch.long
        src = packed.data_ptr() + which * n * mm.cell_size * esz
        _lib.check(_lib.lib().mlora_pool_scatter_rows(
            _stream(mm.device), _lib.ptr(buffer), mm.tot_size, mm.tot_size * mm.cell_size * esz,
            _lib.c_void_p(src), 2 * n * mm.cell_size * esz, _lib.ptr(loc), n, mm.cell_size * esz, mm.layer_num))

    def _packed_on_device(self, adapter) -> torch.Tensor:
        """``[layers, 2, n, H]`` on the pool's device, from this package's adapter class or from an
        object shaped like the reference's (``layers[i].w_combined`` / ``w_combined_home``)."""
        dev = self.mem_manager.device
        if hasattr(adapter, "packed_home"):
            adapter.load_to_gpu(dev)
            return adapter.packed
        per_layer = []
        for lw in adapter.layers:
            w = lw.w_combined if getattr(lw, "w_combined", None) is not None else lw.w_combined_home
            per_layer.append(w.to(dev, non_blocking=True).reshape(2, w.shape[1], -1))
        return torch.stack(per_layer).contiguous()

    def load_lora_A(self, adapter, loc: torch.Tensor, prefetch: bool = False) -> None:
        """``key_buffer[layer][loc] = w_combined[0]`` for every layer (infer_adapter.py:45-66)."""
        packed = self._packed_on_device(adapter)
        self._scatter(self.mem_manager.key_buffer, packed, 0, loc)
        if prefetch:
            packed.record_stream(torch.cuda.current_stream(self.mem_manager.device))

    def load_lora_B(self, adapter, loc: torch.Tensor, prefetch: bool = False) -> None:
        """``value_buffer[layer][loc] = w_combined[1]`` for every layer (infer_adapter.py:70-91)."""
        packed = self._packed_on_device(adapter)
        self._scatter(self.mem_manager.value_buffer, packed, 1, loc)
        if prefetch:
            packed.record_stream(torch.cuda.current_stream(self.mem_manager.device))

    # ---- residency ---------------------------------------------------------------------------
    def load_adapters(self, adapters, prefetch: bool = False, contiguous: bool = False) -> None:
        """infer_adapter.py:94-173.  ``contiguous=True`` gives every new adapter one run of consecutive
        pool rows (falling back to first fit when no run is free)."""
        if len(adapters) == 0:
            return
        n_rows = lambda ad: ad.r * getattr(ad, "n_slots", 4)
        new_adapters = []
        tot_size = 0
        if prefetch:
            self.cur_tag ^= 1
            capacity = self.mem_manager.can_use_mem_size
            for adapter in adapters:
                self.prefetch_tag[adapter.lora_dir] = self.cur_tag
                if adapter is not None and adapter.lora_dir not in self.idx_map:
                    if tot_size + n_rows(adapter) > capacity:
                        break
                    new_adapters.append(adapter)
                    tot_size += n_rows(adapter)
        else:
            for adapter in adapters:
                if adapter is not None and adapter.lora_dir not in self.idx_map:
                    new_adapters.append(adapter)
                    tot_size += n_rows(adapter)
        # the same adapter named twice in one call is loaded once (the reference would append it twice
        # and leave the first copy unreachable)
        seen, uniq = set(), []
        for ad in new_adapters:
            if ad.lora_dir not in seen:
                seen.add(ad.lora_dir)
                uniq.append(ad)
        new_adapters = uniq
        tot_size = sum(n_rows(ad) for ad in new_adapters)
        if not new_adapters:
            return

        dev = self.mem_manager.device
        if contiguous:
            parts = []
            for ad in new_adapters:
                got = self.mem_manager.alloc_contiguous(n_rows(ad))
                parts.append(got[0] if got is not None else self.mem_manager.alloc(n_rows(ad)))
            new_loc = torch.cat(parts)
        else:
            new_loc = self.mem_manager.alloc(tot_size)

        loc_offset = self.a_loc.shape[0]
        starts, cum = [], 0
        for ad in new_adapters:
            starts.append(loc_offset + cum)
            self.idx_map[ad.lora_dir] = len(self.adapter_dirs)
            self.adapter_dirs.append(ad.lora_dir)
            self.lens.append(n_rows(ad))
            cum += n_rows(ad)
        self.a_start = torch.cat((self.a_start, torch.tensor(starts, dtype=torch.long, device=dev)))
        self.a_len = torch.cat((self.a_len, torch.tensor([n_rows(ad) for ad in new_adapters], dtype=torch.long,
                                                         device=dev)))
        self.a_loc = torch.cat((self.a_loc, new_loc))
        self.a_scaling = torch.cat((self.a_scaling, torch.tensor([ad.scaling for ad in new_adapters],
                                                                 dtype=self.mem_manager.dtype, device=dev)))

        def copy_all():
            cum = 0
            for ad in new_adapters:
                loc = new_loc[cum:cum + n_rows(ad)]
                self.load_lora_A(ad, loc, prefetch)
                self.load_lora_B(ad, loc, prefetch)
                if hasattr(ad, "offload_from_gpu"):
                    ad.offload_from_gpu()
                cum += n_rows(ad)

        if prefetch and self.prefetch_stream is not None:
            # the rows were handed out on the current stream: the copy stream starts after that
            self.prefetch_stream.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(self.prefetch_stream):
                copy_all()
            new_loc.record_stream(self.prefetch_stream)
        else:
            copy_all()

    def offload_adapters(self, reserve_adapter_dirs) -> None:
        """infer_adapter.py:176-256: keep the named adapters and those tagged by the latest prefetch,
        free the rows of the rest, rebuild the index tensors."""
        if len(reserve_adapter_dirs) == len(self.adapter_dirs):
            return
        dev = self.mem_manager.device
        if self.prefetch_stream is not None:
            # rows freed below may be handed out again at once: copies still running on the prefetch stream
            # must have landed first
            torch.cuda.current_stream(dev).wait_stream(self.prefetch_stream)
        if len(reserve_adapter_dirs) == 0:
            self.mem_manager.free(self.a_loc)
            self.adapter_dirs = []
            self.lens = []
            self.a_loc = torch.empty(0, dtype=torch.long, device=dev)
            self.a_start = torch.empty(0, dtype=torch.long, device=dev)
            self.a_len = torch.empty(0, dtype=torch.long, device=dev)
            self.a_scaling = torch.empty(0, dtype=self.mem_manager.dtype, device=dev)
            self.idx_map = {}
            return

        left_ind, new_dirs, removed_rows = [], [], 0
        new_idx_map: Dict[str, int] = {}
        for i, adapter_dir in enumerate(self.adapter_dirs):
            if (adapter_dir not in reserve_adapter_dirs and
                    (adapter_dir not in self.prefetch_tag or self.prefetch_tag[adapter_dir] != self.cur_tag)):
                removed_rows += self.lens[i]
            else:
                left_ind.append(i)
                new_idx_map[adapter_dir] = len(new_dirs)
                new_dirs.append(adapter_dir)
        self.idx_map = new_idx_map
        if len(left_ind) == len(self.adapter_dirs):
            return
        n_old = len(self.adapter_dirs)
        new_lens = [self.lens[i] for i in left_ind]
        tot_size = sum(new_lens)
        keep = torch.tensor(left_ind, dtype=torch.int32, device=dev)
        new_a_len = torch.empty(len(left_ind), dtype=torch.long, device=dev)
        new_a_start = torch.empty(len(left_ind), dtype=torch.long, device=dev)
        new_a_scaling = torch.empty(len(left_ind), dtype=self.a_scaling.dtype, device=dev)
        new_a_loc = torch.empty(tot_size, dtype=torch.long, device=dev)
        mm = self.mem_manager
        _lib.check(_lib.lib().mlora_index_compact(
            _stream(dev), _lib.ptr(keep), len(left_ind), n_old, _lib.ptr(self.a_start), _lib.ptr(self.a_len),
            _lib.ptr(self.a_loc), self.a_loc.shape[0], _lib.ptr(self.a_scaling), _lib.ptr(new_a_start),
            _lib.ptr(new_a_len), _lib.ptr(new_a_loc), tot_size, _lib.ptr(new_a_scaling), _lib.ptr(mm.mem_state),
            mm.tot_size, _lib.ptr(mm._status)))
        mm.can_use_mem_size += removed_rows
        self.adapter_dirs = new_dirs
        self.lens = new_lens
        self.a_start, self.a_len, self.a_loc, self.a_scaling = new_a_start, new_a_len, new_a_loc, new_a_scaling
