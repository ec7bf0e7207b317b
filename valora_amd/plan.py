"""Planned multi-LoRA op: build the adapter-grouped work tiles once per batch, then apply
shrink + expand for every (layer, target) of the step.

The reference rebuilds its segment tensors once per forward
(valora/server/router/model_infer/model_rpc.py:381) and then issues 8 op launches per layer with
the same per-token ids (valora/models/peft/lora_unordered_batch_infer.py:946-988,1611-1622);
``LoraPlan`` is that once-per-forward object for the gfx950 kernels.  The intermediate
``v = x @ A.T`` never becomes a caller-visible tensor: it lives in the plan's scratch buffer
between the two launches, rounded to the operand dtype exactly once -- where the reference stores
its ``delta`` tensor.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib, tile_table


class LoraPlan:
    def __init__(self, ids: torch.Tensor, a_start: torch.Tensor, a_len: torch.Tensor, max_rank: int,
                 n_slots: int = 4, hidden: int = 4096, bm_shrink: Optional[int] = None,
                 bm_expand: Optional[int] = None, ksplit: Optional[int] = None,
                 reduce_in_expand: Optional[bool] = None, one_launch: Optional[bool] = None,
                 one_launch_no_wait: bool = False, shrink_recompute: bool = False, expand_column_loop: bool = False,
                 one_launch_never_ready: bool = False):
        """``ids``: int64 per-token adapter index (negative = no adapter); ``a_start`` / ``a_len``:
        the pool index (``a_len = n_slots * rank``); ``max_rank``: widest rank among the resident
        adapters (the reference's ``max_lora_dim``, lora_unordered_batch_infer.py:181-182).
        ``one_launch``: shrink and expand as work items of one grid (decode-like batches; forces
        16-token tiles, needs ``max_rank <= 64``); ``None`` takes the tile table's choice.
        ``one_launch_no_wait`` makes every expand item take its give-up path at once, ``one_launch_never_ready`` after
        waiting out its bound, ``shrink_recompute`` makes the
        128-token shrink sum its K chunks by computing them all in one workgroup, ``expand_column_loop`` makes the
        expand of 16-token tiles walk over two column chunks per workgroup whatever the grid size (all for tests)."""
        if not ids.is_cuda:
            raise RuntimeError("ids must be a CUDA tensor")
        if ids.dtype != torch.long or a_start.dtype != torch.long or a_len.dtype != torch.long:
            raise RuntimeError("expected scalar type Long")
        self.device = ids.device
        self.T = int(ids.numel())
        self.n_adapters = int(a_start.numel())
        self.n_slots = n_slots
        self.max_rank = int(max_rank)
        cfg = tile_table.lookup(self.T, self.max_rank, hidden, self.n_adapters)
        self.bm_shrink = cfg.bm_shrink if bm_shrink is None else bm_shrink
        self.bm_expand = cfg.bm_expand if bm_expand is None else bm_expand
        self.ksplit = max(1, cfg.ksplit if ksplit is None else ksplit)
        rie = cfg.reduce_in_expand if reduce_in_expand is None else reduce_in_expand
        self.flags = _lib.REDUCE_IN_EXPAND if rie else 0
        self.one_launch = bool(cfg.one_launch if one_launch is None else one_launch)
        if self.one_launch and (self.max_rank > 64 or bm_shrink not in (None, 16) or bm_expand not in (None, 16)):
            if one_launch:
                raise RuntimeError("No suitable kernel. the one-launch op needs 16-token tiles and max_rank <= 64")
            self.one_launch = False
        if self.one_launch:
            self.bm_shrink = self.bm_expand = 16
            self.ksplit = max(2, self.ksplit)
            self.flags = (_lib.REDUCE_IN_EXPAND | _lib.ONE_LAUNCH | (_lib.ONE_LAUNCH_NO_WAIT if one_launch_no_wait else 0) |
                          (_lib.ONE_LAUNCH_NEVER_READY if one_launch_never_ready else 0))
        if shrink_recompute:
            self.flags |= _lib.SHRINK_RECOMPUTE
        if expand_column_loop:
            self.flags |= _lib.EXPAND_COLUMN_LOOP
        L = _lib.lib()
        nbytes = int(L.mlora_plan_bytes(self.T, self.n_adapters))
        self.buf = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=self.device)
        self.handle = _lib.Plan(_lib.ptr(self.buf), self.buf.numel(), 0, 0, 0, 0)
        self._keep = (ids.contiguous(), a_start, a_len)
        self.rebuild()
        # room for a multi-target call from the start: the buffer is never replaced, so a HIP graph captured
        # from this plan or work still queued on another stream keeps pointing at live memory
        self.scratch_per_target = int(L.mlora_scratch_bytes(self.T, self.max_rank, self.ksplit))
        nbytes = _lib.MAX_TARGETS * self.scratch_per_target
        if self.one_launch:
            nbytes = max(nbytes, max(int(L.mlora_one_launch_scratch_bytes(self.T, self.n_adapters, self.max_rank,
                                                                          self.ksplit, n)) for n in (1, 2, 3, 4)))
        self.scratch = torch.empty(nbytes, dtype=torch.uint8, device=self.device)

    def rebuild(self, ids: Optional[torch.Tensor] = None) -> None:
        """Cut the tiles again, in place, for the next batch of the same size (``ids`` of the same length; None
        re-reads the tensor the plan was made from, whose contents may have changed).  One launch on the current
        stream, no allocation: a serving loop that replays one HIP graph per step captures this call at the
        head of the step and refills its ids tensor before each replay (the reference rebuilds its segment
        tensors once per forward, valora/server/router/model_infer/model_rpc.py:381)."""
        if ids is not None:
            if ids.dtype != torch.long or ids.numel() != self.T or ids.device != self.device:
                raise RuntimeError(f"rebuild takes {self.T} int64 ids on {self.device}")
            self._keep = (ids.contiguous(),) + self._keep[1:]
        ids, a_start, a_len = self._keep
        _lib.check(_lib.lib().mlora_build_plan(_lib.current_stream(self.device), self.handle, _lib.ptr(ids), self.T,
                                               _lib.ptr(a_start), _lib.ptr(a_len), self.n_adapters, self.n_slots,
                                               self.bm_shrink, self.bm_expand))

    # -- introspection (synchronises; for tests and diagnostics) --------------------------------
    def header(self) -> dict:
        h = self.buf[:128].view(torch.int32).cpu().tolist()
        names = ["magic", "T", "n_adapters", "n_tiles_shrink", "n_tiles_expand", "n_groups", "max_rank",
                 "reserved", "bm_shrink", "bm_expand", "n_active"]
        return dict(zip(names, h))

    def perm(self) -> torch.Tensor:
        n = self.header()["n_active"]
        return self.buf.view(torch.int32)[32:32 + n].clone()

    def _section(self, index: int) -> torch.Tensor:
        # layout mirrors plan_layout() in csrc/mlora_internal.h
        T, A = self.T, self.n_adapters
        up8 = lambda v: (v + 7) // 8 * 8
        max_tiles = (T + 15) // 16 + min(A, T)
        off_perm = 32
        off_pad = up8(off_perm + T)
        off_prank = up8(off_pad + T)
        off_ts = up8(off_prank + T)
        off_te = off_ts + max_tiles * 8
        words = self.buf.view(torch.int32)
        h = self.header()
        if index == 0:
            return words[off_pad:off_pad + h["n_active"]].clone()
        if index == 1:
            return words[off_prank:off_prank + h["n_active"]].clone()
        if index == 2:
            return words[off_ts:off_ts + h["n_tiles_shrink"] * 8].view(-1, 8).clone()
        return words[off_te:off_te + h["n_tiles_expand"] * 8].view(-1, 8).clone()

    def position_adapters(self): return self._section(0)
    def position_ranks(self): return self._section(1)
    def tiles_shrink(self): return self._section(2)
    def tiles_expand(self): return self._section(3)

    # -- the op -------------------------------------------------------------------------------------
    def _check(self, x, y, key_buffer, value_buffer):
        for t, w in ((x, key_buffer), (y, value_buffer)):
            if t is None:
                continue
            if t.dim() != 2 or t.size(0) != self.T or not t.is_contiguous():
                raise RuntimeError(f"x and y must be contiguous [T={self.T}, H] matrices")
            if _lib.dtype_code(t.dtype) < 0 or w.dtype != t.dtype:
                raise RuntimeError(f"No suitable kernel. h_in={t.size(1)} h_out={t.size(1)} dtype={t.dtype}")

    def shrink(self, x: torch.Tensor, key_buffer: torch.Tensor, a_start, a_len, a_loc, slot: int) -> None:
        """First launch of the op alone: ``v = x @ A_a.T`` into ``self.scratch``."""
        self._check(x, None, key_buffer, None)
        pa = _lib.make_pool(key_buffer, a_start, a_len, a_loc, x.size(1), self.n_slots)
        _lib.check(_lib.lib().mlora_shrink(
            _lib.current_stream(self.device), self.handle, _lib.ptr(self.scratch), self.scratch.numel(),
            _lib.ptr(x), self.T, x.size(1), self.max_rank, pa, int(slot), int(self.ksplit), None, 0, 0, 0,
            self.flags, _lib.dtype_code(x.dtype)))

    def expand(self, y: torch.Tensor, value_buffer: torch.Tensor, a_start, a_len, a_loc, slot: int,
               scales: torch.Tensor) -> None:
        """Second launch alone: ``y += scale_a * v @ B_a`` with v taken from ``self.scratch``."""
        self._check(None, y, None, value_buffer)
        if scales.dtype != y.dtype:
            scales = scales.to(y.dtype)
        pb = _lib.make_pool(value_buffer, a_start, a_len, a_loc, y.size(1), self.n_slots)
        _lib.check(_lib.lib().mlora_expand(
            _lib.current_stream(self.device), self.handle, _lib.ptr(y), self.T, y.size(1), _lib.ptr(self.scratch),
            None, 0, self.max_rank, pb, int(slot), _lib.ptr(scales), int(self.ksplit), self.flags,
            _lib.dtype_code(y.dtype)))

    def apply_multi(self, ys, x: torch.Tensor, key_buffer: torch.Tensor, value_buffers, a_start: torch.Tensor,
                    a_len: torch.Tensor, a_loc: torch.Tensor, slots, scales: torch.Tensor) -> None:
        """Several targets that read the same ``x`` (q, k, v of a layer; gate and up) in two launches:
        ``ys[i] += scale_a * (x @ A_a[slots[i]].T) @ B_a[slots[i]]``.  ``value_buffers`` is one pool tensor or
        one per target.  Same results as ``apply`` called once per target."""
        n = len(ys)
        if not 1 <= n <= _lib.MAX_TARGETS or len(slots) != n:
            raise RuntimeError(f"apply_multi takes 1..{_lib.MAX_TARGETS} targets with one slot each")
        vbs = list(value_buffers) if isinstance(value_buffers, (list, tuple)) else [value_buffers] * n
        h_in, h_out = x.size(1), ys[0].size(1)
        for y, vb in zip(ys, vbs):
            self._check(x, y, key_buffer, vb)
            if y.size(1) != h_out:
                raise RuntimeError("all targets of one call must have the same output width")
        if scales.dtype != x.dtype:
            scales = scales.to(x.dtype)
        pa = _lib.make_pool(key_buffer, a_start, a_len, a_loc, h_in, self.n_slots)
        tg = (_lib.Target * n)()
        for i in range(n):
            tg[i] = _lib.Target(_lib.ptr(ys[i]), _lib.ptr(vbs[i]), vbs[i].numel() // h_out, int(slots[i]))
        # (a call whose expand half is more than 16 items per tile -- q+k+v, a 4096 -> 11008 target -- is run as two
        # launches by the library whatever the flag says: same tiles, same split, same bits)
        flags = self.flags
        _lib.check(_lib.lib().mlora_lora_apply_multi(
            _lib.current_stream(self.device), self.handle, _lib.ptr(self.scratch), self.scratch.numel(), _lib.ptr(x),
            self.T, h_in, h_out, self.max_rank, pa, n, tg, _lib.ptr(scales), int(self.ksplit), flags,
            _lib.dtype_code(x.dtype)))

    def apply(self, y: torch.Tensor, x: torch.Tensor, key_buffer: torch.Tensor, value_buffer: torch.Tensor,
              a_start: torch.Tensor, a_len: torch.Tensor, a_loc: torch.Tensor, slot: int,
              scales: torch.Tensor) -> None:
        """``y[t] += scale_a * (x[t] @ A_a.T) @ B_a`` in place for every token with an adapter."""
        if x.dim() != 2 or y.dim() != 2 or x.size(0) != self.T or y.size(0) != self.T:
            raise RuntimeError(f"x and y must be [T={self.T}, H] matrices")
        if not (x.is_contiguous() and y.is_contiguous()):
            raise RuntimeError("x and y must be contiguous")
        code = _lib.dtype_code(x.dtype)
        if code < 0 or y.dtype != x.dtype or key_buffer.dtype != x.dtype or value_buffer.dtype != x.dtype:
            raise RuntimeError(f"No suitable kernel. h_in={x.size(1)} h_out={y.size(1)} dtype={x.dtype}")
        if scales.dtype != x.dtype:
            scales = scales.to(x.dtype)
        h_in, h_out = x.size(1), y.size(1)
        pa = _lib.make_pool(key_buffer, a_start, a_len, a_loc, h_in, self.n_slots)
        pb = _lib.make_pool(value_buffer, a_start, a_len, a_loc, h_out, self.n_slots)
        _lib.check(_lib.lib().mlora_lora_apply(
            _lib.current_stream(self.device), self.handle, _lib.ptr(self.scratch), self.scratch.numel(),
            _lib.ptr(y), _lib.ptr(x), self.T, h_in, h_out, self.max_rank, pa, pb, int(slot), _lib.ptr(scales),
            int(self.ksplit), self.flags, code))
