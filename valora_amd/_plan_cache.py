"""Reuse of the per-batch plan by the drop-in entry points.

The reference's entry points take the per-token adapter ids with every call, and its caller passes
the SAME tensors for all 8 calls of a layer and for all layers of a forward pass
(valora/models/peft/lora_unordered_batch_infer.py:946-1063: ``self.batch_req_bins``,
``self.infer_adapter.a_start / a_len``) -- sometimes as fresh views of them (``self.output_counts[1:]``,
``self.start_ids[1:]``, :1006-1008).  Sorting the tokens and cutting tiles once per call would cost
more than the op itself at decode sizes, so the shims keep the plans of the last few distinct
argument sets.

A tensor is identified by where its data lives and what PyTorch knows about its history:
``(data_ptr, numel, dtype, _version)``.  A fresh view of the same memory has the same key, so it
hits.  The entry holds a reference to every tensor it was built from, which pins their storages: as
long as the entry lives, no other tensor can be handed the same address by the caching allocator, so
an equal key really means the same memory, and ``_version`` says it has not been written through
PyTorch since.  Tensors created under ``torch.inference_mode`` carry no version counter; they are
cached by address alone while ``cache_inference_tensors`` is true (an in-place write to such a
tensor is then not noticed).  Writes that bypass PyTorch's bookkeeping (a foreign kernel given the
raw pointer) are never seen: ``set_enabled(False)`` turns the reuse off.

At most ``_MAX_ENTRIES`` plans are kept (least recently used first out); each holds its scratch
buffer (``mlora_scratch_bytes`` x 4 targets: KBs at decode sizes, tens of MB for long prefills) and
the small index tensors it pins.  ``clear()`` drops them all.
"""
from __future__ import annotations

from typing import Callable, List, Sequence, Tuple

import torch

_MAX_ENTRIES = 8
_enabled = True
cache_inference_tensors = True
_entries: List[tuple] = []      # (keys, scalars, value, pinned tensors), most recent last
hits = 0
misses = 0


def set_enabled(flag: bool) -> None:
    global _enabled
    _enabled = bool(flag)
    if not _enabled:
        clear()


def enabled() -> bool:
    return _enabled


def clear() -> None:
    _entries.clear()


def _key(t: torch.Tensor):
    """None if the tensor cannot be cached (no way to tell whether it was modified)."""
    if t.is_inference():
        if not cache_inference_tensors:
            return None
        version = -1
    else:
        version = t._version
    return (t.data_ptr(), t.numel(), t.dtype, version)


def lookup(tensors: Sequence[torch.Tensor], scalars: Tuple, build: Callable[[], object]):
    """The value built for tensors at these addresses (unmodified since) and these scalars, or a new one.
    Returns None without building if one of the tensors cannot be identified."""
    global hits, misses
    keys = tuple(_key(t) for t in tensors)
    if any(k is None for k in keys):
        return None
    for i in range(len(_entries) - 1, -1, -1):
        k, sc, value, _pins = _entries[i]
        if k == keys and sc == scalars:
            if i != len(_entries) - 1:
                _entries.append(_entries.pop(i))
            hits += 1
            return value
    misses += 1
    value = build()
    _entries.append((keys, scalars, value, tuple(tensors)))
    del _entries[:-_MAX_ENTRIES]
    return value
