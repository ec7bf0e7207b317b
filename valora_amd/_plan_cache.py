"""Python face of the plan cache the drop-in entry points keep (it lives in ``csrc/binding.cpp``, beside
the entry points that use it on every call).

The reference's entry points take the per-token adapter ids with every call, and its caller passes
the SAME tensors for all 8 calls of a layer and for all layers of a forward pass
(valora/models/peft/lora_unordered_batch_infer.py:946-1063: ``self.batch_req_bins``,
``self.infer_adapter.a_start / a_len``) -- sometimes as fresh views of them (``self.output_counts[1:]``,
``self.start_ids[1:]``, :1006-1008).  Sorting the tokens and cutting tiles once per call would cost
more than the op itself at decode sizes, so the plans of the last few distinct argument sets are kept.

A tensor is identified by where its data lives and what PyTorch knows about its history:
``(data_ptr, numel, dtype, _version)``.  A fresh view of the same memory has the same key, so it
hits.  The entry holds a reference to every tensor it was built from, which pins their storages: as
long as the entry lives, no other tensor can be handed the same address by the caching allocator, so
an equal key really means the same memory, and ``_version`` says it has not been written through
PyTorch since.  Tensors created under ``torch.inference_mode`` carry no version counter; they are
cached by address alone while ``cache_inference_tensors()`` is true (an in-place write to such a
tensor is then not noticed).  Writes that bypass PyTorch's bookkeeping (a foreign kernel given the
raw pointer) are never seen: ``set_enabled(False)`` turns the reuse off.  A plan serves the context it was
built in and no other: one whose build was only recorded into a stream capture serves that capture alone, and
one cut eagerly (a warm-up before the capture) is not used under capture -- the graph records a build of its own,
so a replay cuts the tiles of whatever the ids tensor holds by then, in buffers that live as long as the graph.

At most ``max_entries()`` plans are kept (least recently used first out); each holds its workspace
(``mlora_workspace_bytes``: KBs at decode sizes, tens of MB for long prefills) and the small index
tensors it pins.  ``clear()`` drops them all.  ``hits`` / ``misses`` count lookups since the module was loaded.
"""
from __future__ import annotations

from typing import Callable, Sequence, Tuple

from ._ext import binding as _b

clear = _b.cache_clear
size = _b.cache_size
enabled = _b.cache_enabled
set_enabled = _b.cache_set_enabled
cache_inference_tensors = _b.cache_inference_tensors
set_cache_inference_tensors = _b.cache_set_inference_tensors
max_entries = _b.cache_max_entries


def __getattr__(name: str):
    if name == "hits":
        return _b.cache_hits()
    if name == "misses":
        return _b.cache_misses()
    raise AttributeError(name)


def lookup(tensors: Sequence, scalars: Tuple[int, ...], build: Callable[[], object]):
    """The value stored for tensors at these addresses (unmodified since) and these integers, or a new one
    from ``build()``.  Returns None without building if one of the tensors cannot be identified or the
    cache is off."""
    tensors, scalars = list(tensors), [int(s) for s in scalars]
    identifiable, value = _b.cache_lookup(tensors, scalars)
    if not identifiable:
        return None
    if value is None:
        value = build()
        _b.cache_insert(tensors, scalars, value)
    return value
