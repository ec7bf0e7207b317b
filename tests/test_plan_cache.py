"""Host logic of the plan reuse in the drop-in shims: an entry is reused only for the very same,
unmodified tensor objects and scalars.  CPU only (the cache holds whatever the builder returns)."""
import gc

import torch

from valora_amd import _plan_cache as C


def test_identity_version_and_scalars_decide():
    C.clear()
    built = []

    def build():
        built.append(len(built))
        return ("plan", len(built))

    ids = torch.arange(8)
    a_start = torch.zeros(3, dtype=torch.long)
    a_len = torch.full((3,), 32, dtype=torch.long)
    p1 = C.lookup((ids, a_start, a_len), (8, 16, 4096), build)
    assert C.lookup((ids, a_start, a_len), (8, 16, 4096), build) is p1 and len(built) == 1
    # other scalars: another entry
    p2 = C.lookup((ids, a_start, a_len), (8, 16, 11008), build)
    assert p2 is not p1 and len(built) == 2
    # equal contents in a different tensor object do not match
    assert C.lookup((ids.clone(), a_start, a_len), (8, 16, 4096), build) is not p1 and len(built) == 3
    # an in-place change through torch bumps the version: the old entry is dead
    ids.add_(1)
    p4 = C.lookup((ids, a_start, a_len), (8, 16, 4096), build)
    assert p4 is not p1 and len(built) == 4
    assert C.lookup((ids, a_start, a_len), (8, 16, 4096), build) is p4 and len(built) == 4
    # any of the tensors counts, not only the ids
    a_len[0] = 64
    assert C.lookup((ids, a_start, a_len), (8, 16, 4096), build) is not p4 and len(built) == 5


def test_entries_die_with_their_tensors_and_are_bounded():
    C.clear()
    n = [0]

    def build():
        n[0] += 1
        return n[0]

    keep = []
    for i in range(20):
        t = torch.zeros(4, dtype=torch.long)
        keep.append(t)
        C.lookup((t,), (i,), build)
    assert len(C._entries) <= C._MAX_ENTRIES
    # the most recent ones are still there
    assert C.lookup((keep[-1],), (19,), build) == 20 and n[0] == 20
    # the oldest was evicted and is rebuilt
    assert C.lookup((keep[0],), (0,), build) == 21
    # entries whose tensors are gone are dropped at the next insertion
    del keep[:]
    del t
    gc.collect()
    last = torch.zeros(1)
    C.lookup((last,), ("x",), build)
    assert len(C._entries) == 1 and all(r() is not None for r in C._entries[0][0])


def test_disabled_cache_keeps_nothing():
    C.clear()
    C.set_enabled(False)
    try:
        assert not C.enabled() and C._entries == []
    finally:
        C.set_enabled(True)
    assert C.enabled()
