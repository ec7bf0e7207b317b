"""Host logic of the plan reuse in the drop-in shims: an entry is reused for tensors that live at the same
address and have not been modified through PyTorch since -- fresh views of the same memory included -- and
for the same scalars.  CPU only: the cache of the compiled binding, driven through its Python face (it holds
whatever the builder returns)."""
import torch

from valora_amd import _plan_cache as C


def _builder():
    built = []

    def build():
        built.append(len(built))
        return ("plan", len(built))
    return built, build


def test_address_version_and_scalars_decide():
    C.clear()
    built, build = _builder()
    ids = torch.arange(8)
    a_start = torch.zeros(3, dtype=torch.long)
    a_len = torch.full((3,), 32, dtype=torch.long)
    p1 = C.lookup((ids, a_start, a_len), (8, 16, 4096), build)
    assert C.lookup((ids, a_start, a_len), (8, 16, 4096), build) is p1 and len(built) == 1
    # other scalars: another entry
    p2 = C.lookup((ids, a_start, a_len), (8, 16, 11008), build)
    assert p2 is not p1 and len(built) == 2
    # equal contents at another address do not match
    assert C.lookup((ids.clone(), a_start, a_len), (8, 16, 4096), build) is not p1 and len(built) == 3
    # an in-place change through torch bumps the version: the old entry is dead
    ids.add_(1)
    p4 = C.lookup((ids, a_start, a_len), (8, 16, 4096), build)
    assert p4 is not p1 and len(built) == 4
    assert C.lookup((ids, a_start, a_len), (8, 16, 4096), build) is p4 and len(built) == 4
    # any of the tensors counts, not only the ids
    a_len[0] = 64
    assert C.lookup((ids, a_start, a_len), (8, 16, 4096), build) is not p4 and len(built) == 5


def test_fresh_views_of_the_same_memory_hit():
    """The reference's compensation branch passes ``output_counts[1:]`` / ``start_ids[1:]`` anew with every
    call (lora_unordered_batch_infer.py:1006-1008): a new tensor object each time, the same memory."""
    C.clear()
    built, build = _builder()
    oc = torch.ones(128, dtype=torch.long)
    st = torch.arange(129)
    ids = torch.arange(40)
    first = C.lookup((ids, oc[1:], st[1:]), (40,), build)
    h0 = C.hits
    for _ in range(5):
        assert C.lookup((ids, oc[1:], st[1:]), (40,), build) is first
    assert C.hits - h0 == 5 and len(built) == 1
    # another slice of the same storage is other data
    assert C.lookup((ids, oc[2:], st[1:]), (40,), build) is not first and len(built) == 2
    # a write through ANY view of the storage is seen (views share the version counter)
    oc[5] = 7
    assert C.lookup((ids, oc[1:], st[1:]), (40,), build) is not first and len(built) == 3


def test_recycled_addresses_cannot_match():
    """The entry pins the tensors it was built from, so the allocator cannot hand their address to a new
    tensor while the entry lives: a new tensor with other contents never inherits a plan."""
    C.clear()
    built, build = _builder()
    seen = set()
    for i in range(50):
        t = torch.full((16,), i, dtype=torch.long)       # a new tensor per 'forward pass', freed by the caller
        assert t.data_ptr() not in seen or C.size() >= C.max_entries()
        C.lookup((t,), (16,), build)
        seen.add(t.data_ptr())
        del t
    assert len(built) == 50 and C.size() == C.max_entries()


def test_entries_are_bounded_and_lru():
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
    assert C.size() == C.max_entries()
    assert C.lookup((keep[-1],), (19,), build) == 20 and n[0] == 20      # the most recent ones are still there
    assert C.lookup((keep[0],), (0,), build) == 21                       # the oldest was evicted and is rebuilt
    C.clear()
    assert C.size() == 0


def test_inference_tensors():
    """Tensors created under inference_mode have no version counter: cached by address while
    cache_inference_tensors is true, never cached when it is false."""
    C.clear()
    built, build = _builder()
    with torch.inference_mode():
        ids = torch.arange(8)
        a = C.lookup((ids,), (8,), build)
        assert C.lookup((ids,), (8,), build) is a and len(built) == 1
        C.set_cache_inference_tensors(False)
        try:
            assert C.lookup((ids,), (8,), build) is None and len(built) == 1
        finally:
            C.set_cache_inference_tensors(True)


def test_disabled_cache_keeps_nothing():
    C.clear()
    C.set_enabled(False)
    try:
        assert not C.enabled() and C.size() == 0
    finally:
        C.set_enabled(True)
    assert C.enabled()
