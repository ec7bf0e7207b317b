"""GPU: the adapter-grouped plan and the run-length encoder.

The run-length encoding must be bit-exact with the reference's count_consecutive_requests
(checked against the CPU oracle).  The grouped tile list is the build's own structure and is
checked by invariants: perm is a permutation of the tokens that have an adapter, every group's
size equals the histogram of ids, order inside a group is the original order (stable), tiles
partition the groups."""
import numpy as np
import pytest
import torch

from oracle import lora_oracle as O

pytestmark = pytest.mark.gpu


def _check_plan(ids_cpu, a_len_cpu, n_slots, bm_s, bm_e, dev):
    from valora_amd.plan import LoraPlan
    A = a_len_cpu.numel()
    a_start = (torch.cumsum(a_len_cpu, 0) - a_len_cpu).to(dev)
    plan = LoraPlan(ids_cpu.to(dev), a_start, a_len_cpu.to(dev), 64, n_slots=n_slots, bm_shrink=bm_s,
                    bm_expand=bm_e, ksplit=1)
    h = plan.header()
    ranks = (a_len_cpu // n_slots).tolist()
    valid = [t for t, a in enumerate(ids_cpu.tolist()) if 0 <= a < A and ranks[a] > 0]
    assert h["magic"] == 0x4d4c5241 and h["T"] == ids_cpu.numel()
    assert h["n_active"] == len(valid)
    perm = plan.perm().cpu().tolist()
    assert sorted(perm) == valid, "perm must be a permutation of the tokens that have an adapter"
    pa = plan.position_adapters().cpu().tolist()
    pr = plan.position_ranks().cpu().tolist()
    assert pa == [int(ids_cpu[t]) for t in perm]
    assert pr == [ranks[a] for a in pa]
    assert pa == sorted(pa), "positions are grouped by ascending adapter"
    for i in range(1, len(perm)):
        if pa[i] == pa[i - 1]:
            assert perm[i] > perm[i - 1], "original order is kept inside a group (stable)"
    hist = np.bincount([int(ids_cpu[t]) for t in valid], minlength=A) if valid else np.zeros(A, int)
    assert h["n_groups"] == int((hist > 0).sum())
    assert h["max_rank"] == max([ranks[a] for a in range(A) if hist[a] > 0], default=0)
    for tiles, bm, key in ((plan.tiles_shrink(), bm_s, "n_tiles_shrink"), (plan.tiles_expand(), bm_e, "n_tiles_expand")):
        tiles = tiles.cpu().tolist()
        assert len(tiles) == h[key] == int(sum(-(-c // bm) for c in hist if c > 0))
        pos = 0
        for (a, r, p0, cnt, st, *_rest) in tiles:
            assert p0 == pos and 1 <= cnt <= bm and r == ranks[a] and st == int(a_start[a])
            assert all(x == a for x in pa[p0:p0 + cnt])
            pos += cnt
        assert pos == len(valid)


@pytest.mark.parametrize("T,A,style", [
    (1, 1, "random"), (256, 64, "zipf"), (1000, 7, "random"), (4416, 32, "runs"), (64, 600, "random"),
    (5000, 5000, "random"), (300, 8192, "random"), (3000, 2048, "random"), (3000, 2049, "random"), (777, 3, "holes"), (20000, 16, "runs"), (0, 4, "random")])
def test_plan_invariants(dev, T, A, style):
    g = torch.Generator().manual_seed(T * 31 + A)
    a_len = torch.randint(1, 9, (A,), generator=g) * 8 * 4
    if style == "zipf":
        from valora_amd.workloads import zipf_ids
        ids = zipf_ids(A, T, 0.6, g)
    elif style == "runs":
        ids = torch.repeat_interleave(torch.randint(0, A, (T,), generator=g),
                                      torch.randint(1, 600, (T,), generator=g))[:T]
    elif style == "holes":
        ids = torch.randint(-2, A + 2, (T,), generator=g)       # out-of-range ids = no adapter
        a_len[1] = 0                                            # rank-0 adapter = no adapter
    else:
        ids = torch.randint(0, A, (T,), generator=g) if T else torch.zeros(0, dtype=torch.long)
    for bm_s, bm_e in ((16, 32), (64, 256)):
        _check_plan(ids, a_len, 4, bm_s, bm_e, dev)


@pytest.mark.parametrize("T", [1, 2, 63, 64, 65, 1024, 1025, 5000])
@pytest.mark.parametrize("style", ["random", "runs", "equal", "distinct"])
def test_count_consecutive_bit_exact(dev, T, style):
    from valora_amd.segments import count_consecutive_requests
    g = torch.Generator().manual_seed(T)
    lora_rank = torch.tensor([32, 64, 128, 256, 32, 96])
    if style == "random":
        ids = torch.randint(0, 6, (T,), generator=g)
    elif style == "runs":
        ids = torch.repeat_interleave(torch.randint(0, 6, (T,), generator=g),
                                      torch.randint(1, 40, (T,), generator=g))[:T]
    elif style == "equal":
        ids = torch.full((T,), 4)
    else:
        ids = torch.arange(T) % 6
    oc, rc, li, st, num = count_consecutive_requests(lora_rank.to(dev), ids.to(dev))
    want = O.count_consecutive_requests(lora_rank, ids)
    P = int(num.item())
    assert P == len(want[0])
    for got, w in zip((oc, rc, li, st), want):
        assert got.dtype == torch.long and got[:P].cpu().tolist() == w
