"""Seeded sweep of the planned LoRA op over shapes and tile parameters nobody picked by hand: odd
token counts, widths that are multiples of 8 but of nothing larger, mixed ranks, 1 to 5 pool slots,
every shrink tile height with every split-K finish, ids with holes.  Each case is compared with
oracle/lora_oracle.py at the stated tolerance, rows without an adapter must come back bit-identical,
and a two-target call must equal the two single calls bit for bit."""
import random

import pytest
import torch

from oracle import lora_oracle as O
from valora_amd import workloads as W
from valora_amd.plan import LoraPlan
from tests._util import assert_parity

pytestmark = pytest.mark.gpu

WIDTHS = [8, 24, 72, 136, 264, 520, 1000, 1032, 2056, 4096]
RANKS = [8, 16, 24, 32, 40, 64, 128]


def draw(seed):
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    T = rnd.choice([1, 2, 15, 16, 17, 31, 33, 63, 65, 127, 129, 200, 257, 511, 700])
    h_in, h_out = rnd.choice(WIDTHS), rnd.choice(WIDTHS)
    n_adapters = rnd.choice([1, 2, 3, 5, 9, 17])
    big = rnd.random() < 0.25
    ranks = [rnd.choice(RANKS if big else RANKS[:6]) for _ in range(n_adapters)]
    n_slots = rnd.choice([1, 2, 4, 4, 5])
    cfg = dict(bm_shrink=rnd.choice([16, 32, 64, 128, 256]), bm_expand=rnd.choice([16, 32, 48, 64, 96, 128, 192, 256]),
               ksplit=rnd.choice([1, 2, 3, 4, 8]), reduce_in_expand=rnd.random() < 0.5)
    if max(ranks) > 64 and cfg["bm_shrink"] in (64, 256):
        cfg["bm_shrink"] //= 2      # ranks above 64 have no 64- or 256-token shrink tile (the library says so)
    style = rnd.choice(["random", "sorted", "holes", "one", "none"])
    return dtype, T, h_in, h_out, ranks, n_slots, cfg, style


@pytest.mark.parametrize("seed", range(48))
def test_random_shape(dev, seed):
    dtype, T, h_in, h_out, ranks, n_slots, cfg, style = draw(seed)
    what = f"seed {seed}: T={T} h_in={h_in} h_out={h_out} ranks={ranks} slots={n_slots} {cfg} {style} {dtype}"
    print(what, flush=True)
    g = torch.Generator().manual_seed(1000 + seed)
    A = len(ranks)
    scal = [0.25 + 0.5 * ((7 * i) % 5) for i in range(A)]
    pool = W.make_pool(ranks, h_in, h_out, dtype, g, True, n_slots=n_slots, std=0.05, scalings=scal, heads=1,
                       extra_rows=3)
    if style == "random":
        ids = torch.randint(0, A, (T,), generator=g)
    elif style == "sorted":
        ids = torch.randint(0, A, (T,), generator=g).sort().values
    elif style == "holes":
        ids = torch.randint(-1, A, (T,), generator=g)
    elif style == "one":
        ids = torch.full((T,), A - 1, dtype=torch.long)
    else:
        ids = torch.full((T,), -1, dtype=torch.long)
    x = torch.randn(T, h_in, generator=g).to(dtype)
    slots = [seed % n_slots, (seed + 1) % n_slots]
    y0 = [torch.randn(T, h_out, generator=g).to(dtype) for _ in slots]
    R = max(ranks)

    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    plan = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, R, n_slots=n_slots, hidden=h_in, **cfg)
    xd = x.to(dev)
    single = []
    for slot, y in zip(slots, y0):
        yd = y.to(dev)
        plan.apply(yd, xd, pd.key_buffer, pd.value_buffer, *idx, slot, pd.a_scaling)
        want = O.lora_op(y, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, slot,
                         pool.a_scaling, n_slots=n_slots)
        got = yd.cpu()
        assert_parity(got, want, what + f" slot {slot}")
        assert torch.equal(got[ids < 0], y[ids < 0]), what
        single.append(got)
    if slots[0] != slots[1]:
        ys = [y.to(dev) for y in y0]
        plan.apply_multi(ys, xd, pd.key_buffer, pd.value_buffer, *idx, slots, pd.a_scaling)
        for got, one in zip(ys, single):
            assert torch.equal(got.cpu(), one), what + " (two targets in one call)"


@pytest.mark.parametrize("seed", range(400, 448))
def test_random_shape_one_launch(dev, seed):
    """The one-launch op on shapes nobody picked: one to three targets, ranks up to 64, any split-K count, ids with
    holes, twice on one plan (the hand-off's launch tags move on).  Compared with the oracle, and bit for bit with the
    two launches of the same split (the library caps K chunks x targets at 16 shrink items per tile, so the
    two-launch plan is cut with the capped count)."""
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    T = rnd.choice([1, 2, 15, 16, 17, 31, 33, 63, 65, 127, 129, 200, 257, 511, 700, 1500])
    h_in, h_out = rnd.choice(WIDTHS + [5120]), rnd.choice(WIDTHS + [5120])
    A = rnd.choice([1, 2, 3, 5, 9, 17, 40])
    ranks = [rnd.choice([8, 16, 24, 32, 40, 48, 64]) for _ in range(A)]
    n_slots = rnd.choice([1, 2, 4, 4, 5])
    ks = rnd.choice([2, 3, 4, 5, 8])
    style = rnd.choice(["random", "sorted", "holes", "one", "none", "zipf"])
    nt = rnd.choice([1, 1, 2, 3]) if n_slots >= 3 else (rnd.choice([1, 2]) if n_slots == 2 else 1)
    what = f"seed {seed}: T={T} h_in={h_in} h_out={h_out} ranks={ranks} slots={n_slots} ks={ks} targets={nt} {style} {dtype}"
    print(what, flush=True)
    g = torch.Generator().manual_seed(5000 + seed)
    pool = W.make_pool(ranks, h_in, h_out, dtype, g, True, n_slots=n_slots, std=0.05,
                       scalings=[0.25 + 0.5 * ((7 * i) % 5) for i in range(A)], heads=1, extra_rows=3)
    ids = {"random": lambda: torch.randint(0, A, (T,), generator=g),
           "sorted": lambda: torch.randint(0, A, (T,), generator=g).sort().values,
           "holes": lambda: torch.randint(-1, A, (T,), generator=g),
           "one": lambda: torch.full((T,), A - 1, dtype=torch.long),
           "zipf": lambda: W.zipf_ids(A, T, 0.8, g),
           "none": lambda: torch.full((T,), -1, dtype=torch.long)}[style]()
    x = torch.randn(T, h_in, generator=g).to(dtype)
    slots = rnd.sample(range(n_slots), nt)
    y0 = [torch.randn(T, h_out, generator=g).to(dtype) for _ in slots]
    R = max(ranks)
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    xd, idd = x.to(dev), ids.to(dev)
    one = LoraPlan(idd, pd.a_start, pd.a_len, R, n_slots=n_slots, hidden=h_in, one_launch=True, ksplit=ks)
    two = LoraPlan(idd, pd.a_start, pd.a_len, R, n_slots=n_slots, hidden=h_in, one_launch=False, bm_shrink=16,
                   bm_expand=16, ksplit=min(ks, 16 // nt), reduce_in_expand=True)
    want = [O.lora_op(y0[i], x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, slot,
                      pool.a_scaling, n_slots=n_slots) for i, slot in enumerate(slots)]
    for rep in range(2):
        y1, y2 = [y.to(dev) for y in y0], [y.to(dev) for y in y0]
        if nt == 1:
            one.apply(y1[0], xd, pd.key_buffer, pd.value_buffer, *idx, slots[0], pd.a_scaling)
            two.apply(y2[0], xd, pd.key_buffer, pd.value_buffer, *idx, slots[0], pd.a_scaling)
        else:
            one.apply_multi(y1, xd, pd.key_buffer, pd.value_buffer, *idx, slots, pd.a_scaling)
            two.apply_multi(y2, xd, pd.key_buffer, pd.value_buffer, *idx, slots, pd.a_scaling)
        for i in range(nt):
            got = y1[i].cpu()
            assert_parity(got, want[i], what + f" target {i} call {rep}")
            assert torch.equal(got, y2[i].cpu()), what + " (one launch against two)"
            assert torch.equal(got[ids < 0], y0[i][ids < 0]), what


@pytest.mark.parametrize("seed", range(100, 124))
def test_random_shape_drop_in_bgmv(dev, seed):
    """The same draw through the reference's operator signature (two dispatch_bgmv calls with the
    caller's own [T, R] intermediate between them; the library picks the tile parameters)."""
    from valora_amd.kernels import dispatch_bgmv
    dtype, T, h_in, h_out, ranks, _, _, style = draw(seed)
    R = max(ranks)
    if h_in <= R:
        h_in = 1032      # the operator reads the direction from the widths: shrink needs h_in > R
    if h_out <= R:
        h_out = 520
    what = f"seed {seed}: T={T} h_in={h_in} h_out={h_out} ranks={ranks} {style} {dtype}"
    print(what, flush=True)
    g = torch.Generator().manual_seed(2000 + seed)
    A = len(ranks)
    pool = W.make_pool(ranks, h_in, h_out, dtype, g, True, std=0.05, scalings=[0.5 + 0.125 * i for i in range(A)],
                       heads=1)
    ids = {"random": torch.randint(0, A, (T,), generator=g), "sorted": torch.randint(0, A, (T,), generator=g).sort().values,
           "holes": torch.randint(-1, A, (T,), generator=g), "one": torch.full((T,), A - 1, dtype=torch.long),
           "none": torch.full((T,), -1, dtype=torch.long)}[style]
    x = torch.randn(T, h_in, generator=g).to(dtype)
    y0 = torch.randn(T, h_out, generator=g).to(dtype)
    slot = seed % 4
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    delta = torch.zeros(T, R, dtype=dtype, device=dev)
    y = y0.to(dev)
    dispatch_bgmv(delta, x.to(dev), pd.key_buffer, *idx, ids.to(dev), slot, pd.a_scaling)
    dispatch_bgmv(y, delta, pd.value_buffer, *idx, ids.to(dev), slot, pd.a_scaling)
    cidx = (pool.a_start, pool.a_len, pool.a_loc)
    want_v = O.bgmv_shrink(torch.zeros(T, R, dtype=dtype), x, pool.key_buffer, *cidx, ids, slot)
    assert_parity(delta.cpu(), want_v, what + " shrink")
    want = O.bgmv_expand(y0, delta.cpu(), pool.value_buffer, *cidx, ids, slot, pool.a_scaling)
    assert_parity(y.cpu(), want, what + " expand")
    assert torch.equal(y.cpu()[ids < 0], y0[ids < 0]), what


@pytest.mark.parametrize("bm_shrink", [16, 32, 128])
@pytest.mark.parametrize("ksplit,h_in", [(16, 4096), (32, 4096), (32, 11008), (64, 1032), (64, 8192)])
def test_many_k_chunks(dev, bm_shrink, ksplit, h_in):
    """Split-K counts the tile table uses for small batches and wide inputs, including more chunks than the
    width has 128-element pieces (the surplus chunks are empty and must contribute zeros), with both ways
    of summing the chunks."""
    g = torch.Generator().manual_seed(ksplit + h_in)
    ranks, T, h_out = [64, 16, 128, 8], 70, 520
    pool = W.make_pool(ranks, h_in, h_out, torch.bfloat16, g, True, std=0.05, scalings=[1.0, 0.5, 2.0, 0.25], heads=1)
    ids = torch.randint(-1, len(ranks), (T,), generator=g)
    x = torch.randn(T, h_in, generator=g).bfloat16()
    y0 = torch.randn(T, h_out, generator=g).bfloat16()
    want = O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 2,
                     pool.a_scaling)
    pd = pool.to(dev)
    for rie in (False, True):
        plan = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, 128, hidden=h_in, bm_shrink=bm_shrink, bm_expand=32,
                        ksplit=ksplit, reduce_in_expand=rie)
        y = y0.to(dev)
        plan.apply(y, x.to(dev), pd.key_buffer, pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, 2, pd.a_scaling)
        assert_parity(y.cpu(), want, f"ksplit {ksplit} h_in {h_in} bm {bm_shrink} rie {rie}")
        assert torch.equal(y.cpu()[ids < 0], y0[ids < 0])


TABLE_CASES = [
    # (hidden, tokens, rank, resident adapters): shapes of the widths the tile table holds measured entries
    # for beside 4096 and 11008, decode-like and prefill-like, through the configuration the table gives them
    (5120, 8, 16, 8), (5120, 64, 32, 32), (5120, 256, 16, 100), (5120, 1000, 64, 8), (5120, 2300, 128, 8),
    (6144, 5, 64, 8), (6144, 64, 16, 32), (6144, 256, 32, 32), (6144, 700, 16, 100), (6144, 3000, 64, 32),
    (8192, 8, 32, 8), (8192, 40, 128, 8), (8192, 256, 16, 8), (8192, 1024, 32, 32), (8192, 2048, 64, 8),
    (13824, 3, 16, 8), (13824, 64, 64, 32), (13824, 200, 16, 32), (13824, 900, 32, 8), (13824, 2100, 64, 8),
    (2048, 8, 16, 8), (2048, 256, 32, 32), (2048, 3000, 64, 8), (3072, 60, 64, 8), (3072, 1024, 16, 100),
    (7168, 7, 32, 8), (7168, 256, 16, 32), (7168, 2500, 128, 8), (14336, 64, 16, 32), (14336, 1500, 64, 8),
    (28672, 8, 16, 8), (28672, 200, 32, 8), (28672, 1100, 64, 8),
    # one adapter for the whole batch, and the 128- / 512- / 2048-token buckets
    (4096, 1, 16, 1), (4096, 100, 64, 1), (4096, 500, 16, 1), (4096, 1500, 32, 1), (4096, 5000, 64, 1), (4096, 700, 128, 1),
    (11008, 300, 16, 1), (11008, 2000, 64, 1), (8192, 120, 32, 1), (2048, 1300, 16, 1), (28672, 400, 16, 1),
    (4096, 100, 16, 100), (4096, 400, 32, 32), (4096, 1500, 16, 100), (4096, 2000, 64, 32), (11008, 500, 64, 8),
    (4096, 300, 16, 500),
    # 256-token shrink tiles (the table's choice for 16384 single-adapter tokens) and the 8192-token bucket
    (4096, 16384, 64, 1), (4096, 16000, 32, 1), (4096, 9000, 64, 1), (4096, 8000, 64, 8), (11008, 6000, 16, 32),
]


@pytest.mark.parametrize("hidden,T,rank,n_adapters", TABLE_CASES)
def test_table_configurations_of_other_widths(dev, hidden, T, rank, n_adapters):
    """Widths 2048 ... 28672.  The plan takes its tile heights, split-K count and launch structure from the table entry of the shape
    (one launch for several of the small ones); whatever the entry says, the result is the oracle's."""
    from valora_amd import tile_table
    g = torch.Generator().manual_seed(hidden + T + rank)
    dtype = torch.bfloat16 if (T + rank) % 32 else torch.float16
    h_out = 4096 if hidden > 8192 else hidden          # 11008 and wider are MLP widths: down-projection shape
    pool = W.make_pool([rank] * n_adapters, hidden, h_out, dtype, g, True, n_slots=1, std=0.03, heads=1)
    req = 1 if T <= 1024 else 128
    ids = torch.repeat_interleave(W.zipf_ids(n_adapters, (T + req - 1) // req, 0.7, g), req)[:T]
    x = torch.randn(T, hidden, generator=g).to(dtype)
    y0 = torch.randn(T, h_out, generator=g).to(dtype)
    cfg = tile_table.lookup(T, rank, hidden, n_adapters)
    what = f"hidden {hidden} T {T} rank {rank} adapters {n_adapters}: {cfg}"
    print(what, flush=True)
    pd = pool.to(dev)
    plan = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, rank, n_slots=1, hidden=hidden)
    assert (plan.bm_shrink, plan.bm_expand) == ((16, 16) if plan.one_launch else (cfg.bm_shrink, cfg.bm_expand))
    assert plan.one_launch == (cfg.one_launch and rank <= 64)
    y = y0.to(dev)
    plan.apply(y, x.to(dev), pd.key_buffer, pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, 0, pd.a_scaling)
    want = O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 0,
                     pool.a_scaling, n_slots=1)
    assert_parity(y.cpu(), want, what)


@pytest.mark.parametrize("seed", range(300, 330))
def test_expand_column_loop_gives_the_same_bits(dev, seed):
    """The expand of 16-token tiles as one workgroup per (tile, 256-column chunk) and as one workgroup per two chunks
    (what the library picks by itself for grids several times the device, forced here for any size): same bits, for
    finished v and for split-K partials summed in the expand, one target and several, ranks up to 128, output widths
    that end inside a chunk or leave the second chunk of a pair empty."""
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    T = rnd.choice([1, 3, 16, 17, 40, 100, 256, 300])
    h_in = rnd.choice([256, 520, 1032, 4096])
    h_out = rnd.choice([264, 512, 520, 768, 1000, 1032, 2056, 4096, 11008])
    A = rnd.choice([1, 3, 9, 33, 70])
    ranks = [rnd.choice([8, 16, 24, 32, 64, 128] if rnd.random() < 0.3 else [8, 16, 32]) for _ in range(A)]
    ksplit = rnd.choice([1, 2, 4])
    rie = ksplit > 1 and rnd.random() < 0.6
    n_targets = rnd.choice([1, 1, 2, 3])
    what = f"seed {seed}: {dtype} T={T} {h_in}->{h_out} A={A} ks={ksplit} rie={rie} targets={n_targets}"
    print(what, flush=True)
    g = torch.Generator().manual_seed(3000 + seed)
    pool = W.make_pool(ranks, h_in, h_out, dtype, g, True, n_slots=4, std=0.05, heads=1)
    ids = torch.randint(-1 if seed % 3 == 0 else 0, A, (T,), generator=g)
    x = torch.randn(T, h_in, generator=g).to(dtype)
    y0 = [torch.randn(T, h_out, generator=g).to(dtype) for _ in range(n_targets)]
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    R = max(ranks)
    kw = dict(hidden=h_in, bm_shrink=rnd.choice([16, 32]), bm_expand=16, ksplit=ksplit, reduce_in_expand=rie, one_launch=False)
    outs = []
    for loop in (False, True):
        plan = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, R, expand_column_loop=loop, **kw)
        ys = [y.to(dev) for y in y0]
        if n_targets == 1:
            plan.apply(ys[0], x.to(dev), pd.key_buffer, pd.value_buffer, *idx, 2, pd.a_scaling)
        else:
            plan.apply_multi(ys, x.to(dev), pd.key_buffer, pd.value_buffer, *idx, list(range(n_targets)), pd.a_scaling)
        outs.append([y.cpu() for y in ys])
    for a, b in zip(*outs):
        assert torch.equal(a, b), what
    slot0 = 2 if n_targets == 1 else 0
    want = O.lora_op(y0[0], x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, slot0,
                     pool.a_scaling)
    assert_parity(outs[1][0], want, what)
    assert torch.equal(outs[1][0][ids < 0], y0[0][ids < 0])
