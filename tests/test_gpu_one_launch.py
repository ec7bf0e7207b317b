"""GPU: the one-launch op (shrink and expand items of one grid, hand-off inside the launch).

Its contract is "bit-identical to the two-launch op with the same ksplit whose expand sums the K chunks", on
every path an item can take: partials handed over by the shrink items, partials recomputed because the wait
was given up (forced from the host with a wait bound of zero -- no kernel is ever made to wait or hang), items
the device cannot hold from the start (they take part in the hand-off like the others), several targets in one
call, and -- the part a single call cannot show -- launch after launch on one plan, where a stamp left behind by
the previous launch must never be taken for a fresh one."""
import random

import pytest
import torch

from oracle import lora_oracle as O
from valora_amd import workloads as W
from valora_amd.plan import LoraPlan
from tests._util import assert_parity

pytestmark = pytest.mark.gpu


def _pair(wd, name, R, hidden, ksplit, **kw):
    t = wd.target(name); p = t.pool
    one = LoraPlan(wd.ids, p.a_start, p.a_len, R, hidden=hidden, one_launch=True, ksplit=ksplit, **kw)
    two = LoraPlan(wd.ids, p.a_start, p.a_len, R, hidden=hidden, one_launch=False, bm_shrink=16, bm_expand=16,
                   ksplit=one.ksplit, reduce_in_expand=True)
    assert one.one_launch and not two.one_launch
    return one, two


def test_launch_after_launch_on_one_plan(dev):
    """32 'layers' with their own x, y and pool on ONE plan, three times over, single-target and three-target
    calls interleaved (so the number of shrink items per tile changes from launch to launch): every result
    equals the two-launch op's, bit for bit."""
    w = W.config2(hidden=1024, n_tokens=200, n_adapters=48)
    wd = w.to(dev)
    t = wd.target("q"); p = t.pool
    R = max(p.ranks)
    one, two = _pair(wd, "q", R, 1024, 4)
    g = torch.Generator(device=dev).manual_seed(5)
    L = 32
    kb = [(torch.randn(p.key_buffer.shape, generator=g, device=dev) * 0.05).to(w.dtype) for _ in range(4)]
    vb = [(torch.randn(p.value_buffer.shape, generator=g, device=dev) * 0.05).to(w.dtype) for _ in range(4)]
    xs = [torch.randn(w.T, 1024, generator=g, device=dev).to(w.dtype) for _ in range(L)]
    y0 = [torch.randn(w.T, 1024, generator=g, device=dev).to(w.dtype) for _ in range(L)]
    idx = (p.a_start, p.a_len, p.a_loc)
    for rep in range(3):
        got = [y.clone() for y in y0]
        want = [y.clone() for y in y0]
        for plan, ys in ((one, got), (two, want)):
            for l in range(L):
                if l % 5 == 3:     # a q+k+v style call: three targets share x
                    trio = [ys[l], ys[(l + 1) % L], ys[(l + 2) % L]]
                    plan.apply_multi(trio, xs[l], kb[l % 4], vb[l % 4], *idx, [0, 1, 2], p.a_scaling)
                else:
                    plan.apply(ys[l], xs[l], kb[l % 4], vb[l % 4], *idx, l % 4, p.a_scaling)
        torch.cuda.synchronize()
        for l in range(L):
            assert torch.equal(got[l], want[l]), f"repetition {rep}, layer {l}"
    # and the numbers are the operator's: one layer against the oracle
    y = y0[0].clone()
    one.apply(y, xs[0], kb[0], vb[0], *idx, 0, p.a_scaling)
    ref = O.lora_op(y0[0].cpu(), xs[0].cpu(), kb[0].cpu(), vb[0].cpu(), p.a_start.cpu(), p.a_len.cpu(),
                    p.a_loc.cpu(), w.ids, 0, p.a_scaling.cpu())
    assert_parity(y.cpu(), ref, "one launch vs oracle")


def test_graph_replays_of_a_layer_loop(dev):
    """The benchmark's shape of use: a loop over layers on one plan captured in a HIP graph and replayed,
    with eager work in between; every replay equals the eager two-launch result."""
    w = W.config2(hidden=512, n_tokens=128, n_adapters=40)
    wd = w.to(dev)
    t = wd.target("q"); p = t.pool
    one, two = _pair(wd, "q", max(p.ranks), 512, 4)
    g = torch.Generator(device=dev).manual_seed(9)
    L = 6
    xs = [torch.randn(w.T, 512, generator=g, device=dev).to(w.dtype) for _ in range(L)]
    y0 = [torch.randn(w.T, 512, generator=g, device=dev).to(w.dtype) for _ in range(L)]
    ys = [y.clone() for y in y0]
    idx = (p.a_start, p.a_len, p.a_loc)

    def loop(plan, out):
        for l in range(L):
            plan.apply(out[l], xs[l], p.key_buffer, p.value_buffer, *idx, l % 4, p.a_scaling)

    want = [y.clone() for y in y0]
    loop(two, want)
    torch.cuda.synchronize()
    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(s):
        loop(one, ys)                         # warm-up on the capture stream
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            loop(one, ys)
    torch.cuda.current_stream(dev).wait_stream(s)
    for i in range(5):
        for y, src in zip(ys, y0):
            y.copy_(src)
        junk = torch.randn(1 << 20, device=dev).sum()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for l in range(L):
            assert torch.equal(ys[l], want[l]), f"replay {i}, layer {l}"
        assert torch.isfinite(junk)


@pytest.mark.parametrize("seed", range(24))
def test_one_launch_random_shapes(dev, seed):
    rnd = random.Random(500 + seed)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    T = rnd.choice([1, 2, 15, 16, 17, 33, 64, 100, 129, 256, 300])
    h_in, h_out = rnd.choice([256, 264, 520, 1032, 2056, 4096]), rnd.choice([8, 72, 264, 520, 1000, 1032, 4096])
    A = rnd.choice([1, 2, 5, 17, 64])
    ranks = [rnd.choice([8, 16, 24, 32, 40, 64]) for _ in range(A)]
    n_slots = rnd.choice([1, 2, 4, 5])
    ks = rnd.choice([2, 3, 4, 5, 8, 16])
    n_targets = rnd.choice([1, 1, 2, 3, 4])
    no_wait = rnd.random() < 0.3
    style = rnd.choice(["random", "sorted", "holes", "one"])
    what = (f"seed {seed}: {dtype} T={T} {h_in}->{h_out} ranks={ranks[:6]}.. slots={n_slots} ks={ks} "
            f"targets={n_targets} no_wait={no_wait} {style}")
    print(what, flush=True)
    g = torch.Generator().manual_seed(2000 + seed)
    pool = W.make_pool(ranks, h_in, h_out, dtype, g, True, n_slots=n_slots, std=0.05,
                       scalings=[0.25 + 0.5 * ((7 * i) % 5) for i in range(A)], heads=1, extra_rows=3)
    if style == "random":
        ids = torch.randint(0, A, (T,), generator=g)
    elif style == "sorted":
        ids = torch.randint(0, A, (T,), generator=g).sort().values
    elif style == "holes":
        ids = torch.randint(-1, A, (T,), generator=g)
    else:
        ids = torch.full((T,), A - 1, dtype=torch.long)
    x = torch.randn(T, h_in, generator=g).to(dtype)
    y0 = [torch.randn(T, h_out, generator=g).to(dtype) for _ in range(n_targets)]
    slots = [(seed + i) % n_slots for i in range(n_targets)]
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    R = max(ranks)
    one = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, R, n_slots=n_slots, hidden=h_in, one_launch=True, ksplit=ks,
                   one_launch_no_wait=no_wait)
    two = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, R, n_slots=n_slots, hidden=h_in, one_launch=False,
                   bm_shrink=16, bm_expand=16, ksplit=one.ksplit, reduce_in_expand=True)
    xd = x.to(dev)
    for rep in range(2):                       # twice on the same plan
        got = [y.to(dev) for y in y0]
        if n_targets == 1:
            one.apply(got[0], xd, pd.key_buffer, pd.value_buffer, *idx, slots[0], pd.a_scaling)
        else:
            one.apply_multi(got, xd, pd.key_buffer, pd.value_buffer, *idx, slots, pd.a_scaling)
        for i in range(n_targets):
            ref = O.lora_op(y0[i], x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids,
                            slots[i], pool.a_scaling, n_slots=n_slots)
            assert_parity(got[i].cpu(), ref, what + f" target {i} rep {rep}")
            none = (ids < 0)
            assert torch.equal(got[i].cpu()[none], y0[i][none]), what + ": rows without an adapter changed"
    # bit-identical to two launches wherever the library kept the requested split (a multi-target call may cut
    # ksplit so that ksplit * targets <= 16; then the summation order differs and only the tolerance holds)
    if one.ksplit * n_targets <= 16:
        want = [y.to(dev) for y in y0]
        if n_targets == 1:
            two.apply(want[0], xd, pd.key_buffer, pd.value_buffer, *idx, slots[0], pd.a_scaling)
        else:
            two.apply_multi(want, xd, pd.key_buffer, pd.value_buffer, *idx, slots, pd.a_scaling)
        for i in range(n_targets):
            assert torch.equal(got[i], want[i]), what + f": target {i} differs from the two-launch op"


@pytest.mark.parametrize("ks", [4, 5])
def test_items_the_device_cannot_hold_from_the_start(dev, ks):
    """64 tiles of one token each at 4096 -> 4096: with 5 K chunks the grid is larger than what the device
    holds at once, so the last tiles' expand items start late by construction; with 4 it just fits.  Either way
    the result is the two-launch op's."""
    dtype = torch.float16
    g = torch.Generator().manual_seed(77)
    A, T, h = 64, 64, 4096
    pool = W.make_pool([16] * A, h, h, dtype, g, True, std=0.05)
    ids = torch.randperm(A, generator=g)
    x = torch.randn(T, h, generator=g).to(dtype)
    y0 = torch.randn(T, h, generator=g).to(dtype)
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    one = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, 16, hidden=h, one_launch=True, ksplit=ks)
    two = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, 16, hidden=h, one_launch=False, bm_shrink=16, bm_expand=16,
                   ksplit=ks, reduce_in_expand=True)
    for rep in range(3):
        a, b = y0.to(dev), y0.to(dev)
        one.apply(a, x.to(dev), pd.key_buffer, pd.value_buffer, *idx, 1, pd.a_scaling)
        two.apply(b, x.to(dev), pd.key_buffer, pd.value_buffer, *idx, 1, pd.a_scaling)
        assert torch.equal(a, b), f"rep {rep}"
    ref = O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 1,
                    pool.a_scaling)
    assert_parity(a.cpu(), ref, "late items")


@pytest.mark.parametrize("n_tiles", [64, 65, 66, 76])
def test_batches_at_the_edge_of_what_the_device_holds(dev, n_tiles):
    """The benchmark's decode shape (256 tokens, 64 rank-16 adapters, 4096 -> 4096, 4 K chunks) with adapter counts
    made so that the batch has exactly `n_tiles` tiles of up to 16 tokens: 64 fill the device, 65 and 66 are what
    a Zipf(0.6) draw gives now and then, 76 is the most this shape can have.  The tiles beyond the device's
    capacity start late and use the hand-off like the others; layer after layer on one plan, results equal the
    two-launch op's bit for bit."""
    dtype = torch.float16
    A, T, h = 64, 256, 4096
    extra = n_tiles - 64                      # adapters that own 17 tokens: two tiles each
    cnt = [17] * extra + [1] * (A - extra)
    spare = T - sum(cnt)
    k = extra
    while spare > 0:                          # hand the rest out without crossing another multiple of 16
        add = min(spare, 15)
        cnt[k] += add
        spare -= add
        k += 1
    assert sum(cnt) == T and sum((c + 15) // 16 for c in cnt) == n_tiles
    g = torch.Generator().manual_seed(900 + n_tiles)
    ids = torch.repeat_interleave(torch.arange(A), torch.tensor(cnt))[torch.randperm(T, generator=g)]
    pool = W.make_pool([16] * A, h, h, dtype, g, True, std=0.05)
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    one = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, 16, hidden=h, one_launch=True, ksplit=4)
    two = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, 16, hidden=h, one_launch=False, bm_shrink=16, bm_expand=16,
                   ksplit=4, reduce_in_expand=True)
    assert one.header()["n_tiles_expand"] == n_tiles
    gd = torch.Generator(device=dev).manual_seed(n_tiles)
    xs = [torch.randn(T, h, generator=gd, device=dev).to(dtype) for _ in range(6)]
    y0 = [torch.randn(T, h, generator=gd, device=dev).to(dtype) for _ in range(6)]
    for rep in range(2):
        got, want = [y.clone() for y in y0], [y.clone() for y in y0]
        for l in range(6):
            one.apply(got[l], xs[l], pd.key_buffer, pd.value_buffer, *idx, l % 4, pd.a_scaling)
            two.apply(want[l], xs[l], pd.key_buffer, pd.value_buffer, *idx, l % 4, pd.a_scaling)
        torch.cuda.synchronize()
        for l in range(6):
            assert torch.equal(got[l], want[l]), f"{n_tiles} tiles, repetition {rep}, layer {l}"
    ref = O.lora_op(y0[0].cpu(), xs[0].cpu(), pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc,
                    ids, 0, pool.a_scaling)
    assert_parity(got[0].cpu(), ref, f"{n_tiles} tiles vs oracle")


def test_a_batch_several_times_the_device_runs_as_one_launch(dev):
    """A mixed batch whose one-launch grid is many times what the device holds (and three targets on top): the
    items run as a pipeline of shrink items followed by expand items, all through the hand-off; same bits as
    two launches."""
    w = W.config3(hidden=512, mlp=1024, len_div=2, n_decode=64, targets=("q", "k", "v"))
    wd = w.to(dev)
    t = wd.target("q"); p = t.pool
    R = max(p.ranks)
    one, two = _pair(wd, "q", R, 512, 4)
    a, b = wd.y0["q"].clone(), wd.y0["q"].clone()
    one.apply(a, wd.x[512], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)
    two.apply(b, wd.x[512], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)
    assert torch.equal(a, b)
    for rep in range(2):
        ya = [wd.y0[n].clone() for n in ("q", "k", "v")]
        yb = [wd.y0[n].clone() for n in ("q", "k", "v")]
        for plan, ys in ((one, ya), (two, yb)):
            plan.apply_multi(ys, wd.x[512], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, [0, 1, 2], p.a_scaling)
        for u, v in zip(ya, yb):
            assert torch.equal(u, v), f"three targets, repetition {rep}"


def test_one_launch_op_and_in_launch_split_k_sum_share_a_plan(dev):
    """Through the C ABI nothing stops a caller from running the one-launch op and a stand-alone split-K shrink
    (which sums its chunks inside the launch) on the same plan, in any order: their hand-off words are separate."""
    from oracle import lora_oracle as O
    from tests._util import assert_parity
    from valora_amd import _lib
    from valora_amd.plan import LoraPlan
    L = _lib.lib()
    w = W.config2(hidden=1024, n_tokens=96, n_adapters=24)
    wd = w.to(dev)
    t = wd.target("q"); p = t.pool
    pc = w.target("q").pool
    R = max(p.ranks)
    plan = LoraPlan(wd.ids, p.a_start, p.a_len, R, hidden=t.h_in, one_launch=True, ksplit=4)
    pa = _lib.make_pool(p.key_buffer, p.a_start, p.a_len, p.a_loc, t.h_in, 4)
    code = _lib.dtype_code(w.dtype)
    want_y = O.lora_op(w.y0["q"], w.x[t.h_in], pc.key_buffer, pc.value_buffer, pc.a_start, pc.a_len, pc.a_loc, w.ids, t.slot,
                       pc.a_scaling)
    want_d = O.bgmv_shrink(torch.zeros(w.T, R, dtype=w.dtype), w.x[t.h_in], pc.key_buffer, pc.a_start, pc.a_len, pc.a_loc,
                           w.ids, t.slot)
    first = None
    for rep in range(3):
        y = wd.y0["q"].clone()
        plan.apply(y, wd.x[t.h_in], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)
        delta = torch.zeros(w.T, R, dtype=w.dtype, device=dev)
        _lib.check(L.mlora_shrink(_lib.current_stream(dev), plan.handle, _lib.ptr(plan.scratch), plan.scratch.numel(),
                                  _lib.ptr(wd.x[t.h_in]), w.T, t.h_in, R, pa, t.slot, 4, _lib.ptr(delta), R, 0, 0, 0, code))
        torch.cuda.synchronize()
        assert_parity(y.cpu(), want_y, f"one-launch op, round {rep}")
        assert_parity(delta.cpu(), want_d, f"split-K shrink on the same plan, round {rep}")
        if first is None:
            first = (y.clone(), delta.clone())
        assert torch.equal(y, first[0]) and torch.equal(delta, first[1])


def test_two_streams_with_a_plan_each_run_side_by_side(dev):
    """Two layer loops on two streams, each with its own plan, scratch and outputs, overlap on the device: neither
    grid has the device to itself, so items start late and waits run out -- every wait is bounded and the give-up
    path gives the same bits, so both loops finish and equal their serial two-launch results."""
    L = 12
    sides = []
    for k, (n_tokens, n_adapters) in enumerate(((256, 64), (200, 48))):
        w = W.config2(hidden=2048, n_tokens=n_tokens, n_adapters=n_adapters)
        wd = w.to(dev)
        p = wd.target("q").pool
        one, two = _pair(wd, "q", max(p.ranks), 2048, 4)
        g = torch.Generator(device=dev).manual_seed(40 + k)
        xs = [torch.randn(w.T, 2048, generator=g, device=dev).to(w.dtype) for _ in range(L)]
        y0 = [torch.randn(w.T, 2048, generator=g, device=dev).to(w.dtype) for _ in range(L)]
        want = [y.clone() for y in y0]
        for l in range(L):
            two.apply(want[l], xs[l], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, l % 4, p.a_scaling)
        sides.append((one, p, xs, y0, want, torch.cuda.Stream(device=dev)))
    torch.cuda.synchronize()
    for rep in range(3):
        outs = [[y.clone() for y in side[3]] for side in sides]
        torch.cuda.synchronize()
        for l in range(L):                      # enqueue alternately so that the two streams' launches overlap
            for (one, p, xs, _, _, s), out in zip(sides, outs):
                with torch.cuda.stream(s):
                    one.apply(out[l], xs[l], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, l % 4, p.a_scaling)
        torch.cuda.synchronize()
        for k, (side, out) in enumerate(zip(sides, outs)):
            for l in range(L):
                assert torch.equal(out[l], side[4][l]), f"repetition {rep}, stream {k}, layer {l}"


def test_a_wait_that_runs_out(dev):
    """Every expand item looks for a stamp nobody leaves (a flag from the host), waits out its bound and then computes
    its tile's partials itself: the whole way out of the bounded wait, on a healthy device, with every kernel ending
    normally.  Same bits as two launches; the op takes the bound (30 us) plus the recomputation, not more."""
    w = W.config2(hidden=1024, n_tokens=64, n_adapters=16)
    wd = w.to(dev)
    t = wd.target("q"); p = t.pool
    R = max(p.ranks)
    slow = LoraPlan(wd.ids, p.a_start, p.a_len, R, hidden=1024, one_launch=True, ksplit=4, one_launch_never_ready=True)
    one, two = _pair(wd, "q", R, 1024, 4)
    outs = []
    for plan in (slow, one, two):
        y = wd.y0["q"].clone()
        plan.apply(y, wd.x[1024], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)
        outs.append(y)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[2]) and torch.equal(outs[1], outs[2])

    def timed(plan, reps=20):
        y = wd.y0["q"].clone()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            plan.apply(y, wd.x[1024], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    us_slow, us_fast = timed(slow), timed(one)
    print(f"one-launch op: {us_fast:.1f} us; with every wait running out: {us_slow:.1f} us", flush=True)
    assert us_slow > 30.0, "the waits must really have run to their bound"
    assert us_slow < 150.0, "and not past it: 30 us of waiting, then the tile's partials computed in place"


def test_operands_the_one_launch_kernel_cannot_take_run_as_two_launches(dev):
    """The one-launch kernel reads element 0 of the index and of every target's pool where it has nothing to fetch,
    and hands partials over in cache lines of the scratch buffer: an empty index, a target pool of zero rows or a
    scratch buffer that is only 16-byte aligned make the library run the call as two launches (whose loads are
    guarded).  No fault, the documented result: rows whose weights cannot be found keep their values."""
    from valora_amd import _lib
    L = _lib.lib()
    w = W.config2(hidden=512, n_tokens=48, n_adapters=12)
    wd = w.to(dev)
    t = wd.target("q"); p = t.pool
    R = max(p.ranks)
    plan = LoraPlan(wd.ids, p.a_start, p.a_len, R, hidden=512, one_launch=True, ksplit=4)
    code = _lib.dtype_code(w.dtype)
    st = _lib.current_stream(dev)
    x, y0 = wd.x[512], wd.y0["q"]
    want = y0.clone()
    plan.apply(want, x, p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)

    def call(pa, tg, scratch_ptr, scratch_bytes):
        y = y0.clone()
        tgs = (_lib.Target * 1)(_lib.Target(_lib.ptr(y), tg[0], tg[1], t.slot))
        _lib.check(L.mlora_lora_apply_multi(st, plan.handle, scratch_ptr, scratch_bytes, _lib.ptr(x), w.T, 512, 512, R, pa, 1,
                                            tgs, _lib.ptr(p.a_scaling), plan.ksplit, plan.flags, code))
        torch.cuda.synchronize()
        return y

    pa = _lib.make_pool(p.key_buffer, p.a_start, p.a_len, p.a_loc, 512, 4)
    full = (_lib.ptr(p.value_buffer), p.value_buffer.numel() // 512)
    sp, sb = _lib.ptr(plan.scratch), plan.scratch.numel()
    assert torch.equal(call(pa, full, sp, sb), want)
    # scratch that starts 16 bytes into a line
    off = _lib.c_void_p(plan.scratch.data_ptr() + 16)
    assert torch.equal(call(pa, full, off, sb - 16), want), "a 16-byte aligned scratch buffer gives the same bits"
    # a B pool of zero rows: nothing can be found, y keeps its values
    assert torch.equal(call(pa, (_lib.ptr(p.value_buffer), 0), sp, sb), y0)
    # an empty index: no adapter has rows
    empty = torch.empty(0, dtype=torch.long, device=dev)
    pe = _lib.make_pool(p.key_buffer, p.a_start, p.a_len, empty, 512, 4)
    assert torch.equal(call(pe, full, sp, sb), y0)
