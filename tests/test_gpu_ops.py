"""GPU parity of the op entry points against the CPU oracle, always through the C ABI.

Tolerance (stated by the benchmark definition): max-abs error <= 2e-2 and relative L2 error
<= 1e-3 against the reference semantics with fp32 accumulation."""
import pytest
import torch

from oracle import lora_oracle as O
from valora_amd import workloads as W
from tests._util import assert_parity

pytestmark = pytest.mark.gpu


def _case(seed, T, h_in, h_out, ranks, dtype, paged=True, id_style="random", scal=None):
    g = torch.Generator().manual_seed(seed)
    heads = 32 if h_in % 32 == 0 and h_out % 32 == 0 else 8
    pool = W.make_pool(list(ranks), h_in, h_out, dtype, g, paged, std=0.05, scalings=scal, heads=heads)
    A = len(ranks)
    if id_style == "random":
        ids = torch.randint(0, A, (T,), generator=g)
    elif id_style == "runs":
        ids = torch.repeat_interleave(torch.randint(0, A, (T,), generator=g),
                                      torch.randint(1, 70, (T,), generator=g))[:T]
    else:
        ids = torch.randint(-1, A + 1, (T,), generator=g)
    x = torch.randn(T, h_in, generator=g).to(dtype)
    y0 = torch.randn(T, h_out, generator=g).to(dtype)
    R = max(ranks)
    v = torch.randn(T, R, generator=g).to(dtype)
    return pool, ids, x, y0, v, R


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,h,ranks,ids_style", [
    (128, 1024, (8, 16), "runs"),            # the reference's own test shape
    (1, 4096, (16,), "random"),
    (37, 4096, (8, 16, 32, 64), "random"),
    (300, 3328, (16, 32, 64), "random"),     # hidden size of the reference's op bench
    (77, 1000, (16, 8, 24), "random"),       # h % r != 0: rank groups straddle pool rows
    (50, 11008, (64, 8), "runs"),
    (200, 768, (128, 64, 8), "random"),      # rank 128
    (90, 2048, (8, 16, 32), "holes"),        # ids outside [0, A): rows must stay untouched
    (256, 4096, (16,) * 200, "random"),      # more adapters than the tile table has a bucket for
    (3000, 1024, (64,), "random"),           # one adapter for the whole batch
])
def test_dispatch_bgmv_shrink_and_expand(dev, dtype, T, h, ranks, ids_style):
    from valora_amd.kernels import dispatch_bgmv
    pool, ids, x, y0, v, R = _case(T + h, T, h, h, ranks, dtype, True, ids_style,
                                   [0.5 + 0.25 * i for i in range(len(ranks))])
    pd = pool.to(dev)
    for slot in (0, 3):
        # shrink into a buffer pre-filled with a sentinel: columns >= r and skipped rows keep it
        delta0 = torch.full((T, R), 3.0, dtype=dtype)
        delta = delta0.to(dev)
        dispatch_bgmv(delta, x.to(dev), pd.key_buffer, pd.a_start, pd.a_len, pd.a_loc, ids.to(dev), slot, pd.a_scaling)
        want = O.bgmv_shrink(delta0, x, pool.key_buffer, pool.a_start, pool.a_len, pool.a_loc,
                             torch.where((ids >= 0) & (ids < len(ranks)), ids, torch.full_like(ids, -1)), slot)
        assert_parity(delta.cpu(), want, f"shrink slot {slot}")
        untouched = want == 3.0
        assert torch.equal(delta.cpu()[untouched], want[untouched])
        y = y0.to(dev)
        dispatch_bgmv(y, v.to(dev), pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, ids.to(dev), slot, pd.a_scaling)
        want = O.bgmv_expand(y0, v, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc,
                             torch.where((ids >= 0) & (ids < len(ranks)), ids, torch.full_like(ids, -1)), slot,
                             pool.a_scaling)
        assert_parity(y.cpu(), want, f"expand slot {slot}")
        skipped = ~((ids >= 0) & (ids < len(ranks)))
        assert torch.equal(y.cpu()[skipped], y0[skipped])


def test_reference_scratch_narrower_than_rank(dev):
    """An adapter whose rank exceeds the scratch width only contributes its first columns
    (grid.x = feat_out in the shrink, tx = feat_in / 8 lanes in the expand)."""
    from valora_amd.kernels import dispatch_bgmv
    dtype = torch.float16
    pool, ids, x, y0, v, R = _case(5, 40, 512, 512, (8, 32), dtype)
    pd = pool.to(dev)
    delta0 = torch.full((40, 8), 2.0, dtype=dtype)
    delta = delta0.to(dev)
    dispatch_bgmv(delta, x.to(dev), pd.key_buffer, pd.a_start, pd.a_len, pd.a_loc, ids.to(dev), 1, pd.a_scaling)
    full = O.bgmv_shrink(torch.zeros(40, 32, dtype=dtype), x, pool.key_buffer, pool.a_start, pool.a_len,
                         pool.a_loc, ids, 1)
    assert_parity(delta.cpu(), full[:, :8], "narrow shrink")


def test_views_and_pool_aliasing(dev):
    """Row-sliced views (q[delora_tk_index:]) and y living in the same allocation as the pool
    (decode writes k/v rows of the KV pool that also holds the adapters)."""
    from valora_amd.kernels import dispatch_bgmv
    dtype = torch.float16
    pool, ids, x, y0, v, R = _case(9, 64, 1024, 1024, (16, 8), dtype)
    pd = pool.to(dev)
    n = pool.n_rows
    big = torch.zeros(n + 64, 32, 32, dtype=dtype, device=dev)     # pool rows then 64 "KV" rows
    big[:n] = pd.value_buffer
    big[n:] = y0.to(dev).view(64, 32, 32)
    yview = big[n:].view(64, 1024)[8:]                              # skip 8 rows, still contiguous
    dispatch_bgmv(yview, v.to(dev)[8:], big, pd.a_start, pd.a_len, pd.a_loc, ids.to(dev)[8:], 2, pd.a_scaling)
    want = O.bgmv_expand(y0[8:], v[8:], pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids[8:], 2,
                         pool.a_scaling)
    assert_parity(yview.cpu(), want, "aliased expand")
    assert torch.equal(big[n:].view(64, 1024)[:8].cpu(), y0[:8])
    assert torch.equal(big[:n].cpu(), pool.value_buffer)


def test_error_behaviour(dev):
    from valora_amd.kernels import dispatch_bgmv
    dtype = torch.float16
    pool, ids, x, y0, v, R = _case(2, 16, 512, 512, (8,), dtype)
    pd = pool.to(dev)
    args = (pd.a_start, pd.a_len, pd.a_loc)
    d = torch.zeros(16, 8, dtype=dtype, device=dev)
    with pytest.raises(RuntimeError, match="CHECK_EQ\\(indicies.size\\(0\\), x.size\\(0\\)\\)"):
        dispatch_bgmv(d, x.to(dev), pd.key_buffer, *args, ids.to(dev)[:5], 0, pd.a_scaling)
    with pytest.raises(RuntimeError, match="x must be contiguous"):
        dispatch_bgmv(d, x.to(dev).t().contiguous().t(), pd.key_buffer, *args, ids.to(dev), 0, pd.a_scaling)
    with pytest.raises(RuntimeError, match="w must be a 3D tensor"):
        dispatch_bgmv(d, x.to(dev), pd.key_buffer.view(-1, 512), *args, ids.to(dev), 0, pd.a_scaling)
    with pytest.raises(RuntimeError, match="No suitable kernel"):
        dispatch_bgmv(d.float(), x.to(dev).float(), pd.key_buffer.float(), *args, ids.to(dev), 0, pd.a_scaling)
    with pytest.raises(RuntimeError, match="No suitable kernel. h_in=512 h_out=12"):
        dispatch_bgmv(torch.zeros(16, 12, dtype=dtype, device=dev), x.to(dev), pd.key_buffer, *args,
                      ids.to(dev), 0, pd.a_scaling)
    with pytest.raises(RuntimeError, match="expected scalar type Long"):
        dispatch_bgmv(d, x.to(dev), pd.key_buffer, *args, ids.to(dev).int(), 0, pd.a_scaling)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_sgmm_and_prefill_entry_points(dev, dtype):
    """ATMM-signature and Triton-signature entry points on a ragged batch: covered rows match the
    oracle, rows outside the given problems / beyond max_input_len are untouched."""
    from valora_amd.atmm_ops import dispatch_bgmv as dispatch_sgmm, shrink_accumulate
    from valora_amd.lora_prefill import lora_get_qkvo_fwd_expand, lora_get_qkvo_fwd_shrink
    g = torch.Generator().manual_seed(77)
    ranks = [8, 16, 32, 16]
    h = 512
    pool = W.make_pool(ranks, h, h, dtype, g, True, std=0.05, scalings=[1.0, 0.5, 2.0, 1.5])
    seq = torch.tensor([40, 3, 70, 1, 1, 33, 64], dtype=torch.int32)
    req = torch.tensor([2, 2, 0, 1, 1, 3, 0])
    start = (torch.cumsum(seq, 0) - seq).to(torch.int32)
    ids = torch.repeat_interleave(req, seq.long())
    T, R = int(ids.numel()), 32
    x = torch.randn(T, h, generator=g).to(dtype)
    y0 = torch.randn(T, h, generator=g).to(dtype)
    v = torch.randn(T, R, generator=g).to(dtype)
    pd = pool.to(dev)
    idx = (pool.a_start, pool.a_len, pool.a_loc)
    idxd = (pd.a_start, pd.a_len, pd.a_loc)
    # --- ATMM signature: only the first P problems
    oc, rc, li, st = O.count_consecutive_requests(pool.a_len, ids)
    for P in (len(oc), 3, 0):
        t = lambda l: torch.tensor(l + [1] * 4, dtype=torch.long, device=dev)
        tmp = torch.zeros(60 * 8, dtype=torch.int8, device=dev)
        d0 = torch.full((T, R), 1.5, dtype=dtype)
        d = d0.to(dev)
        dispatch_sgmm(d, x.to(dev), pd.key_buffer, *idxd, ids.to(dev), 1, pd.a_scaling, t(oc), t(rc), t(li), t(st),
                      tmp, P, 64, 32, 32, 32, 32, 32)
        want = O.sgmm_canonical(d0, x, pool.key_buffer, *idx, ids, 1, pool.a_scaling, oc, st, P)
        assert_parity(d.cpu(), want, f"sgmm shrink P={P}")
        y = y0.to(dev)
        dispatch_sgmm(y, v.to(dev), pd.value_buffer, *idxd, ids.to(dev), 1, pd.a_scaling, t(oc), t(rc), t(li), t(st),
                      tmp, P, 64, 64, 32, 64, 64, 32)
        want = O.sgmm_canonical(y0, v, pool.value_buffer, *idx, ids, 1, pool.a_scaling, oc, st, P)
        assert_parity(y.cpu(), want, f"sgmm expand P={P}")
        covered = sum(oc[:P])
        assert torch.equal(y.cpu()[covered:], y0[covered:])
    # beta = 1 on the shrink (ATMM's accumulate)
    shrink_accumulate(True)
    try:
        d0 = torch.randn(T, R, generator=g).to(dtype)
        d = d0.to(dev)
        dispatch_sgmm(d, x.to(dev), pd.key_buffer, *idxd, ids.to(dev), 0, pd.a_scaling, t(oc), t(rc), t(li), t(st),
                      tmp, len(oc), 64, 32, 32, 32, 32, 32)
        fresh = O.bgmv_shrink(torch.zeros(T, R, dtype=torch.float32), x.float(), pool.key_buffer.float(), *idx, ids, 0)
        want = (d0.float() + fresh).to(dtype)
        assert_parity(d.cpu(), want, "sgmm accumulate")
    finally:
        shrink_accumulate(False)
    # --- Triton signature; max_input_len = 40 leaves the tails of the 70- and 64-row requests alone
    for mx in (int(seq.max()), 40):
        o0 = torch.full((T, R), 2.5, dtype=dtype)
        o = o0.to(dev)
        lora_get_qkvo_fwd_shrink(x.to(dev), pd.key_buffer.view(-1, h), o, pd.a_loc, pd.a_start, pd.a_len,
                                 start.to(dev), seq.to(dev), req.to(dev), h, 2, R, mx)
        want = O.triton_shrink(x, pool.key_buffer.view(-1, h), o0, pool.a_loc, pool.a_start, pool.a_len, start, seq,
                               req, h, 2, R, mx)
        assert_parity(o.cpu(), want, f"prefill shrink mx={mx}")
        assert torch.equal(o.cpu() == 2.5, want == 2.5)
        y = y0.to(dev)
        lora_get_qkvo_fwd_expand(v.to(dev), pd.value_buffer.view(-1, h), y, pd.a_scaling, pd.a_loc, pd.a_start,
                                 pd.a_len, start.to(dev), seq.to(dev), req.to(dev), h, 2, R, mx)
        want = O.triton_expand(v, pool.value_buffer.view(-1, h), y0, pool.a_scaling, pool.a_loc, pool.a_start,
                               pool.a_len, start, seq, req, h, 2, R, mx)
        assert_parity(y.cpu(), want, f"prefill expand mx={mx}")


def test_edge_cases_empty_and_no_adapter(dev):
    """T = 0, a batch where no token has an adapter, one token, and pools with 1 or 2 slots."""
    from valora_amd.kernels import dispatch_bgmv
    from valora_amd.plan import LoraPlan
    dtype = torch.float16
    pool, ids, x, y0, v, R = _case(31, 20, 512, 512, (8, 16), dtype)
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    # T = 0: nothing happens, nothing is read
    e = torch.zeros(0, 512, dtype=dtype, device=dev)
    d = torch.zeros(0, 16, dtype=dtype, device=dev)
    dispatch_bgmv(d, e, pd.key_buffer, *idx, torch.zeros(0, dtype=torch.long, device=dev), 0, pd.a_scaling)
    dispatch_bgmv(e, d, pd.value_buffer, *idx, torch.zeros(0, dtype=torch.long, device=dev), 0, pd.a_scaling)
    plan = LoraPlan(torch.zeros(0, dtype=torch.long, device=dev), pd.a_start, pd.a_len, 16, hidden=512)
    plan.apply(e, e.clone(), pd.key_buffer, pd.value_buffer, *idx, 0, pd.a_scaling)
    assert plan.header()["n_active"] == 0
    # no token has an adapter: y comes back bit-identical
    none = torch.full((20,), -1, dtype=torch.long, device=dev)
    y = y0.to(dev)
    plan = LoraPlan(none, pd.a_start, pd.a_len, 16, hidden=512)
    plan.apply(y, x.to(dev), pd.key_buffer, pd.value_buffer, *idx, 1, pd.a_scaling)
    assert torch.equal(y.cpu(), y0)
    # one token
    y = y0[:1].to(dev)
    plan = LoraPlan(ids[:1].to(dev), pd.a_start, pd.a_len, 16, hidden=512)
    plan.apply(y, x[:1].to(dev), pd.key_buffer, pd.value_buffer, *idx, 2, pd.a_scaling)
    want = O.lora_op(y0[:1], x[:1], pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc,
                     ids[:1], 2, pool.a_scaling)
    assert_parity(y.cpu(), want, "one token")
    # pools with other slot counts (a_len = n_slots * r)
    for n_slots in (1, 2, 7):
        g = torch.Generator().manual_seed(n_slots)
        p2 = W.make_pool([8, 32, 16], 256, 384, dtype, g, True, n_slots=n_slots, std=0.05, heads=8)
        ids2 = torch.randint(0, 3, (50,), generator=g)
        x2 = torch.randn(50, 256, generator=g).to(dtype)
        y2 = torch.randn(50, 384, generator=g).to(dtype)
        p2d = p2.to(dev)
        slot = n_slots - 1
        plan = LoraPlan(ids2.to(dev), p2d.a_start, p2d.a_len, 32, n_slots=n_slots, hidden=256)
        yy = y2.to(dev)
        plan.apply(yy, x2.to(dev), p2d.key_buffer, p2d.value_buffer, p2d.a_start, p2d.a_len, p2d.a_loc, slot,
                   p2d.a_scaling)
        want = O.lora_op(y2, x2, p2.key_buffer, p2.value_buffer, p2.a_start, p2.a_len, p2.a_loc, ids2, slot,
                         p2.a_scaling, n_slots=n_slots)
        assert_parity(yy.cpu(), want, f"n_slots={n_slots}")
        yy = y2.to(dev)
        plan16 = LoraPlan(ids2.to(dev), p2d.a_start, p2d.a_len, 32, n_slots=n_slots, hidden=256, one_launch=True)
        plan16.apply(yy, x2.to(dev), p2d.key_buffer, p2d.value_buffer, p2d.a_start, p2d.a_len, p2d.a_loc, slot,
                     p2d.a_scaling)
        assert_parity(yy.cpu(), want, f"one launch n_slots={n_slots}")


def test_plan_reuse_across_drop_in_calls(dev):
    """The shims keep the plan of a batch while the caller keeps passing the same, unmodified tensors; a
    modified or a different ids tensor gets a plan of its own."""
    from valora_amd import _plan_cache
    from valora_amd.kernels import dispatch_bgmv
    w = W.config2(hidden=512, n_tokens=96, n_adapters=24)
    wd = w.to(dev)
    t = wd.target("q"); p = t.pool; pc = w.target("q").pool
    R = max(p.ranks)

    def run(ids_dev):
        y = wd.y0["q"].clone()
        delta = torch.zeros(wd.T, R, dtype=wd.dtype, device=dev)
        dispatch_bgmv(delta, wd.x[t.h_in], p.key_buffer, p.a_start, p.a_len, p.a_loc, ids_dev, t.slot, p.a_scaling)
        dispatch_bgmv(y, delta, p.value_buffer, p.a_start, p.a_len, p.a_loc, ids_dev, t.slot, p.a_scaling)
        return y.cpu()

    def want(ids_cpu):
        return O.lora_op(w.y0["q"], w.x[t.h_in], pc.key_buffer, pc.value_buffer, pc.a_start, pc.a_len, pc.a_loc,
                         ids_cpu, t.slot, pc.a_scaling)

    _plan_cache.clear()
    h0, m0 = _plan_cache.hits, _plan_cache.misses
    ids = wd.ids.clone()
    assert_parity(run(ids), want(w.ids), "first call")
    assert_parity(run(ids), want(w.ids), "second call")
    assert _plan_cache.misses - m0 == 1 and _plan_cache.hits - h0 == 3          # one build for four calls
    # modified in place: the version counter moves, the old plan must not be used
    ids2_cpu = (w.ids + 1) % 24
    ids.copy_(ids2_cpu)
    assert_parity(run(ids), want(ids2_cpu), "after an in-place change of the ids")
    assert _plan_cache.misses - m0 == 2
    # a different tensor object with other contents
    ids3_cpu = torch.flip(w.ids, dims=(0,)).contiguous()
    assert_parity(run(ids3_cpu.to(dev)), want(ids3_cpu), "new ids tensor")
    assert _plan_cache.misses - m0 == 3
    # switched off: same results, nothing cached
    _plan_cache.set_enabled(False)
    try:
        h1, m1 = _plan_cache.hits, _plan_cache.misses
        assert_parity(run(ids), want(ids2_cpu), "cache disabled")
        assert (_plan_cache.hits, _plan_cache.misses) == (h1, m1)
    finally:
        _plan_cache.set_enabled(True)


def test_one_call_entry_points_with_a_caller_held_plan(dev):
    """What a binding that keeps ONE plan per batch does: mlora_tile_lookup + mlora_build_plan once, then every
    dispatch_bgmv call of the layer with that plan -- no per-call sort, no workspace for the expand.  Same bits
    as the calls that build their own plan."""
    import ctypes
    from valora_amd import _lib
    L = _lib.lib()
    dtype = torch.bfloat16
    pool, ids, x, y0, v, R = _case(91, 300, 1024, 1024, (8, 16, 32, 16), dtype)
    pd = pool.to(dev)
    T, h = 300, 1024
    stream = _lib.current_stream(dev)
    ids_d, xd = ids.to(dev), x.to(dev)
    pk = _lib.make_pool(pd.key_buffer, pd.a_start, pd.a_len, pd.a_loc, h, 4)
    pv = _lib.make_pool(pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, h, 4)
    cfg = _lib.TileConfig()
    _lib.check(L.mlora_tile_lookup(T, R, h, 4, cfg))
    buf = torch.empty(int(L.mlora_plan_bytes(T, 4)), dtype=torch.uint8, device=dev)
    plan = _lib.Plan(_lib.ptr(buf), buf.numel())
    _lib.check(L.mlora_build_plan(stream, plan, _lib.ptr(ids_d), T, _lib.ptr(pd.a_start), _lib.ptr(pd.a_len), 4, 4,
                                  cfg.bm_shrink, cfg.bm_expand))
    assert (plan.T, plan.n_adapters, plan.n_slots) == (T, 4, 4)
    ws = torch.empty(int(L.mlora_workspace_bytes(T, 4, R)), dtype=torch.uint8, device=dev)
    code = _lib.dtype_code(dtype)
    out = {}
    for held in (True, False):
        delta = torch.full((T, R), 0.25, dtype=dtype, device=dev)
        y = y0.to(dev)
        p = plan if held else None
        _lib.check(L.mlora_dispatch_bgmv(stream, _lib.ptr(delta), _lib.ptr(xd), pk, None if held else _lib.ptr(ids_d), 2,
                                         _lib.ptr(pd.a_scaling), T, h, R, code, _lib.ptr(ws), ws.numel(), p))
        # the expand on a caller-held plan takes no workspace at all
        _lib.check(L.mlora_dispatch_bgmv(stream, _lib.ptr(y), _lib.ptr(delta), pv, None if held else _lib.ptr(ids_d), 2,
                                         _lib.ptr(pd.a_scaling), T, R, h, code, None if held else _lib.ptr(ws),
                                         0 if held else ws.numel(), p))
        torch.cuda.synchronize()
        out[held] = (delta.cpu(), y.cpu())
    assert torch.equal(out[True][0], out[False][0]) and torch.equal(out[True][1], out[False][1])
    want = O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 2,
                     pool.a_scaling)
    assert_parity(out[True][1], want, "caller-held plan")
    # a plan cut for another index is refused
    other = _lib.make_pool(pd.key_buffer, pd.a_start[:3], pd.a_len[:3], pd.a_loc, h, 4)
    rc = L.mlora_dispatch_bgmv(stream, _lib.ptr(y), _lib.ptr(xd), other, None, 2, _lib.ptr(pd.a_scaling), T, h, R, code,
                               _lib.ptr(ws), ws.numel(), plan)
    assert rc == -1 and b"plan was built for 4 adapters" in L.mlora_last_error()


def test_plan_cache_hits_for_the_reference_call_patterns(dev):
    """On the GPU, through the shims: the same tensors for all calls of a layer hit; fresh [1:] views of the
    segment tensors hit; tensors created under inference_mode hit; a new ids tensor misses."""
    from valora_amd import _plan_cache
    from valora_amd.atmm_ops import dispatch_bgmv as dispatch_sgmm
    from valora_amd.kernels import dispatch_bgmv
    dtype = torch.float16
    pool, ids, x, y0, v, R = _case(92, 120, 512, 512, (8, 16, 16), dtype)
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    ids_d, xd = ids.to(dev), x.to(dev)
    _plan_cache.clear()
    h0, m0 = _plan_cache.hits, _plan_cache.misses
    for layer in range(3):
        for slot in range(3):
            delta = torch.zeros(120, R, dtype=dtype, device=dev)
            y = y0.to(dev)
            dispatch_bgmv(delta, xd, pd.key_buffer, *idx, ids_d, slot, pd.a_scaling)
            dispatch_bgmv(y, delta, pd.value_buffer, *idx, ids_d, slot, pd.a_scaling)
    assert _plan_cache.misses - m0 == 1 and _plan_cache.hits - h0 == 17
    # fresh offset views of the segment tensors with every call
    oc, rc_, li, st = O.count_consecutive_requests(pool.a_len, ids)
    P = len(oc)
    t = lambda l: torch.tensor([9] + l + [1] * 4, dtype=torch.long, device=dev)
    oc_d, st_d, rc_d, li_d = t(oc), t(st), t(rc_), t(li)
    tmp = torch.zeros(60 * (P + 5), dtype=torch.int8, device=dev)
    m1 = _plan_cache.misses
    for _ in range(4):
        delta = torch.zeros(120, R, dtype=dtype, device=dev)
        dispatch_sgmm(delta, xd, pd.key_buffer, *idx, ids_d, 1, pd.a_scaling, oc_d[1:], rc_d[1:], li_d[1:], st_d[1:],
                      tmp, P, 64, 32, 32, 32, 32, 32)
    assert _plan_cache.misses - m1 == 1, "fresh views of the same segment tensors must reuse the plan"
    want = O.sgmm_canonical(torch.zeros(120, R, dtype=dtype), x, pool.key_buffer, pool.a_start, pool.a_len, pool.a_loc, ids,
                            1, pool.a_scaling, oc, st, P)
    assert_parity(delta.cpu(), want, "sgmm through fresh views")
    # inference tensors
    with torch.inference_mode():
        ids_i = ids.to(dev)
        m2 = _plan_cache.misses
        for _ in range(3):
            delta = torch.zeros(120, R, dtype=dtype, device=dev)
            dispatch_bgmv(delta, xd, pd.key_buffer, *idx, ids_i, 0, pd.a_scaling)
        assert _plan_cache.misses - m2 == 1
    # a new ids tensor with other contents
    m3 = _plan_cache.misses
    ids2 = torch.flip(ids, dims=(0,)).contiguous().to(dev)
    delta = torch.zeros(120, R, dtype=dtype, device=dev)
    dispatch_bgmv(delta, xd, pd.key_buffer, *idx, ids2, 0, pd.a_scaling)
    assert _plan_cache.misses - m3 == 1
    want = O.bgmv_shrink(torch.zeros(120, R, dtype=dtype), x, pool.key_buffer, pool.a_start, pool.a_len, pool.a_loc,
                         torch.flip(ids, dims=(0,)), 0)
    assert_parity(delta.cpu(), want, "new ids tensor")
