"""The op calls only launch kernels on the caller's stream, so a layer loop can be captured in a HIP
graph (the benchmark does).  A captured graph is replayed several times with eager work and
synchronisations in between, and every replay is checked against the eager result."""
import pytest
import torch

from valora_amd import workloads as W
from valora_amd.plan import LoraPlan

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,kw,names", [
    (2, dict(hidden=512, n_tokens=96, n_adapters=24), ("q",)),
    (3, dict(hidden=256, mlp=704, len_div=8, n_decode=40), ("q", "k", "v")),
    (4, dict(hidden=256, mlp=704, len_div=4, n_req=6), ("gate", "up")),
])
def test_graph_replays_match_eager(dev, n, kw, names):
    w = W.CONFIGS[n](**kw) if n == 2 else W.CONFIGS[n](targets=names, **kw)
    wd = w.to(dev)
    ts = [wd.target(x) for x in names]
    p = ts[0].pool
    R = max(p.ranks)
    plan = LoraPlan(wd.ids, p.a_start, p.a_len, R, hidden=ts[0].h_in)
    x = wd.x[ts[0].h_in]
    y0 = [wd.y0[nm].clone() for nm in names]
    ys = [t.clone() for t in y0]
    slots = [t.slot for t in ts]

    def op():
        if len(names) == 1:
            plan.apply(ys[0], x, p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, slots[0], p.a_scaling)
        else:
            plan.apply_multi(ys, x, p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, slots, p.a_scaling)

    def reset():
        for t, t0 in zip(ys, y0):
            t.copy_(t0)

    op()
    torch.cuda.synchronize()
    eager = [t.clone() for t in ys]

    s = torch.cuda.Stream(device=dev)
    s.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(s):
        reset()
        op()                                  # warm-up on the capture stream
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        reset()
        with torch.cuda.graph(graph, stream=s):
            op()
    torch.cuda.current_stream(dev).wait_stream(s)
    for i in range(4):
        reset()
        junk = torch.randn(1 << 20, device=dev).sum()     # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(ys, eager):
            assert torch.equal(got, want), f"replay {i}"
        assert torch.isfinite(junk)


def test_entry_points_under_capture_and_rebuild(dev):
    """The reference's entry points inside a HIP graph, the way a serving loop captures a step: the first call of
    a new batch happens DURING the capture, so the plan's build is only recorded.  Such a plan serves that capture
    alone: an eager call with the same tensors before the first replay must not find it (its tiles were never
    cut), and the replays must keep working afterwards.  A step graph that refills its ids tensor with `copy_`
    rebuilds the plan inside the graph on every replay (the version counter moved, and the build is a graph node)."""
    from oracle import lora_oracle as O
    from tests._util import assert_parity
    from valora_amd import _plan_cache
    from valora_amd.kernels import dispatch_bgmv
    dtype = torch.float16
    g = torch.Generator().manual_seed(77)
    T, H, R = 200, 1024, 16
    pool = W.make_pool([16, 8, 16, 16, 8], H, H, dtype, g, True, std=0.05)
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    ids_a = torch.randint(0, 5, (T,), generator=g)
    ids_b = torch.randint(0, 5, (T,), generator=g)
    x = torch.randn(T, H, generator=g).to(dtype)
    y0 = torch.randn(T, H, generator=g).to(dtype)
    xd, ids_d = x.to(dev), ids_a.to(dev)
    y_graph, y_eager = y0.to(dev), y0.to(dev)
    delta = torch.zeros(T, R, dtype=dtype, device=dev)
    delta2 = torch.zeros(T, R, dtype=dtype, device=dev)

    def want(ids):
        return O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 2,
                         pool.a_scaling)

    def pair(y, d):
        dispatch_bgmv(d, xd, pd.key_buffer, *idx, ids_d, 2, pd.a_scaling)
        dispatch_bgmv(y, d, pd.value_buffer, *idx, ids_d, 2, pd.a_scaling)

    _plan_cache.clear()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        m0 = _plan_cache.misses
        with torch.cuda.graph(graph, stream=s):
            pair(y_graph, delta)                     # first sight of this batch: the plan build is a graph node
        assert _plan_cache.misses - m0 == 1
        # eager, same tensors, before any replay: needs a plan of its own
        pair(y_eager, delta2)
        torch.cuda.synchronize()
        assert _plan_cache.misses - m0 == 2, "a plan recorded into a capture must not serve eager calls"
        assert_parity(y_eager.cpu(), want(ids_a), "eager call after a capture")
        for rep in range(3):
            y_graph.copy_(y0)
            graph.replay()
            torch.cuda.synchronize()
            assert_parity(y_graph.cpu(), want(ids_a), f"replay {rep}")
            assert torch.equal(y_graph, y_eager)
        # the next batch of the same size: refill the ids tensor the graph reads; the replay cuts the tiles again
        ids_d.copy_(ids_b.to(dev))
        y_graph.copy_(y0)
        graph.replay()
        torch.cuda.synchronize()
        assert_parity(y_graph.cpu(), want(ids_b), "replay after the ids were refilled")
    torch.cuda.current_stream().wait_stream(s)


def test_warm_up_then_capture_then_refill(dev):
    """torch's own recipe for graphs: warm up EAGERLY on the static tensors, capture, then `ids.copy_(new batch)` and
    replay.  The eager warm-up leaves a plan in the cache under the very key the captured calls use; the capture
    must not reuse it (the graph would then hold no build of its own and keep applying the warm-up batch's
    adapters), but record a build that every replay runs on whatever the ids tensor holds by then.  The plan and
    workspace the graph uses must also outlive the cache's own turnover: more than `cache_max_entries` other
    batches go through the entry points between replays."""
    from oracle import lora_oracle as O
    from tests._util import assert_parity
    from valora_amd import _plan_cache
    from valora_amd.kernels import dispatch_bgmv
    dtype = torch.float16
    g = torch.Generator().manual_seed(78)
    T, H, R = 160, 1024, 16
    pool = W.make_pool([16, 8, 16, 8, 16, 16], H, H, dtype, g, True, std=0.05)
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    batches = [torch.randint(0, 6, (T,), generator=g) for _ in range(3)]
    x = torch.randn(T, H, generator=g).to(dtype)
    y0 = torch.randn(T, H, generator=g).to(dtype)
    xd, ids_d = x.to(dev), batches[0].to(dev)
    y = y0.to(dev)
    delta = torch.zeros(T, R, dtype=dtype, device=dev)

    def want(ids):
        return O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 1,
                         pool.a_scaling)

    def pair():
        dispatch_bgmv(delta, xd, pd.key_buffer, *idx, ids_d, 1, pd.a_scaling)
        dispatch_bgmv(y, delta, pd.value_buffer, *idx, ids_d, 1, pd.a_scaling)

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(3):                     # eager warm-up on the static tensors: leaves an eager plan in the cache
            y.copy_(y0)
            pair()
        torch.cuda.synchronize()
        assert_parity(y.cpu(), want(batches[0]), "eager warm-up")
        graph = torch.cuda.CUDAGraph()
        m0 = _plan_cache.misses
        with torch.cuda.graph(graph, stream=s):
            pair()
        assert _plan_cache.misses - m0 == 1, "the capture must record a plan build of its own"
        for rep, ids in enumerate((batches[1], batches[2], batches[0])):
            ids_d.copy_(ids.to(dev))
            y.copy_(y0)
            graph.replay()
            torch.cuda.synchronize()
            assert_parity(y.cpu(), want(ids), f"replay {rep} after the ids were refilled")
        # turn the cache over with other batches (each a new ids tensor: a new key), then replay again
        others = []
        for k in range(_plan_cache.max_entries() + 3):
            ids_k = torch.randint(0, 6, (T,), generator=g).to(dev)
            yk, dk = y0.to(dev), torch.zeros(T, R, dtype=dtype, device=dev)
            dispatch_bgmv(dk, xd, pd.key_buffer, *idx, ids_k, 1, pd.a_scaling)
            dispatch_bgmv(yk, dk, pd.value_buffer, *idx, ids_k, 1, pd.a_scaling)
            others.append((ids_k, yk, dk))
        junk = [torch.randn(1 << 18, device=dev) for _ in range(8)]      # eager allocations that could land on freed memory
        torch.cuda.synchronize()
        ids_d.copy_(batches[1].to(dev))
        y.copy_(y0)
        graph.replay()
        torch.cuda.synchronize()
        assert_parity(y.cpu(), want(batches[1]), "replay after the cache turned over")
        assert all(torch.isfinite(j).all() for j in junk)
    torch.cuda.current_stream().wait_stream(s)
