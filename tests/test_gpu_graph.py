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
