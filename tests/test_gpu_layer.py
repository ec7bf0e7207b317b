"""A decoder layer with LoRA on all seven projections: the planned LoRA calls wired into a forward
pass (stock PyTorch base ops) against an fp32 CPU evaluation of the same layer with every token's
own dense weights W + scale * A @ B."""
import pytest
import torch
import torch.nn.functional as F

from valora_amd import workloads as W
from valora_amd.layer import LayerPlans, LayerPools, LayerWeights, layer_forward, rmsnorm, rope, segment_attention

pytestmark = pytest.mark.gpu

NAMES = ("q", "k", "v", "o", "gate", "up", "down")


def reference_layer(x, w, wl, seq_lens, heads, cos, sin, with_lora=True):
    """fp32 on the CPU; tokens are processed per adapter with dense effective weights."""
    x = x.float()
    ids = wl.ids

    def proj(inp, base, name):
        out = inp @ base.float()
        if with_lora:
            t = wl.target(name)
            for a in sorted(set(ids.tolist())):
                if a < 0:
                    continue
                A, B = t.pool.dense(a, t.slot)
                rows = (ids == a).nonzero().flatten()
                out[rows] += float(t.pool.a_scaling[a]) * (inp[rows] @ A.float()) @ B.float()
        return out

    h = rmsnorm(x, w.ln1.float())
    q, k, v = proj(h, w.wq, "q"), proj(h, w.wk, "k"), proj(h, w.wv, "v")
    q, k = rope(q, cos.float(), sin.float(), heads), rope(k, cos.float(), sin.float(), heads)
    a = segment_attention(seq_lens, heads)(q, k, v)
    x = x + proj(a, w.wo, "o")
    h2 = rmsnorm(x, w.ln2.float())
    m = F.silu(proj(h2, w.w_gate, "gate")) * proj(h2, w.w_up, "up")
    return x + proj(m, w.w_down, "down")


@pytest.mark.parametrize("n,kw,shape", [
    (3, dict(hidden=256, mlp=704, len_div=8, n_decode=40), (256, 704, 8)),
    (5, dict(hidden=256, mlp=704, len_div=8, n_decode=48, n_adapters=20), (256, 704, 8)),
    # configuration 5 at its full size: 7B shape, 1152 tokens, 64 resident adapters of ranks 16-64
    (5, dict(), (4096, 11008, 32)),
], ids=["config3-small", "config5-small", "config5-full"])
def test_layer_forward_with_lora_on_seven_projections(dev, n, kw, shape):
    wl = W.CONFIGS[n](targets=NAMES, **kw)
    (H, MLP, heads), dt = shape, wl.dtype
    g = torch.Generator().manual_seed(100 + n)
    # LoRA weights large enough that dropping them is far outside the tolerance
    for name in ("q", "gate", "down"):
        p = wl.target(name).pool
        p.key_buffer.mul_(3.0)
        p.value_buffer.mul_(3.0)
    mk = lambda i, o: (torch.randn(i, o, generator=g) / i ** 0.5).to(dt)
    w = LayerWeights(mk(H, H), mk(H, H), mk(H, H), mk(H, H), mk(H, MLP), mk(H, MLP), mk(MLP, H),
                     (1 + 0.1 * torch.randn(H, generator=g)).to(dt), (1 + 0.1 * torch.randn(H, generator=g)).to(dt))
    T = wl.T
    x = torch.randn(T, H, generator=g).to(dt)
    d = H // heads
    pos = torch.cat([torch.arange(int(s)) for s in wl.b_seq_len.tolist()]).float()
    freq = 1.0 / (10000 ** (torch.arange(0, d, 2).float() / d))
    ang = torch.cat((pos[:, None] * freq[None], pos[:, None] * freq[None]), dim=-1)
    cos, sin = ang.cos().to(dt), ang.sin().to(dt)
    seq = wl.b_seq_len.tolist()

    want = reference_layer(x, w, wl, seq, heads, cos, sin)
    base = reference_layer(x, w, wl, seq, heads, cos, sin, with_lora=False)

    wd = wl.to(dev)
    pa, pu, pd_ = wd.target("q").pool, wd.target("gate").pool, wd.target("down").pool
    pools = LayerPools((pa.key_buffer, pa.value_buffer), (pu.key_buffer, pu.value_buffer),
                       (pd_.key_buffer, pd_.value_buffer), pa.a_start, pa.a_len, pa.a_loc, pa.a_scaling)
    plans = LayerPlans(wd.ids, pa.a_start, pa.a_len, max(pa.ranks), H, MLP)
    wdev = LayerWeights(*[getattr(w, f).to(dev) for f in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down", "ln1", "ln2")])
    got = layer_forward(x.to(dev), wdev, pools, plans, segment_attention(seq, heads), heads, cos.to(dev), sin.to(dev))
    got_base = layer_forward(x.to(dev), wdev, None, None, segment_attention(seq, heads), heads, cos.to(dev), sin.to(dev))

    rel = lambda a, b: float((a.float().cpu() - b).norm() / b.norm())
    tol = 2e-2      # bf16 activations through nine matrix products and two normalisations
    assert rel(got, want) <= tol, rel(got, want)
    assert rel(got_base, base) <= tol
    assert rel(got_base, want) >= 5 * tol, "the LoRA contribution must be visible in this test"
