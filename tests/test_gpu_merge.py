"""GPU parity of merge / unmerge of an adapter into the base weights and of the deLoRA compensation
op against oracle/lora_oracle.py.  Small-integer weights make the comparison bit-exact; random
weights are compared to one unit in the last place of the result (the accumulation order inside a
GEMM is not part of the reference's contract)."""
import pytest
import torch

from oracle import lora_oracle as O
from valora_amd import workloads as W
from valora_amd.merge import DeLoraPlan, merge_adapter, unmerge_adapter
from tests._util import assert_parity
from tests.test_merge_oracle_pins import int_pool

pytestmark = pytest.mark.gpu


def ulp_of(t):
    a = t.float().abs().clamp_min(2.0 ** -14)
    mant = 10 if t.dtype == torch.float16 else 7
    return torch.exp2(torch.floor(torch.log2(a)) - mant)


def run_merge(dev, Ws, pool, adapter, scaling, slots, sign, max_rank=None, ld=None):
    H_in, H_out = Ws[0].shape
    if ld is None:
        Wd = [w.clone().to(dev) for w in Ws]
    else:    # weights that are column slices of a wider matrix
        big = [torch.zeros(H_in, ld, dtype=Ws[0].dtype, device=dev) for _ in Ws]
        for b, w in zip(big, Ws):
            b[:, :H_out] = w.to(dev)
        Wd = [b[:, :H_out] for b in big]
    p = pool.to(dev)
    fn = merge_adapter if sign > 0 else unmerge_adapter
    fn(Wd, p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, adapter, scaling,
       max_rank or max(pool.ranks), slots=slots, n_slots=pool.n_slots)
    return [w.cpu() for w in Wd]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,ranks", [(64, [8, 16, 8]), (256, [32, 64, 8, 16]), (1000, [128, 8]), (4096, [16, 64])])
def test_merge_integer_weights_bit_exact(dev, dtype, H, ranks):
    pool = int_pool(H, ranks, dtype, seed=H)
    g = torch.Generator().manual_seed(H + 1)
    for adapter in range(len(ranks)):
        Ws = [torch.randint(-8, 9, (H, H), generator=g).to(dtype) for _ in range(4)]
        for sign in (1, -1):
            want = O.merge_adapter(Ws, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc,
                                   adapter, 2.0, sign=sign)
            got = run_merge(dev, Ws, pool, adapter, 2.0, (0, 1, 2, 3), sign)
            for k in range(4):
                assert torch.equal(got[k], want[k]), f"adapter {adapter} slot {k} sign {sign}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_merge_random_weights_and_views(dev, dtype):
    g = torch.Generator().manual_seed(8)
    H = 512
    pool = W.make_pool([16, 64, 32], H, H, dtype, g, True, std=0.05, scalings=[2.0, 0.5, 1.0], heads=8)
    Ws = [(torch.randn(H, H, generator=g) * 0.05).to(dtype) for _ in range(3)]
    for adapter, scaling in ((0, 2.0), (1, 0.3), (2, 1.7)):
        want = O.merge_adapter(Ws, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, adapter,
                               scaling, slots=(3, 0, 1))
        for ld in (None, H + 64):
            got = run_merge(dev, Ws, pool, adapter, scaling, (3, 0, 1), 1, ld=ld)
            for k in range(3):
                d = (got[k].float() - want[k].float()).abs()
                # one ulp of the rounded GEMM result (|ab| <= |W| + |W'|) may move the sum by as much
                big = torch.maximum(want[k].float().abs(), Ws[k].float().abs()).to(dtype)
                assert (d <= 2 * ulp_of(big)).all(), f"adapter {adapter} slot {k}: more than one ulp of ab"
                assert (d > 0).float().mean() < 0.02
        # merge then unmerge: back to within one rounding of the start, like the reference
        m = run_merge(dev, Ws, pool, adapter, scaling, (3, 0, 1), 1)
        back = run_merge(dev, m, pool, adapter, scaling, (3, 0, 1), -1)
        for k in range(3):
            big = torch.maximum(m[k].float().abs(), Ws[k].float().abs()).to(dtype)
            assert ((back[k].float() - Ws[k].float()).abs() <= 2 * ulp_of(big)).all()


def test_merge_rejects_bad_arguments(dev):
    g = torch.Generator().manual_seed(9)
    pool = W.make_pool([8], 64, 64, torch.float16, g, True, heads=8).to(dev)
    w = torch.zeros(64, 64, dtype=torch.float16, device=dev)
    args = (pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc)
    with pytest.raises(RuntimeError, match="adapter"):
        merge_adapter([w], *args, 5, 1.0, 8, slots=(0,))
    with pytest.raises(RuntimeError, match="slot"):
        merge_adapter([w], *args, 0, 1.0, 8, slots=(4,))
    with pytest.raises(RuntimeError, match="one shape"):
        merge_adapter([w, w[:32]], *args, 0, 1.0, 8, slots=(0, 1))
    with pytest.raises(RuntimeError, match="max_rank"):
        merge_adapter([w], *args, 0, 1.0, 12, slots=(0,))


@pytest.mark.parametrize("n", [2, 3, 5])
def test_delora_compensation(dev, n):
    """The merged adapter lives in W; every other request is compensated.  Compared with the oracle and,
    end to end, with base + LoRA of the token's own adapter."""
    small = {2: dict(hidden=512, n_tokens=96, n_adapters=24), 3: dict(hidden=256, mlp=704, len_div=8, n_decode=40),
             5: dict(hidden=256, mlp=704, len_div=8, n_decode=48, n_adapters=20)}[n]
    w = W.CONFIGS[n](**small)
    wd = w.to(dev)
    t = w.target("q"); p = t.pool; pd = wd.target("q").pool
    merged = int(torch.bincount(w.ids[w.ids >= 0]).argmax())
    R = max(p.ranks)
    plan = DeLoraPlan(wd.ids, merged, pd.a_start, pd.a_len, R, hidden=t.h_in)
    y = wd.y0["q"].clone()
    plan.apply(y, wd.x[t.h_in], pd.key_buffer, pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, t.slot, pd.a_scaling)
    want = O.delora_compensate(w.y0["q"], w.x[t.h_in], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc,
                               w.ids, merged, t.slot, p.a_scaling)
    assert_parity(y.cpu(), want, f"config{n} deLoRA compensation")
    same = (w.ids == merged)
    assert torch.equal(y.cpu()[same], w.y0["q"][same])

    # end to end: x @ W_merged + compensation == x @ W + LoRA_own(x)
    g = torch.Generator().manual_seed(n)
    H = t.h_in
    Wb = (torch.randn(H, H, generator=g) * 0.02).to(w.dtype)
    Wm = Wb.clone().to(dev)
    merge_adapter([Wm], pd.key_buffer, pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, merged,
                  float(p.a_scaling[merged]), R, slots=(t.slot,))
    x = wd.x[H]
    out = (x.float() @ Wm.float())
    comp = torch.zeros(w.T, H, dtype=w.dtype, device=dev)
    plan.apply(comp, x, pd.key_buffer, pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, t.slot, pd.a_scaling)
    out = (out + comp.float()).cpu()
    lora = O.lora_op(torch.zeros(w.T, H, dtype=w.dtype), w.x[H], p.key_buffer, p.value_buffer, p.a_start, p.a_len,
                     p.a_loc, w.ids, t.slot, p.a_scaling, round_v=False).float()
    ref = w.x[H].float() @ Wb.float() + lora
    has = w.ids >= 0
    err = (out - ref)[has].abs().max()
    assert err <= (6e-2 if w.dtype == torch.bfloat16 else 8e-3) * (1 + ref[has].abs().max()), err


@pytest.mark.parametrize("seed", range(24))
def test_merge_random_shapes(dev, seed):
    """Non-square weights, widths that are multiples of 8 only, 1-5 pool slots, any subset of slots,
    weights that are column slices of a wider matrix (whose other columns must stay untouched)."""
    import random
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    h_in, h_out = (rnd.choice([8, 24, 72, 136, 264, 520, 1000, 1032, 2056]) for _ in range(2))
    ranks = [rnd.choice([8, 16, 24, 32, 40, 64, 128]) for _ in range(rnd.choice([1, 2, 4]))]
    n_slots = rnd.choice([1, 2, 4, 5])
    slots = rnd.sample(range(n_slots), rnd.randint(1, min(4, n_slots)))
    adapter, scaling, sign = rnd.randrange(len(ranks)), rnd.choice([1.0, 2.0, 0.5, 1.7, 0.3]), rnd.choice([1, -1])
    pad = rnd.choice([0, 8, 64])
    what = f"seed {seed} {dtype} {h_in}x{h_out} ranks {ranks} slots {slots}/{n_slots} s {scaling} sign {sign} pad {pad}"
    print(what, flush=True)
    g = torch.Generator().manual_seed(seed)
    pool = W.make_pool(ranks, h_in, h_out, dtype, g, True, n_slots=n_slots, std=0.05, heads=1)
    Ws = [(torch.randn(h_in, h_out, generator=g) * 0.05).to(dtype) for _ in slots]
    want = O.merge_adapter(Ws, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, adapter,
                           scaling, slots=slots, n_slots=n_slots, sign=sign)
    big = [torch.zeros(h_in, h_out + pad, dtype=dtype, device=dev) for _ in Ws]
    for b, w in zip(big, Ws):
        b[:, :h_out] = w.to(dev)
    Wd = [b[:, :h_out] for b in big]
    p = pool.to(dev)
    fn = merge_adapter if sign > 0 else unmerge_adapter
    fn(Wd, p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, adapter, scaling, max(ranks), slots=slots,
       n_slots=n_slots)
    for k in range(len(slots)):
        d = (Wd[k].cpu().float() - want[k].float()).abs()
        lim = 2 * ulp_of(torch.maximum(want[k].float().abs(), Ws[k].float().abs()).to(dtype))
        assert (d <= lim).all(), what + f" target {k}: more than one ulp of ab"
        assert (d > 0).float().mean() < 0.03, what
        assert not big[k][:, h_out:].any(), what + " wrote outside the weight's columns"
