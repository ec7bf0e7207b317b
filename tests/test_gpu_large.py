"""Token counts far above the benchmark configurations, up to the library's stated maximum (2**22 tokens):
the plan (sort, tile lists), both kernels and the drop-in entry points index with the widths of the real
shapes, so rows, tiles and grids of this size must not overflow anything.  Narrow rows keep the operands at a
few hundred MB; the oracle is the per-adapter matrix product of oracle/lora_oracle.py on the CPU."""
import pytest
import torch

from oracle import lora_oracle as O
from valora_amd import _lib
from valora_amd import workloads as W
from valora_amd.plan import LoraPlan
from tests._util import assert_parity

pytestmark = pytest.mark.gpu

MAX_TOKENS = 1 << 22


def _case(T, h_in, h_out, ranks, n_slots, seed, dtype=torch.bfloat16, style="random"):
    g = torch.Generator().manual_seed(seed)
    pool = W.make_pool(ranks, h_in, h_out, dtype, g, True, n_slots=n_slots, std=0.05, heads=1,
                       scalings=[0.5 + 0.25 * (i % 4) for i in range(len(ranks))])
    if style == "random":
        ids = torch.randint(-1, len(ranks), (T,), generator=g)
    else:   # long runs of one adapter, as prefill requests give them
        ids = torch.repeat_interleave(torch.randint(0, len(ranks), ((T + 4095) // 4096,), generator=g), 4096)[:T]
    x = torch.randn(T, h_in, generator=g).to(dtype)
    y0 = torch.randn(T, h_out, generator=g).to(dtype)
    return pool, ids, x, y0


@pytest.mark.parametrize("T,h_in,h_out,ranks,style", [
    (200_003, 256, 512, [8, 16, 32, 64, 16, 8, 24], "random"),
    ((1 << 20) + 1, 64, 128, [8, 16, 8, 16, 24], "runs"),
    (MAX_TOKENS, 64, 64, [8, 16, 8], "random"),
], ids=["200k", "1M", "max"])
def test_planned_op_on_very_large_batches(dev, T, h_in, h_out, ranks, style):
    pool, ids, x, y0 = _case(T, h_in, h_out, ranks, 2, T % 1000, style=style)
    want = O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 1,
                     pool.a_scaling, n_slots=2)
    pd = pool.to(dev)
    plan = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, max(ranks), n_slots=2, hidden=h_in)
    h = plan.header()
    assert h["T"] == T and h["n_active"] == int((ids >= 0).sum())
    y = y0.to(dev)
    plan.apply(y, x.to(dev), pd.key_buffer, pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, 1, pd.a_scaling)
    got = y.cpu()
    assert_parity(got, want, f"T={T} {h_in}->{h_out} ranks {ranks} {style}")
    assert torch.equal(got[ids < 0], y0[ids < 0])
    # the sorted order the plan holds is a permutation of the tokens with an adapter, grouped by adapter, in
    # token order inside a group
    perm = plan.perm().cpu().long()
    assert perm.numel() == h["n_active"]
    key = ids[perm] * (T + 1) + perm
    assert bool((key[1:] > key[:-1]).all())


def test_drop_in_entry_point_on_a_very_large_batch(dev):
    from valora_amd.kernels import dispatch_bgmv
    T, h_in, h_out, ranks = 300_001, 128, 256, [16, 8, 32, 16]
    pool, ids, x, y0 = _case(T, h_in, h_out, ranks, 4, 7, dtype=torch.float16)
    R = max(ranks)
    cidx = (pool.a_start, pool.a_len, pool.a_loc)
    want_v = O.bgmv_shrink(torch.zeros(T, R, dtype=x.dtype), x, pool.key_buffer, *cidx, ids, 2)
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    delta = torch.zeros(T, R, dtype=x.dtype, device=dev)
    y = y0.to(dev)
    dispatch_bgmv(delta, x.to(dev), pd.key_buffer, *idx, ids.to(dev), 2, pd.a_scaling)
    dispatch_bgmv(y, delta, pd.value_buffer, *idx, ids.to(dev), 2, pd.a_scaling)
    assert_parity(delta.cpu(), want_v, "large dispatch_bgmv shrink")
    want = O.bgmv_expand(y0, delta.cpu(), pool.value_buffer, *cidx, ids, 2, pool.a_scaling)
    assert_parity(y.cpu(), want, "large dispatch_bgmv expand")


def test_more_tokens_than_the_maximum_are_refused(dev):
    L = _lib.lib()
    assert L.mlora_plan_bytes(MAX_TOKENS, 4) > 0
    ids = torch.zeros(8, dtype=torch.long, device=dev)
    a = torch.zeros(4, dtype=torch.long, device=dev)
    buf = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
    handle = _lib.Plan(_lib.ptr(buf), buf.numel(), 0, 0, 0, 0)
    rc = L.mlora_build_plan(_lib.current_stream(dev), handle, _lib.ptr(ids), MAX_TOKENS + 1, _lib.ptr(a), _lib.ptr(a), 4, 4,
                            16, 16)
    assert rc != 0 and b"T=" in L.mlora_last_error()


def test_rows_beyond_two_to_the_31_elements(dev):
    """x and y of more than 2**31 elements each (262 147 tokens of 8192): every row offset needs 64 bits.  The
    operands are drawn on the GPU; the oracle gets the first and the last rows (the op treats rows independently)."""
    T, H, ranks = (1 << 18) + 3, 8192, [16, 64, 8, 32]
    assert T * H > (1 << 31)
    g = torch.Generator().manual_seed(31)
    pool = W.make_pool(ranks, H, H, torch.bfloat16, g, True, n_slots=1, std=0.02, heads=1)
    ids = torch.repeat_interleave(torch.randint(-1, len(ranks), ((T + 127) // 128,), generator=g), 128)[:T]
    gd = torch.Generator(device=dev).manual_seed(32)
    x = torch.randn(T, H, generator=gd, device=dev, dtype=torch.float32).bfloat16()
    y = torch.randn(T, H, generator=gd, device=dev, dtype=torch.float32).bfloat16()
    rows = torch.cat([torch.arange(0, 700), torch.arange(T - 1500, T)])
    x_s, y0_s, ids_s = x[rows.to(dev)].cpu(), y[rows.to(dev)].cpu(), ids[rows]
    assert len(set(ids_s.tolist())) >= 3
    pd = pool.to(dev)
    plan = LoraPlan(ids.to(dev), pd.a_start, pd.a_len, max(ranks), n_slots=1, hidden=H)
    plan.apply(y, x, pd.key_buffer, pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, 0, pd.a_scaling)
    want = O.lora_op(y0_s, x_s, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids_s, 0,
                     pool.a_scaling, n_slots=1)
    assert_parity(y[rows.to(dev)].cpu(), want, "rows at both ends of a 2**31-element matrix")


def test_row_scatter_and_gather_in_a_pool_beyond_4_gib(dev):
    """A pool of 8 layers x 70 000 rows x 4096 fp16 (4.6 GB, more than 2**31 elements): rows near the end of the last
    layers are written and read back; torch's indexed assignment on the same tensor is the checker
    (valora/server/router/model_infer/infer_adapter.py:59 is exactly that assignment)."""
    layers, rows, H, n = 8, 70_000, 4096, 192
    assert layers * rows * H > (1 << 31)
    g = torch.Generator(device=dev).manual_seed(5)
    pool = torch.zeros(layers, rows, H, dtype=torch.float16, device=dev)
    packed = torch.randn(layers, n, H, generator=g, device=dev, dtype=torch.float32).half()
    loc = torch.cat([torch.arange(rows - n // 2, rows), torch.randperm(rows - n, generator=torch.Generator().manual_seed(6))[:n // 2]])
    loc_d = loc.to(dev)
    st = _lib.current_stream(dev)
    esz = 2
    _lib.check(_lib.lib().mlora_pool_scatter_rows(st, _lib.ptr(pool), rows, rows * H * esz, _lib.ptr(packed),
                                                  n * H * esz, _lib.ptr(loc_d), n, H * esz, layers))
    for l in (0, layers - 1):
        assert torch.equal(pool[l][loc_d], packed[l])
    assert int(pool.count_nonzero()) == int(packed.count_nonzero())      # nothing written anywhere else
    back = torch.empty_like(packed)
    _lib.check(_lib.lib().mlora_pool_gather_rows(st, _lib.ptr(pool), rows, rows * H * esz, _lib.ptr(back),
                                                 n * H * esz, _lib.ptr(loc_d), n, H * esz, layers))
    assert torch.equal(back, packed)
