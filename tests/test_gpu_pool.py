"""GPU parity of adapter residency (row allocator, row scatter / gather, re-indexing, InferAdapter)
against oracle/pool_oracle.py and the hand-derived vectors; all integer results bit-exact.  The last
tests run the LoRA op on a pool filled through this path."""
import json
import os
import random

import pytest
import torch

from oracle import lora_oracle as O
from oracle import pool_oracle as P
from valora_amd import _lib
from valora_amd.infer_adapter import InferAdapter, LoraAdapterWeights, MemoryAllocator

pytestmark = pytest.mark.gpu

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "pool_index.json")))


def state_of(s, dev):
    return torch.tensor([c == "1" for c in s], dtype=torch.bool, device=dev)


def allocator(dev, tot, layers=1, heads=2, head_dim=8, dtype=torch.float16):
    return MemoryAllocator(tot, tot, dtype, heads, head_dim, layers, device=dev)


@pytest.mark.parametrize("case", GOLD["alloc_cases"], ids=lambda c: c["name"])
def test_allocator_golden(dev, case):
    a = allocator(dev, len(case["state"]))
    a.mem_state.copy_(state_of(case["state"], dev))
    a.can_use_mem_size = case["state"].count("1")
    if case["op"] == "alloc":
        assert a.alloc(case["need"]).tolist() == case["index"]
    elif case["op"] == "alloc_contiguous":
        got = a.alloc_contiguous(case["need"])
        if case["start"] is None:
            assert got is None
        else:
            assert got[0].tolist() == case["index"] and got[1] == case["start"] and got[2] == case["start"] + case["need"]
    else:
        a.free(torch.tensor(case["index"], dtype=torch.long, device=dev))
    assert a.mem_state.cpu().tolist() == state_of(case["after"], "cpu").tolist()
    assert a.can_use_mem_size == case["after"].count("1") or case["op"] == "free"


@pytest.mark.parametrize("tot,max_need,seed", [(37, 9, 0), (1000, 200, 1), (16384, 3000, 2), (50001, 20000, 3),
                                               (200000, 70000, 4)])
def test_allocator_random_sequences_vs_oracle(dev, tot, max_need, seed):
    """Pools smaller and larger than one pass of the scan (16384 rows); fragmented states."""
    rng = random.Random(seed)
    a, o = allocator(dev, tot), P.Allocator(tot)
    # fragment the pool first: take everything, free a random half
    everything = a.alloc(tot)
    o.alloc(tot)
    mask = torch.rand(tot, generator=torch.Generator().manual_seed(seed)) < 0.5
    a.free(everything[mask.to(dev)])
    o.free(torch.arange(tot)[mask])
    held = []
    for step in range(40):
        if held and rng.random() < 0.4:
            ia, io = held.pop(rng.randrange(len(held)))
            a.free(ia)
            o.free(io)
        else:
            need = rng.randint(0, max_need)
            if need > o.can_use_mem_size:
                with pytest.raises(Exception, match="warn no enough pool space"):
                    a.alloc(need)
                continue
            if need > 0 and rng.random() < 0.4:
                need = min(need, 6) if rng.random() < 0.7 else need
                ga, go = a.alloc_contiguous(need), o.alloc_contiguous(need)
                assert (ga is None) == (go is None), f"step {step}"
                if ga is None:
                    continue
                assert ga[1:] == go[1:] and torch.equal(ga[0].cpu(), go[0])
                held.append((ga[0], go[0]))
            else:
                ia, io = a.alloc(need), o.alloc(need)
                assert torch.equal(ia.cpu(), io), f"step {step} need {need}"
                held.append((ia, io))
        assert a.can_use_mem_size == o.can_use_mem_size
        assert torch.equal(a.mem_state.cpu(), o.mem_state), f"step {step}"
    a.free_all()
    assert bool(a.mem_state.all()) and a.can_use_mem_size == tot


def test_allocator_contiguous_window_across_scan_passes(dev):
    """A free run that starts in one 16384-row pass of the scan and ends in the next."""
    tot = 40000
    a, o = allocator(dev, tot), P.Allocator(tot)
    for x in (a, o):
        x.alloc(tot)
    run = torch.arange(16380, 16395)
    short = torch.tensor([5, 6, 7, 100, 101, 16000, 16001, 16002, 16003])
    for idx in (run, short):
        a.free(idx.to(dev))
        o.free(idx)
    for need in (10, 5, 4, 3):
        ga, go = a.alloc_contiguous(need), o.alloc_contiguous(need)
        assert (ga is None) == (go is None)
        if ga is not None:
            assert ga[1:] == go[1:] and torch.equal(ga[0].cpu(), go[0])
        assert torch.equal(a.mem_state.cpu(), o.mem_state)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layers,rows,H,n", [(1, 50, 64, 7), (3, 300, 4096, 64), (32, 2000, 4096, 256), (2, 64, 11008, 33)])
def test_scatter_and_gather_rows(dev, dtype, layers, rows, H, n):
    g = torch.Generator().manual_seed(layers * 1000 + n)
    pool0 = torch.randn(layers, rows, H, generator=g).to(dtype)
    packed = torch.randn(layers, n, H, generator=g).to(dtype)
    loc = torch.randperm(rows, generator=g)[:n]
    want = pool0.clone()
    for l in range(layers):
        want[l][loc] = packed[l]                      # infer_adapter.py:59
    pool_d, packed_d, loc_d = pool0.to(dev), packed.to(dev), loc.to(dev)
    esz = pool_d.element_size()
    st = _lib.current_stream(dev)
    _lib.check(_lib.lib().mlora_pool_scatter_rows(st, _lib.ptr(pool_d), rows, rows * H * esz, _lib.ptr(packed_d),
                                                  n * H * esz, _lib.ptr(loc_d), n, H * esz, layers))
    assert torch.equal(pool_d.cpu(), want)
    back = torch.full_like(packed_d, 7.0)
    _lib.check(_lib.lib().mlora_pool_gather_rows(st, _lib.ptr(pool_d), rows, rows * H * esz, _lib.ptr(back),
                                                 n * H * esz, _lib.ptr(loc_d), n, H * esz, layers))
    assert torch.equal(back.cpu(), packed)
    # rows outside the pool: skipped by the scatter, zeros from the gather
    bad = loc_d.clone()
    bad[0], bad[-1] = -1, rows
    before = pool_d.clone()
    _lib.check(_lib.lib().mlora_pool_scatter_rows(st, _lib.ptr(pool_d), rows, rows * H * esz, _lib.ptr(back),
                                                  n * H * esz, _lib.ptr(bad), n, H * esz, layers))
    assert torch.equal(pool_d, before)
    _lib.check(_lib.lib().mlora_pool_gather_rows(st, _lib.ptr(pool_d), rows, rows * H * esz, _lib.ptr(back),
                                                 n * H * esz, _lib.ptr(bad), n, H * esz, layers))
    assert not back[:, 0].any() and not back[:, -1].any() and torch.equal(back[:, 1:-1].cpu(), packed[:, 1:-1])


def test_rows_argument_errors(dev):
    t = torch.zeros(4, 64, dtype=torch.float16, device=dev)
    loc = torch.zeros(2, dtype=torch.long, device=dev)
    L = _lib.lib()
    st = _lib.current_stream(dev)
    assert L.mlora_pool_scatter_rows(st, _lib.ptr(t), 4, 4 * 128, _lib.ptr(t), 2 * 128, _lib.ptr(loc), 2, 120, 1) != 0
    assert b"16 bytes" in L.mlora_last_error()
    assert L.mlora_pool_scatter_rows(st, None, 4, 4 * 128, _lib.ptr(t), 2 * 128, _lib.ptr(loc), 2, 128, 1) != 0
    assert L.mlora_pool_scatter_rows(st, None, 4, 4 * 128, None, 2 * 128, None, 0, 128, 1) == 0   # nothing to do


NET = dict(num_hidden_layers=2, hidden_size=16, num_attention_heads=2)


def weights_from_oracle_spec(spec, n_slots, seed=0):
    """The same random PEFT matrices for the product's adapter class and the oracle's dicts."""
    g = torch.Generator().manual_seed(seed)
    L, H, heads = NET["num_hidden_layers"], NET["hidden_size"], NET["num_attention_heads"]
    prod, orc = {}, {}
    for name, d in spec.items():
        r = d["r"]
        A = [[torch.randn(r, H, generator=g) for _ in range(n_slots)] for _ in range(L)]
        B = [[torch.randn(H, r, generator=g) for _ in range(n_slots)] for _ in range(L)]
        prod[name] = LoraAdapterWeights.from_dense(name, r, d["scaling"] * r, NET, A, B)
        orc[name] = dict(lora_dir=name, r=r, scaling=d["scaling"],
                         w=[P.w_combined(A[l], B[l], r, heads, H) for l in range(L)])
    return prod, orc


def assert_same_residency(ia: InferAdapter, res: P.Residency):
    assert ia.adapter_dirs == res.adapter_dirs and ia.idx_map == res.idx_map
    for name in ("a_start", "a_len", "a_loc", "a_scaling"):
        assert torch.equal(getattr(ia, name).cpu(), getattr(res, name)), name
    mm = ia.mem_manager
    assert mm.can_use_mem_size == res.mem.can_use_mem_size
    assert torch.equal(mm.mem_state.cpu(), res.mem.mem_state)
    rows = res.a_loc
    assert torch.equal(mm.key_buffer.cpu()[:, rows], res.key_buffer[:, rows])
    assert torch.equal(mm.value_buffer.cpu()[:, rows], res.value_buffer[:, rows])


@pytest.mark.parametrize("key", ["history", "prefetch_history"])
def test_infer_adapter_golden_histories(dev, key):
    h = GOLD[key]
    prod, orc = weights_from_oracle_spec(h["adapters"], h["n_slots"])
    heads, H = NET["num_attention_heads"], NET["hidden_size"]
    mm = MemoryAllocator(h["tot_size"], h["tot_size"], torch.float16, heads, H // heads, NET["num_hidden_layers"], dev)
    ia = InferAdapter.init(mm, prefetch_stream=torch.cuda.Stream(device=dev))
    res = P.Residency(P.Allocator(h["tot_size"]), NET["num_hidden_layers"], heads, H // heads, n_slots=h["n_slots"])
    for step in h["steps"]:
        if step["op"] == "offload":
            ia.offload_adapters(step["reserve"])
            res.offload_adapters(step["reserve"])
        else:
            ia.load_adapters([prod[d] for d in step["dirs"]], prefetch=step["op"] == "prefetch")
            res.load_adapters([orc[d] for d in step["dirs"]], prefetch=step["op"] == "prefetch")
        torch.cuda.synchronize(dev)
        assert ia.adapter_dirs == step["adapter_dirs"]
        assert ia.a_start.tolist() == step["a_start"] and ia.a_len.tolist() == step["a_len"]
        assert ia.a_loc.tolist() == step["a_loc"] and ia.a_scaling.tolist() == step["a_scaling"]
        assert mm.can_use_mem_size == step["free"] == int(mm.mem_state.sum())
        assert_same_residency(ia, res)


def test_infer_adapter_random_history_vs_oracle(dev):
    rng = random.Random(11)
    S = 4
    spec = {f"ad{i}": dict(r=rng.choice([1, 2, 4, 8]), scaling=float(rng.choice([0.25, 0.5, 1.0, 2.0])))
            for i in range(24)}
    prod, orc = weights_from_oracle_spec(spec, S, seed=9)
    heads, H, L = NET["num_attention_heads"], NET["hidden_size"], NET["num_hidden_layers"]
    tot = 320
    mm = MemoryAllocator(tot, tot, torch.float16, heads, H // heads, L, dev)
    ia = InferAdapter.init(mm, prefetch_stream=torch.cuda.Stream(device=dev))
    res = P.Residency(P.Allocator(tot), L, heads, H // heads, n_slots=S)
    for step in range(80):
        p = rng.random()
        if p < 0.55:
            names = list(dict.fromkeys(rng.sample(sorted(spec), rng.randint(1, 5))))
            prefetch = rng.random() < 0.3
            need = sum(spec[d]["r"] * S for d in names if d not in res.idx_map)
            if not prefetch and need > res.mem.can_use_mem_size:
                continue
            ia.load_adapters([prod[d] for d in names], prefetch=prefetch)
            res.load_adapters([orc[d] for d in names], prefetch=prefetch)
        else:
            keep = [d for d in res.adapter_dirs if rng.random() < 0.5]
            ia.offload_adapters(keep)
            res.offload_adapters(keep)
        torch.cuda.synchronize(dev)
        assert_same_residency(ia, res)


def test_offload_everything_by_naming_no_resident_adapter(dev):
    """A reserve list that names nobody resident drops every adapter (the reference's tensor code indexes
    an empty tensor in this case); rows, index and counters end up as after a full offload."""
    spec = {f"e{i}": dict(r=2, scaling=1.0) for i in range(3)}
    prod, _ = weights_from_oracle_spec(spec, 4)
    heads, H, L = NET["num_attention_heads"], NET["hidden_size"], NET["num_hidden_layers"]
    mm = MemoryAllocator(40, 40, torch.float16, heads, H // heads, L, dev)
    ia = InferAdapter.init(mm)
    ia.load_adapters(list(prod.values()))
    ia.offload_adapters(["somebody-else"])
    assert ia.adapter_dirs == [] and ia.idx_map == {} and ia.a_loc.numel() == 0 and ia.a_start.numel() == 0
    assert mm.can_use_mem_size == 40 and bool(mm.mem_state.all())
    ia.load_adapters([prod["e1"]])
    assert ia.a_loc.tolist() == list(range(8)) and ia.a_start.tolist() == [0]


def test_contiguous_rows_option(dev):
    spec = {f"c{i}": dict(r=2, scaling=1.0) for i in range(5)}
    prod, _ = weights_from_oracle_spec(spec, 4)
    heads, H, L = NET["num_attention_heads"], NET["hidden_size"], NET["num_hidden_layers"]
    mm = MemoryAllocator(64, 64, torch.float16, heads, H // heads, L, dev)
    ia = InferAdapter.init(mm)
    ia.load_adapters([prod["c0"], prod["c1"], prod["c2"]])
    ia.offload_adapters(["c0", "c2"])                 # leaves an 8-row hole at rows 8..15
    ia.load_adapters([prod["c3"], prod["c4"]], contiguous=True)
    for d in ia.adapter_dirs:
        i = ia.idx_map[d]
        rows = ia.a_loc[int(ia.a_start[i]): int(ia.a_start[i]) + int(ia.a_len[i])].tolist()
        assert rows == list(range(rows[0], rows[0] + 8)), d
    assert ia.a_loc[int(ia.a_start[ia.idx_map["c3"]])].item() == 8


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_lora_op_on_a_pool_filled_through_infer_adapter(dev, dtype):
    """Adapters go PEFT matrices -> packed -> pool rows -> dispatch_bgmv; the result is compared with
    the closed form on the PEFT matrices, before and after other adapters were dropped."""
    from valora_amd.kernels import dispatch_bgmv
    net = dict(num_hidden_layers=2, hidden_size=256, num_attention_heads=8)
    L, H = 2, 256
    g = torch.Generator().manual_seed(21)
    ranks = [8, 16, 8, 32, 16]
    ads = []
    for i, r in enumerate(ranks):
        A = [[torch.randn(r, H, generator=g) * 0.05 for _ in range(4)] for _ in range(L)]
        B = [[torch.randn(H, r, generator=g) * 0.05 for _ in range(4)] for _ in range(L)]
        ads.append(LoraAdapterWeights.from_dense(f"a{i}", r, 2.0 * r, net, A, B, dtype=dtype))
    mm = MemoryAllocator(4 * sum(ranks) + 40, 0, dtype, 8, H // 8, L, dev)
    mm.key_buffer.normal_()
    mm.value_buffer.normal_()                          # stale contents of free rows must not matter
    ia = InferAdapter.init(mm)
    ia.load_adapters(ads)
    T = 96
    x = torch.randn(T, H, generator=g).to(dtype)
    y0 = torch.randn(T, H, generator=g).to(dtype)

    def run_and_check(names_of_tokens):
        ids = torch.tensor([ia.idx_map[n] for n in names_of_tokens], dtype=torch.long)
        for layer in range(L):
            for slot in (0, 3):
                y = y0.clone().to(dev)
                delta = torch.zeros(T, 32, dtype=dtype, device=dev)
                kb, vb = mm.key_buffer[layer], mm.value_buffer[layer]
                dispatch_bgmv(delta, x.to(dev), kb, ia.a_start, ia.a_len, ia.a_loc, ids.to(dev), slot, ia.a_scaling)
                dispatch_bgmv(y, delta, vb, ia.a_start, ia.a_len, ia.a_loc, ids.to(dev), slot, ia.a_scaling)
                want = y0.float().clone()
                for t, n in enumerate(names_of_tokens):
                    A, B = ads[int(n[1:])].dense(layer, slot)          # [H, r], [r, H] in dtype
                    v = (x[t].float() @ A.float()).to(dtype).float()
                    want[t] += ads[int(n[1:])].scaling * (v @ B.float())
                got = y.cpu().float()
                assert (got - want).abs().max() <= 2e-2 + 2 ** -7 * want.abs().max() * (dtype == torch.bfloat16)
                assert O.rel_l2(got, want) <= (4e-3 if dtype == torch.bfloat16 else 1e-3)

    rng = random.Random(2)
    run_and_check([f"a{rng.randrange(5)}" for _ in range(T)])
    ia.offload_adapters(["a1", "a3", "a4"])
    assert ia.adapter_dirs == ["a1", "a3", "a4"]
    run_and_check([rng.choice(["a1", "a3", "a4"]) for _ in range(T)])
    ia.load_adapters([ads[0]])                          # comes back into the freed rows
    run_and_check([rng.choice(["a0", "a1", "a3", "a4"]) for _ in range(T)])
