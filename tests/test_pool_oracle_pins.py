"""Pins of oracle/pool_oracle.py (the checker of the adapter residency kernels): hand-derived
vectors, plain-loop brute force over exhaustive small states, invariants.  CPU only."""
import itertools
import json
import os
import random

import pytest
import torch

from oracle import pool_oracle as P

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "pool_index.json")))


def state_of(s):
    return torch.tensor([c == "1" for c in s], dtype=torch.bool)


def alloc_with_state(s):
    a = P.Allocator(len(s))
    a.mem_state = state_of(s)
    a.can_use_mem_size = int(a.mem_state.sum())
    return a


def loop_first_fit(state, need):
    """Walk the rows in order and take the free ones."""
    out = []
    for i, free in enumerate(state):
        if len(out) == need:
            break
        if free:
            out.append(i)
    return out


def loop_first_window(state, need):
    for s in range(0, len(state) - need + 1):
        if all(state[s:s + need]):
            return s
    return None


@pytest.mark.parametrize("case", GOLD["alloc_cases"], ids=lambda c: c["name"])
def test_allocator_golden(case):
    a = alloc_with_state(case["state"])
    if case["op"] == "alloc":
        assert a.alloc(case["need"]).tolist() == case["index"]
    elif case["op"] == "alloc_contiguous":
        got = a.alloc_contiguous(case["need"])
        if case["start"] is None:
            assert got is None
        else:
            assert got[0].tolist() == case["index"] and got[1] == case["start"] and got[2] == case["start"] + case["need"]
    else:
        a.free(torch.tensor(case["index"], dtype=torch.long))
    assert a.mem_state.tolist() == state_of(case["after"]).tolist()


def test_allocator_exhaustive_small_states():
    """Every state of a 7-row pool and every request size: tensor formulation == plain loops."""
    for bits in itertools.product([0, 1], repeat=7):
        free = sum(bits)
        for need in range(0, free + 1):
            a = alloc_with_state("".join(map(str, bits)))
            assert a.alloc(need).tolist() == loop_first_fit(list(bits), need)
            assert int(a.mem_state.sum()) == free - need == a.can_use_mem_size
        for need in range(1, free + 1):
            a = alloc_with_state("".join(map(str, bits)))
            got = a.alloc_contiguous(need)
            want = loop_first_window(list(bits), need)
            if want is None:
                assert got is None and a.mem_state.tolist() == [bool(b) for b in bits]
            else:
                assert got[1] == want and got[0].tolist() == list(range(want, want + need))
                assert int(a.mem_state.sum()) == free - need


def test_allocator_random_sequences_and_invariants():
    rng = random.Random(7)
    a = P.Allocator(300)
    shadow = [True] * 300
    held = []
    for _ in range(400):
        if held and rng.random() < 0.45:
            idx = held.pop(rng.randrange(len(held)))
            a.free(idx)
            for i in idx.tolist():
                shadow[i] = True
        else:
            need = rng.randint(0, 40)
            if need > a.can_use_mem_size:
                with pytest.raises(Exception, match="warn no enough pool space"):
                    a.alloc(need)
                continue
            if rng.random() < 0.3 and need > 0:
                got = a.alloc_contiguous(need)
                want = loop_first_window(shadow, need)
                assert (got is None) == (want is None)
                if got is None:
                    continue
                idx = got[0]
                assert idx.tolist() == list(range(want, want + need))
            else:
                idx = a.alloc(need)
                assert idx.tolist() == loop_first_fit(shadow, need)
            for i in idx.tolist():
                assert shadow[i]
                shadow[i] = False
            held.append(idx)
        assert a.mem_state.tolist() == shadow and a.can_use_mem_size == sum(shadow)
    for idx in held:
        a.free(idx)
    assert bool(a.mem_state.all()) and a.can_use_mem_size == 300


def make_adapters(spec, layers, heads, H, n_slots, dtype=torch.float16, seed=0):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, d in spec.items():
        r = d["r"]
        peft_A = [[torch.randn(r, H, generator=g) for _ in range(n_slots)] for _ in range(layers)]
        peft_B = [[torch.randn(H, r, generator=g) for _ in range(n_slots)] for _ in range(layers)]
        w = [P.w_combined(peft_A[l], peft_B[l], r, heads, H, dtype) for l in range(layers)]
        out[name] = dict(lora_dir=name, r=r, scaling=d["scaling"], w=w, peft_A=peft_A, peft_B=peft_B)
    return out


@pytest.mark.parametrize("key", ["history", "prefetch_history"])
def test_residency_golden(key):
    h = GOLD[key]
    layers, heads, H = 2, 2, 16
    ads = make_adapters(h["adapters"], layers, heads, H, h["n_slots"])
    res = P.Residency(P.Allocator(h["tot_size"]), layers, heads, H // heads, n_slots=h["n_slots"])
    for step in h["steps"]:
        if step["op"] == "offload":
            res.offload_adapters(step["reserve"])
        else:
            res.load_adapters([ads[d] for d in step["dirs"]], prefetch=step["op"] == "prefetch")
        assert res.adapter_dirs == step["adapter_dirs"]
        assert res.a_start.tolist() == step["a_start"] and res.a_len.tolist() == step["a_len"]
        assert res.a_loc.tolist() == step["a_loc"]
        assert res.a_scaling.tolist() == step["a_scaling"]
        assert res.mem.can_use_mem_size == step["free"] == int(res.mem.mem_state.sum())
        assert res.idx_map == {d: i for i, d in enumerate(step["adapter_dirs"])}
        # what the pool holds for every resident adapter is what PEFT's matrices say
        for d in res.adapter_dirs:
            for layer in range(layers):
                for slot in range(h["n_slots"]):
                    A, B = res.densify(res.idx_map[d], layer, slot)
                    assert torch.equal(A, ads[d]["peft_A"][layer][slot].T.to(torch.float16))
                    assert torch.equal(B, ads[d]["peft_B"][layer][slot].T.to(torch.float16))


def test_w_combined_layout_literal():
    """A block = lora_A.weight as is; B block = lora_B.weight [H, r] read flat as [r, H];
    a missing slot is zeros (lora_layer_weight.py:452-516)."""
    r, heads, H = 2, 2, 4
    A = torch.arange(r * H, dtype=torch.float32).reshape(r, H)           # lora_A.weight
    B = 100 + torch.arange(H * r, dtype=torch.float32).reshape(H, r)     # lora_B.weight
    w = P.w_combined([A, None], [B, None], r, heads, H)
    assert w.shape == (2, 2 * r, heads, H // heads)
    assert w[0, :r].reshape(r, H).tolist() == A.tolist()
    assert w[1, :r].reshape(-1).tolist() == B.reshape(-1).tolist()
    assert not w[:, r:].any()


def test_residency_random_history_invariants():
    rng = random.Random(3)
    layers, heads, H, S = 1, 2, 8, 4
    spec = {f"ad{i}": dict(r=rng.choice([1, 2, 3]), scaling=float(rng.choice([0.5, 1.0, 2.0]))) for i in range(12)}
    ads = make_adapters(spec, layers, heads, H, S, seed=5)
    res = P.Residency(P.Allocator(96), layers, heads, H // heads, n_slots=S)
    for _ in range(60):
        if rng.random() < 0.5:
            want = rng.sample(sorted(spec), rng.randint(1, 4))
            need = sum(spec[d]["r"] * S for d in dict.fromkeys(want) if d not in res.idx_map)
            if need > res.mem.can_use_mem_size:
                continue
            res.load_adapters([ads[d] for d in dict.fromkeys(want)])
        else:
            keep = [d for d in res.adapter_dirs if rng.random() < 0.6]
            res.offload_adapters(keep)
        # index tensors are consistent and rows are owned exactly once
        assert res.a_len.tolist() == [spec[d]["r"] * S for d in res.adapter_dirs]
        assert res.a_start.tolist() == [sum(res.a_len.tolist()[:i]) for i in range(len(res.adapter_dirs))]
        rows = res.a_loc.tolist()
        assert len(rows) == len(set(rows)) == sum(res.a_len.tolist())
        assert all(not res.mem.mem_state[r_] for r_ in rows)
        assert int(res.mem.mem_state.sum()) == 96 - len(rows) == res.mem.can_use_mem_size
        for d in res.adapter_dirs:
            A, B = res.densify(res.idx_map[d], 0, 1)
            assert torch.equal(A, ads[d]["peft_A"][0][1].T.to(torch.float16))
            assert torch.equal(B, ads[d]["peft_B"][0][1].T.to(torch.float16))
