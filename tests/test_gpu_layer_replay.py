"""GPU: one layer's LoRA calls in the order the reference's caller issues them, through the module names the
reference imports (``valora_amd.install_aliases()``), over several layers and two batches.

The reference's forward pass allocates three ``delta`` tensors, zeroes them once, and every layer then issues
3 shrinks into ``delta[0..2]``, 3 expands into q / k / v, and after attention one more shrink into ``delta[0]``
and one expand into o -- 8 calls per layer with the SAME index tensors
(valora/models/peft/lora_unordered_batch_infer.py:304-308 the scratch, :946-988 the segment-signature branch
with ``[delora_tk_index:]`` row slices, :1453-1530 and :1610-1651 the o projection and the BGMV branch).  What a
single call cannot show: ``delta`` carries the previous layer's (and here even the previous batch's) values in
its columns beyond an adapter's rank and in ``delta[0]`` between q and o, and the plan of the batch is cut on the
first of the 8 x layers calls and found again by all the others.
"""
import sys

import pytest
import torch

import valora_amd
from oracle import lora_oracle as O
from valora_amd import _plan_cache, workloads as W

from tests._util import assert_parity

pytestmark = pytest.mark.gpu

N_LAYERS = 3


def _reference_ops():
    """The op functions as the reference's caller gets them: by its own import names."""
    valora_amd.install_aliases()
    return (sys.modules["valora._kernels"].dispatch_bgmv, sys.modules["atmm_ops"].dispatch_bgmv,
            sys.modules["valora.models.peft.triton_kernel.lora.lora_prefill"])


def _layers(pool, T_rows, h, dtype, dev, seed):
    """Per layer: pool slices with their own weights (the reference indexes key_buffer[layer_id]) and the
    activations the base model would hand over: the layer input, the base projections q, k, v, the attention
    output and the base o projection."""
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(N_LAYERS):
        kb = (torch.randn(pool.key_buffer.shape, generator=g) * 0.05).to(dtype)
        vb = (torch.randn(pool.value_buffer.shape, generator=g) * 0.05).to(dtype)
        acts = {n: torch.randn(T_rows, h, generator=g).to(dtype) for n in ("x", "q", "k", "v", "attn", "o")}
        out.append((kb, vb, acts))
    return out


def _oracle_layer(pool, kb, vb, acts, ids, rows):
    """q, k, v, o of one layer as the operator defines them (oracle.lora_op) on the rows from `rows` on."""
    idx = (pool.a_start, pool.a_len, pool.a_loc)
    want = {}
    for name, src, slot in (("q", "x", 0), ("k", "x", 1), ("v", "x", 2), ("o", "attn", 3)):
        y = acts[name].clone()
        y[rows:] = O.lora_op(acts[name][rows:], acts[src][rows:], kb, vb, *idx, ids, slot, pool.a_scaling)
        want[name] = y
    return want


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_bgmv_branch_layer_call_order(dev, dtype):
    """The BGMV branch (:1610-1651 for o, the same shape of calls for q, k, v): per-token ids, whole tensors.
    Batch 1 mixes ranks 16 and 32; batch 2 (same size, other requests) uses ranks 8 and 16 only, so every column
    from 8 or 16 on of the reused ``delta`` holds batch 1's values when batch 2 runs."""
    dispatch_bgmv, _, _ = _reference_ops()
    h, R, T = 512, 32, 96
    g = torch.Generator().manual_seed(11)
    ranks = [16, 32, 8, 32, 16, 8, 8]
    pool = W.make_pool(ranks, h, h, dtype, g, True, std=0.05, scalings=[0.5 + 0.25 * i for i in range(len(ranks))])
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    big = torch.tensor([0, 1, 3, 4])             # adapters of rank 16 / 32
    small = torch.tensor([2, 5, 6, 0, 4])        # ranks 8 and 16
    batches = [big[torch.randint(0, len(big), (T,), generator=g)], small[torch.randint(0, len(small), (T,), generator=g)]]
    delta = [torch.zeros(T, R, dtype=dtype, device=dev) for _ in range(3)]      # zeroed ONCE (:304-308)
    for b, ids in enumerate(batches):
        req_bins = ids.to(dev)
        layers = _layers(pool, T, h, dtype, dev, 100 + b)
        h0, m0 = _plan_cache.hits, _plan_cache.misses
        for l, (kb, vb, acts) in enumerate(layers):
            kbd, vbd = kb.to(dev), vb.to(dev)
            a = {n: t.to(dev) for n, t in acts.items()}
            for i in range(3):                   # shrinks of q, k, v
                dispatch_bgmv(delta[i], a["x"], kbd, *idx, req_bins, i, pd.a_scaling)
            for i, n in enumerate(("q", "k", "v")):
                dispatch_bgmv(a[n], delta[i], vbd, *idx, req_bins, i, pd.a_scaling)
            dispatch_bgmv(delta[0], a["attn"], kbd, *idx, req_bins, 3, pd.a_scaling)     # o reuses delta[0]
            dispatch_bgmv(a["o"], delta[0], vbd, *idx, req_bins, 3, pd.a_scaling)
            torch.cuda.synchronize()
            want = _oracle_layer(pool, kb, vb, acts, ids, 0)
            for n in ("q", "k", "v", "o"):
                assert_parity(a[n].cpu(), want[n], f"batch {b} layer {l} {n} ({dtype})")
        assert _plan_cache.misses - m0 == 1, "the batch's plan is cut once"
        assert _plan_cache.hits - h0 == 8 * N_LAYERS - 1, "and found again by every other call of the batch"
    # batch 2 left batch 1's values in the columns its adapters do not have
    r_of = torch.tensor(ranks)[batches[1]]
    stale = delta[1].cpu()[r_of == 8][:, 16:]
    assert bool((stale != 0).any()), "the test must really run on a scratch with stale columns"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_sgmm_branch_layer_call_order(dev, dtype):
    """The segment-signature branch (:946-988, :1610-1622): the tensors ``set_sgmm_args`` emits, a leading run of
    the merged adapter whose rows the calls skip through ``[delora_tk_index:]`` views of x, q, k, v and o, the
    decremented problem count.  Batch 2 has no merged run, as many kept rows as batch 1 and smaller ranks; the
    ``delta`` tensors are batch 1's."""
    from valora_amd.segments import set_sgmm_args
    _, dispatch_sgmm, _ = _reference_ops()
    h, R = 256, 32
    ranks = {"A": 16, "B": 32, "C": 32, "M": 16, "D": 8, "E": 8}
    cases = [(["M", "A", "A", "B", "C"], [40, 30, 25, 50, 33], "M"),
             (["D", "D", "E", "A"], [38, 20, 50, 30], None)]
    resident = sorted(ranks)
    g = torch.Generator().manual_seed(12)
    pool = W.make_pool([ranks[d] for d in resident], h, h, dtype, g, True, std=0.05,
                       scalings=[0.5 + 0.25 * i for i in range(len(resident))])
    pd = pool.to(dev)
    idx = (pd.a_start, pd.a_len, pd.a_loc)
    rank_counts = torch.full((128,), 64, dtype=torch.long, device=dev)      # req_queue.py:25
    tmp_d = torch.zeros(128 * 60, dtype=torch.int8, device=dev)
    kept = 138
    delta = [torch.zeros(kept, R, dtype=dtype, device=dev) for _ in range(3)]
    for b, (dirs, lens, merged) in enumerate(cases):
        oc, lora_ids, st, num_problems = set_sgmm_args(dirs, lens, True, merged, device=dev)
        P, (de_req, de_tok) = num_problems[0], num_problems[1]
        if de_req > 0:                           # :277-283
            P -= 1
        T = sum(lens)
        assert T - de_tok == kept
        req_bins = torch.tensor([resident.index(d) for d in dirs])
        batch_req_bins = torch.repeat_interleave(req_bins[de_req:], torch.tensor(lens[de_req:]))
        ids_d = batch_req_bins.to(dev)
        layers = _layers(pool, T, h, dtype, dev, 200 + b)
        h0, m0 = _plan_cache.hits, _plan_cache.misses
        for l, (kb, vb, acts) in enumerate(layers):
            kbd, vbd = kb.to(dev), vb.to(dev)
            a = {n: t.to(dev) for n, t in acts.items()}
            seg = (oc, rank_counts, lora_ids, st, tmp_d, P)
            for i in range(3):
                dispatch_sgmm(delta[i], a["x"][de_tok:], kbd, *idx, ids_d, i, pd.a_scaling, *seg, 64, 32, 32, 32, 32, 32)
            for i, n in enumerate(("q", "k", "v")):
                dispatch_sgmm(a[n][de_tok:], delta[i], vbd, *idx, ids_d, i, pd.a_scaling, *seg, 64, 64, 32, 64, 64, 32)
            dispatch_sgmm(delta[0], a["attn"][de_tok:], kbd, *idx, ids_d, 3, pd.a_scaling, *seg, 64, 32, 32, 32, 32, 32)
            dispatch_sgmm(a["o"][de_tok:], delta[0], vbd, *idx, ids_d, 3, pd.a_scaling, *seg, 64, 64, 32, 64, 64, 32)
            torch.cuda.synchronize()
            want = _oracle_layer(pool, kb, vb, acts, batch_req_bins, de_tok)
            for n in ("q", "k", "v", "o"):
                assert_parity(a[n].cpu(), want[n], f"batch {b} layer {l} {n} ({dtype})")
                assert torch.equal(a[n].cpu()[:de_tok], acts[n][:de_tok]), "rows of the merged leading run are not touched"
        assert _plan_cache.misses - m0 == 1, "the batch's plan is cut once"
        assert _plan_cache.hits - h0 == 8 * N_LAYERS - 1, "and found again by every other call of the batch"
