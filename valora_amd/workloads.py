"""Seeded synthetic workloads: the five benchmark configurations of the multi-LoRA operator.

All random draws come from a CPU ``torch.Generator`` so the same tensors are produced on any
machine; ``Workload.to(device)`` moves them.  Shapes can be shrunk (``hidden``, ``mlp``,
``len_div``) so the CPU oracle finishes in seconds in the parity tests; the defaults are the
full benchmark shapes.

Token order follows the reference's batches: requests in arrival order, each request's tokens
contiguous (valora/server/router/model_infer/infer_batch.py:60-110), per-token adapter id =
``repeat_interleave(req_bins, b_seq_len)`` (valora/models/peft/lora_unordered_batch_infer.py:291-293).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Tuple

import torch

from .pool import AdapterPool


@dataclass
class Target:
    name: str
    pool: AdapterPool
    slot: int
    h_in: int
    h_out: int


@dataclass
class Workload:
    name: str
    dtype: torch.dtype
    req_bins: torch.Tensor            # int64 [n_req]   adapter index per request
    b_seq_len: torch.Tensor           # int32 [n_req]   rows per request in this call
    b_start_loc: torch.Tensor         # int32 [n_req]
    ids: torch.Tensor                 # int64 [T]       per-token adapter index
    x: Dict[int, torch.Tensor]        # h_in -> [T, h_in]
    y0: Dict[str, torch.Tensor]       # target name -> [T, h_out]
    targets: List[Target] = field(default_factory=list)
    notes: str = ""

    @property
    def T(self) -> int:
        return int(self.ids.numel())

    def to(self, device) -> "Workload":
        pools = {}
        tg = []
        for t in self.targets:
            if id(t.pool) not in pools:
                pools[id(t.pool)] = t.pool.to(device)
            tg.append(Target(t.name, pools[id(t.pool)], t.slot, t.h_in, t.h_out))
        return Workload(self.name, self.dtype, self.req_bins.to(device), self.b_seq_len.to(device),
                        self.b_start_loc.to(device), self.ids.to(device),
                        {k: v.to(device) for k, v in self.x.items()},
                        {k: v.to(device) for k, v in self.y0.items()}, tg, self.notes)

    def target(self, name: str) -> Target:
        return next(t for t in self.targets if t.name == name)

    def algorithmic_bytes(self, name: str) -> int:
        """x read once + the touched adapters' A and B slices once + y read and written
        (the [T, r] intermediate is not counted: a fused kernel keeps it on chip)."""
        t = self.target(name)
        s = 2
        used = sorted(set(int(a) for a in self.ids.tolist() if a >= 0))
        w = sum(t.pool.ranks[a] * (t.h_in + t.h_out) * s for a in used)
        return self.T * t.h_in * s + w + 2 * self.T * t.h_out * s

    def flops(self, name: str) -> int:
        t = self.target(name)
        return sum(2 * t.pool.ranks[int(a)] * (t.h_in + t.h_out) for a in self.ids.tolist() if a >= 0)


def zipf_ids(n_adapters: int, n: int, skew: float, g: torch.Generator) -> torch.Tensor:
    p = torch.arange(1, n_adapters + 1, dtype=torch.float64).pow(-skew)
    return torch.multinomial(p / p.sum(), n, replacement=True, generator=g)


def make_pool(ranks, h_in, h_out, dtype, g, paged=True, n_slots=4, std=0.02, scalings=None,
              rows_per_adapter=None, extra_rows=0, heads=32):
    """Random pool: every row ~ N(0, std); ``paged`` scatters each adapter's rows with a random
    permutation (like ``bench_ops.py:118-124`` in the reference's op bench), otherwise rows are
    consecutive (the naive adapter's ``a_loc = arange``, naive_infer_adapter.py:99)."""
    n_rows = sum(n_slots * r for r in ranks) + extra_rows
    pool = AdapterPool(n_rows, h_in, h_out, dtype, "cpu", n_slots, heads)
    pool.key_buffer.copy_((torch.randn(n_rows, h_in, generator=g) * std).view_as(pool.key_buffer))
    pool.value_buffer.copy_((torch.randn(n_rows, h_out, generator=g) * std).view_as(pool.value_buffer))
    if rows_per_adapter is None:
        order = torch.randperm(n_rows, generator=g).tolist() if paged else list(range(n_rows))
        rows_per_adapter, o = [], 0
        for r in ranks:
            rows_per_adapter.append(order[o:o + n_slots * r])
            o += n_slots * r
    starts, lens, locs = [], [], []
    o = 0
    for r, rows in zip(ranks, rows_per_adapter):
        starts.append(o); lens.append(n_slots * r); locs.extend(rows); o += n_slots * r
    pool.a_start = torch.tensor(starts, dtype=torch.long)
    pool.a_len = torch.tensor(lens, dtype=torch.long)
    pool.a_loc = torch.tensor(locs, dtype=torch.long)
    sc = [1.0] * len(ranks) if scalings is None else scalings
    pool.a_scaling = torch.tensor(sc, dtype=torch.float32).to(dtype)
    pool.ranks = list(ranks)
    pool._free = []
    pool.rows_per_adapter = rows_per_adapter
    return pool


def _finish(name, dtype, req_bins, seq_lens, row_scale, pools: Dict[str, Tuple[AdapterPool, int, int, int]],
            g, y0_random, notes=""):
    req_bins = torch.as_tensor(req_bins, dtype=torch.long)
    b_seq_len = torch.as_tensor(seq_lens, dtype=torch.int32)
    b_start_loc = (torch.cumsum(b_seq_len, 0) - b_seq_len).to(torch.int32)
    ids = torch.repeat_interleave(req_bins, b_seq_len.to(torch.long))
    T = int(ids.numel())
    x, y0, targets = {}, {}, []
    for tname, (pool, slot, h_in, h_out) in pools.items():
        if h_in not in x:
            xi = torch.randn(T, h_in, generator=g)
            if row_scale is not None:
                xi = xi * row_scale[:, None]
            x[h_in] = xi.to(dtype)
        y0[tname] = (torch.randn(T, h_out, generator=g) if y0_random else torch.zeros(T, h_out)).to(dtype)
        targets.append(Target(tname, pool, slot, h_in, h_out))
    return Workload(name, dtype, req_bins, b_seq_len, b_start_loc, ids, x, y0, targets, notes)


def _layer_pools(ranks, hidden, mlp, dtype, g, names, paged=True, scalings=None):
    """One row numbering shared by three buffers pairs: attention (hidden->hidden, slots q,k,v,o),
    gate/up (hidden->mlp, slots 0,1) and down (mlp->hidden, slot 0)."""
    attn = make_pool(ranks, hidden, hidden, dtype, g, paged, 4, scalings=scalings)
    out = {}
    for i, n in enumerate(("q", "k", "v", "o")):
        if n in names:
            out[n] = (attn, i, hidden, hidden)
    if "gate" in names or "up" in names:
        gu = make_pool(ranks, hidden, mlp, dtype, g, paged, 4, scalings=scalings,
                       rows_per_adapter=attn.rows_per_adapter)
        if "gate" in names:
            out["gate"] = (gu, 0, hidden, mlp)
        if "up" in names:
            out["up"] = (gu, 1, hidden, mlp)
    if "down" in names:
        dn = make_pool(ranks, mlp, hidden, dtype, g, paged, 4, scalings=scalings,
                       rows_per_adapter=attn.rows_per_adapter)
        out["down"] = (dn, 0, mlp, hidden)
    return out


def config1(hidden=4096, seg_len=128, y0_random=False, paged=True) -> Workload:
    """fp16, 4 prefill segments of 128 tokens, 4 adapters rank 16, segment i uses adapter i."""
    g = torch.Generator(device="cpu").manual_seed(1001)
    pool = make_pool([16] * 4, hidden, hidden, torch.float16, g, paged)
    return _finish("config1", torch.float16, [0, 1, 2, 3], [seg_len] * 4, None,
                   {"q": (pool, 0, hidden, hidden)}, g, y0_random)


def config2(hidden=4096, n_tokens=256, n_adapters=64, rank=16, y0_random=True, paged=True,
            sort_ids=False, alpha_scaling=False) -> Workload:
    """fp16 decode: one token per request, Zipf(0.6) adapter ids over 64 rank-16 adapters."""
    g = torch.Generator(device="cpu").manual_seed(1002)
    sc = [32.0 / rank] * n_adapters if alpha_scaling else None
    pool = make_pool([rank] * n_adapters, hidden, hidden, torch.float16, g, paged, scalings=sc)
    ids = zipf_ids(n_adapters, n_tokens, 0.6, g)
    if sort_ids:
        ids = torch.sort(ids).values
    return _finish("config2", torch.float16, ids, [1] * n_tokens, None,
                   {"q": (pool, 0, hidden, hidden)}, g, y0_random)


def config3(hidden=4096, mlp=11008, len_div=1, n_decode=192, y0_random=True, paged=True,
            targets=("q", "k", "v", "o", "up", "down")) -> Workload:
    """bf16 mixed ragged batch: 8 prefill segments U[32,1024] + 192 decode tokens; 32 adapters
    with ranks drawn from {8,16,32,64}; Zipf(0.8) adapter ids."""
    g = torch.Generator(device="cpu").manual_seed(1003)
    lens = torch.randint(32, 1025, (8,), generator=g).tolist()
    lens = [max(1, l // len_div) for l in lens]
    ranks = [[8, 16, 32, 64][i] for i in torch.randint(0, 4, (32,), generator=g).tolist()]
    req_ids = zipf_ids(32, 8 + n_decode, 0.8, g)
    pools = _layer_pools(ranks, hidden, mlp, torch.bfloat16, g, targets, paged)
    return _finish("config3", torch.bfloat16, req_ids, lens + [1] * n_decode, None, pools, g, y0_random)


def config4(hidden=4096, mlp=11008, len_div=1, n_req=16, y0_random=True, paged=True,
            targets=("q", "k", "v", "o", "gate", "up", "down")) -> Workload:
    """bf16 vision-token-heavy prefill: 16 requests of 256 image tokens (x scaled by 4) followed
    by U[16,128] text tokens; 16 adapters rank 64, request i uses adapter i."""
    g = torch.Generator(device="cpu").manual_seed(1004)
    text = torch.randint(16, 129, (n_req,), generator=g).tolist()
    img = max(1, 256 // len_div)
    text = [max(1, t // len_div) for t in text]
    scale = torch.cat([torch.cat((torch.full((img,), 4.0), torch.ones(t))) for t in text])
    pools = _layer_pools([64] * n_req, hidden, mlp, torch.bfloat16, g, targets, paged)
    return _finish("config4", torch.bfloat16, list(range(n_req)), [img + t for t in text], scale,
                   pools, g, y0_random)


def config5_layer(hidden=4096, mlp=11008, len_div=1, n_decode=128, n_adapters=64, y0_random=True,
                  paged=True, targets=("q", "k", "v", "o", "gate", "up", "down")) -> Workload:
    """bf16, one decoder layer's LoRA work of the 7B-shape step: 128 decode tokens + 2 prefill
    requests of 512 tokens; 64 resident adapters with ranks from {16,32,64}; Zipf(0.8)."""
    g = torch.Generator(device="cpu").manual_seed(1005)
    ranks = [[16, 32, 64][i] for i in torch.randint(0, 3, (n_adapters,), generator=g).tolist()]
    req_ids = zipf_ids(n_adapters, n_decode + 2, 0.8, g)
    pools = _layer_pools(ranks, hidden, mlp, torch.bfloat16, g, targets, paged)
    pre = max(1, 512 // len_div)
    return _finish("config5", torch.bfloat16, req_ids, [1] * n_decode + [pre, pre], None, pools, g,
                   y0_random)


def decode_layer(hidden=4096, mlp=11008, n_tokens=256, n_adapters=64, rank=16, y0_random=True, paged=True,
                 targets=("q", "k", "v", "o", "gate", "up", "down")) -> Workload:
    """The decode batch of configuration 2 (one token per request, Zipf(0.6) over 64 rank-16 adapters, fp16) with
    LoRA on all seven projections of a decoder layer: what a decode-only serving step applies per layer."""
    g = torch.Generator(device="cpu").manual_seed(1002)
    req_ids = zipf_ids(n_adapters, n_tokens, 0.6, g)
    pools = _layer_pools([rank] * n_adapters, hidden, mlp, torch.float16, g, targets, paged)
    return _finish("decode_layer", torch.float16, req_ids, [1] * n_tokens, None, pools, g, y0_random)


CONFIGS = {1: config1, 2: config2, 3: config3, 4: config4, 5: config5_layer}
