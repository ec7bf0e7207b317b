"""Fill ``tile_table.json`` by measurement on the GPU at hand.

The reference ships a hand-collected dictionary of CUTLASS tile shapes for an A100
(valora/models/peft/lora_unordered_batch_infer.py:25-172); this is the tool that produces the
equivalent table here.  For every shape of a grid (tokens x resident adapters x rank x hidden) it
builds a synthetic batch, times the whole op with HIP-graph replays for every (shrink tile height,
split-K, who sums the split-K chunks) triple and then for every expand tile height, and writes the
winner under the key ``tile_table.key`` gives that shape.  Keys already in the table are kept unless
``--overwrite`` is given; the keys the table lists as ``protected`` (the entries of the benchmark
configurations, tuned on the real workloads) are kept even then.

    python -m valora_amd.tune_tiles [--overwrite] [--hidden 4096 11008] [--out FILE]
"""
from __future__ import annotations

import argparse
import itertools
import json
import time

import torch

from . import tile_table as tt
from . import workloads as W
from .plan import LoraPlan


def _time(fn, reps=30, warm=3) -> float:
    """Average microseconds of fn() from HIP events around graph replays on a side stream."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            fn()
        for _ in range(warm):
            g.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
    torch.cuda.current_stream().wait_stream(s)
    return e0.elapsed_time(e1) * 1e3 / reps


def down_projection_width(hidden: int) -> int:
    """Output width of the target whose INPUT is `hidden` wide when that is an MLP width (a down projection back to
    the model width: 11008 / 13824 / 14336 -> 4096 or 5120-ish, 28672 -> 8192); a model width maps to itself."""
    return hidden if hidden <= 8192 else 4096 if hidden < 20000 else 8192


def synthetic_batch(n_tokens: int, n_adapters: int, rank: int, hidden: int, dtype, seed: int, h_out: int = 0):
    """Decode-like (one token per request) up to 1024 tokens; above, requests of 128 tokens, or shorter ones where
    that many would be fewer than the adapter bucket stands for (2048 tokens over 128 adapters: 16-token requests,
    the decode-heavy mix of a continuous batch); adapters drawn Zipf(0.7) per request."""
    g = torch.Generator().manual_seed(seed)
    req_len = 1 if n_tokens <= 1024 else min(128, max(1, n_tokens // max(1, n_adapters)))
    n_req = max(1, n_tokens // req_len)
    req_ids = W.zipf_ids(n_adapters, n_req, 0.7, g)
    ids = torch.repeat_interleave(req_ids, req_len)
    pool = W.make_pool([rank] * n_adapters, hidden, h_out or hidden, dtype, g, paged=True)
    x = torch.randn(ids.numel(), hidden, generator=g).to(dtype)
    return ids, pool, x


def tune_shape(dev, n_tokens, n_adapters, rank, hidden, dtype=torch.float16, copies=4):
    """Joint search: every (shrink tile height, split-K, who sums the chunks) triple is timed as the
    whole op (shrink + expand) with a middle expand tile, then the expand tile height is swept at the
    winner.  Timing the shrink alone would miss that summing in the expand costs the expand, not the shrink."""
    ids, pool, x = synthetic_batch(n_tokens, n_adapters, rank, hidden, dtype, seed=n_tokens + n_adapters + rank)
    ids, x, p = ids.to(dev), x.to(dev), pool.to(dev)
    ys = [torch.zeros(ids.numel(), hidden, dtype=dtype, device=dev) for _ in range(copies)]
    idx = (p.a_start, p.a_len, p.a_loc)
    # a candidate replaces the current best only when it is clearly faster, so ties go to the earlier
    # (smaller, more common) setting instead of to measurement noise
    better = lambda us, best: best is None or us < 0.97 * best[0]

    def op_us(bm, ks, be, rie):
        plan = LoraPlan(ids, p.a_start, p.a_len, rank, hidden=hidden, bm_shrink=bm, ksplit=ks, bm_expand=be,
                        reduce_in_expand=rie)
        return _time(lambda: [plan.apply(y, x, p.key_buffer, p.value_buffer, *idx, 0, p.a_scaling)
                              for y in ys]) / copies

    heights = (16, 32) if n_tokens <= 256 else (16, 32, 64, 128) if n_tokens <= 4096 else (16, 32, 64, 128, 256)
    splits = (4, 8, 16, 32, 2, 1) if n_tokens <= 1024 else (4, 8, 16, 2, 1)
    be0 = 16 if n_tokens <= 1024 else 64
    best = None
    for bm, ks, rie in itertools.product(heights, splits, (False, True)):
        if (rank > 64 and bm in (64, 256)) or (rie and ks == 1) or ks * 128 > hidden:
            continue
        if rie and n_tokens > 4096:        # the partials are re-read once per column chunk: never pays there
            continue
        us = op_us(bm, ks, be0, rie)
        if better(us, best):
            best = (us, bm, ks, rie)
    _, bm, ks, rie = best
    best_e = None
    for be in EXPAND_HEIGHTS if n_tokens > 1024 else (16, 32, 64, 128, 256):
        us = op_us(bm, ks, be, rie)
        if better(us, best_e):
            best_e = (us, be)
    return {"bm_shrink": bm, "ksplit": ks, "bm_expand": best_e[1], "reduce_in_expand": bool(rie)}, best_e[0]


EXPAND_HEIGHTS = (16, 32, 48, 64, 96, 128, 192, 256)


def tune_expand_height(dev, n_tokens, n_adapters, rank, hidden, entry, dtype=torch.float16, copies=4):
    """The expand tile height of an existing entry swept again over EXPAND_HEIGHTS (shrink tiles, split-K and who
    sums the chunks stay): returns the entry to keep, its time and the old entry's time."""
    ids, pool, x = synthetic_batch(n_tokens, n_adapters, rank, hidden, dtype, seed=n_tokens + n_adapters + rank)
    ids, x, p = ids.to(dev), x.to(dev), pool.to(dev)
    ys = [torch.zeros(ids.numel(), hidden, dtype=dtype, device=dev) for _ in range(copies)]
    idx = (p.a_start, p.a_len, p.a_loc)

    def op_us(be):
        plan = LoraPlan(ids, p.a_start, p.a_len, rank, hidden=hidden, bm_shrink=entry["bm_shrink"], ksplit=entry["ksplit"],
                        bm_expand=be, reduce_in_expand=entry.get("reduce_in_expand", False), one_launch=False)
        return _time(lambda: [plan.apply(y, x, p.key_buffer, p.value_buffer, *idx, 0, p.a_scaling)
                              for y in ys]) / copies

    old = op_us(entry["bm_expand"])
    best = (old, entry["bm_expand"])
    for be in EXPAND_HEIGHTS:
        if be == entry["bm_expand"]:
            continue
        us = op_us(be)
        if us < 0.97 * best[0]:
            best = (us, be)
    new = dict(entry)
    new["bm_expand"] = best[1]
    return new, best[0], old


def tune_tall_shrink(dev, n_tokens, n_adapters, rank, hidden, entry, dtype=torch.float16, copies=4):
    """Does a 256-token shrink tile (half the re-reads of A, one workgroup per compute unit) beat an entry that uses
    128-token tiles?  Split-K 4 and 8 are tried with the entry's expand tile; returns the entry to keep and both times."""
    ids, pool, x = synthetic_batch(n_tokens, n_adapters, rank, hidden, dtype, seed=n_tokens + n_adapters + rank)
    ids, x, p = ids.to(dev), x.to(dev), pool.to(dev)
    ys = [torch.zeros(ids.numel(), hidden, dtype=dtype, device=dev) for _ in range(copies)]
    idx = (p.a_start, p.a_len, p.a_loc)

    def op_us(bm, ks):
        plan = LoraPlan(ids, p.a_start, p.a_len, rank, hidden=hidden, bm_shrink=bm, ksplit=ks, bm_expand=entry["bm_expand"],
                        reduce_in_expand=False, one_launch=False)
        return _time(lambda: [plan.apply(y, x, p.key_buffer, p.value_buffer, *idx, 0, p.a_scaling)
                              for y in ys]) / copies

    old = op_us(entry["bm_shrink"], entry["ksplit"])
    best = (old, entry["bm_shrink"], entry["ksplit"])
    for ks in (4, 8, 2):
        if ks * 128 > hidden:
            continue
        us = op_us(256, ks)
        if us < 0.97 * best[0]:
            best = (us, 256, ks)
    new = dict(entry)
    new["bm_shrink"], new["ksplit"] = best[1], best[2]
    return new, best[0], old


def tune_one_launch(dev, n_tokens, n_adapters, rank, hidden, entry, dtype=torch.float16, copies=4):
    """Does the one-launch op (shrink and expand items of one grid, 16-token tiles) beat the two-launch entry of
    this shape?  Returns the entry to keep and both timings.  Only decode-like shapes qualify: rank <= 64.  The
    library runs a call with more than 16 expand items per tile as two launches whatever the entry says, so an
    MLP-wide `hidden` is measured as what it is the input of, a down projection (to a 4096- or 8192-wide output)."""
    h_out = down_projection_width(hidden)
    ids, pool, x = synthetic_batch(n_tokens, n_adapters, rank, hidden, dtype, seed=n_tokens + n_adapters + rank, h_out=h_out)
    ids, x, p = ids.to(dev), x.to(dev), pool.to(dev)
    ys = [torch.zeros(ids.numel(), h_out, dtype=dtype, device=dev) for _ in range(copies)]
    idx = (p.a_start, p.a_len, p.a_loc)

    def op_us(**kw):
        plan = LoraPlan(ids, p.a_start, p.a_len, rank, hidden=hidden, **kw)
        return _time(lambda: [plan.apply(y, x, p.key_buffer, p.value_buffer, *idx, 0, p.a_scaling)
                              for y in ys]) / copies

    two = op_us(bm_shrink=entry["bm_shrink"], ksplit=entry["ksplit"], bm_expand=entry["bm_expand"],
                reduce_in_expand=entry.get("reduce_in_expand", False), one_launch=False)
    best = None
    for ks in (4, 2, 3, 6, 8):
        if ks * 128 > hidden:
            continue
        us = op_us(ksplit=ks, one_launch=True)
        if best is None or us < 0.97 * best[0]:
            best = (us, ks)
    if best[0] < 0.97 * two:
        return {"bm_shrink": 16, "ksplit": best[1], "bm_expand": 16, "reduce_in_expand": True, "one_launch": True}, two, best[0]
    keep = dict(entry)
    keep.pop("one_launch", None)
    return keep, two, best[0]


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--overwrite", action="store_true")
    ap.add_argument("--hidden", type=int, nargs="+", default=[4096])
    ap.add_argument("--tokens", type=int, nargs="+", default=[8, 64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384])
    ap.add_argument("--adapters", type=int, nargs="+", default=[1, 8, 32, 64, 128])
    ap.add_argument("--ranks", type=int, nargs="+", default=list(tt.RANK_BUCKETS))
    ap.add_argument("--out", default=tt.TABLE_PATH)
    ap.add_argument("--one-launch", action="store_true",
                    help="revisit the existing entries of decode-like shapes (<= 2048 tokens, rank <= 64; the protected "
                         "ones too) and mark those where the one-launch op is faster than the entry's two launches")
    ap.add_argument("--tall-shrink", action="store_true",
                    help="revisit the existing entries above 4096 tokens that use 128-token shrink tiles (rank <= 64, summed "
                         "by the reduce launch): 256-token tiles where they are faster; protected entries stay")
    ap.add_argument("--expand-heights", action="store_true",
                    help="revisit the expand tile height of the existing entries above 1024 tokens over the finer list "
                         "(48, 96 and 192 tokens as well); protected and one-launch entries stay")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("tune_tiles needs a GPU")
    dev = torch.device("cuda:0")
    with open(tt.TABLE_PATH) as f:
        table = json.load(f)
    entries = table["entries"]
    t0 = time.time()
    for hidden, n_tokens, n_adapters, rank in itertools.product(args.hidden, args.tokens, args.adapters, args.ranks):
        k = tt.key(n_tokens, rank, hidden, n_adapters)
        if args.tall_shrink:
            e = entries.get(k)
            if (e and n_tokens > 4096 and rank <= 64 and e["bm_shrink"] == 128 and not e.get("reduce_in_expand")
                    and k not in table.get("protected", [])):
                entries[k], us, old = tune_tall_shrink(dev, n_tokens, min(n_adapters, max(1, n_tokens)), rank, hidden, e)
                print(f"{k:24s} shrink tile 128 x {e['ksplit']} ({old:.1f} us) -> {entries[k]['bm_shrink']} x "
                      f"{entries[k]['ksplit']} ({us:.1f} us)  [{time.time() - t0:.0f} s]", flush=True)
                torch.cuda.empty_cache()
                with open(args.out, "w") as f:
                    json.dump(table, f, indent=1)
            continue
        if args.expand_heights:
            e = entries.get(k)
            if e and n_tokens > 1024 and not e.get("one_launch") and k not in table.get("protected", []):
                entries[k], us, old = tune_expand_height(dev, n_tokens, min(n_adapters, max(1, n_tokens)), rank, hidden, e)
                print(f"{k:24s} expand tile {e['bm_expand']} ({old:.1f} us) -> {entries[k]['bm_expand']} ({us:.1f} us)  "
                      f"[{time.time() - t0:.0f} s]", flush=True)
                torch.cuda.empty_cache()
                with open(args.out, "w") as f:
                    json.dump(table, f, indent=1)
            continue
        if args.one_launch:
            if k in entries and n_tokens <= 2048 and rank <= 64:
                new, two, one = tune_one_launch(dev, n_tokens, min(n_adapters, max(1, n_tokens)), rank, hidden, entries[k])
                # a protected entry was tuned on its real workload: the synthetic batch (which may not fit the
                # device as one grid where the real one does) can add the mark there, never take it away
                if not (k in table.get("protected", []) and entries[k].get("one_launch") and not new.get("one_launch")):
                    entries[k] = new
                print(f"{k:24s} two launches {two:.1f} us, one launch {one:.1f} us -> {entries[k]}  "
                      f"[{time.time() - t0:.0f} s]", flush=True)
                torch.cuda.empty_cache()
            continue
        if k in entries and (not args.overwrite or k in table.get("protected", [])):
            print(f"{k:24s} kept {entries[k]}", flush=True)
            continue
        cfg, us = tune_shape(dev, n_tokens, min(n_adapters, max(1, n_tokens)), rank, hidden)
        entries[k] = cfg
        print(f"{k:24s} {cfg}  {us:.1f} us/op  [{time.time() - t0:.0f} s]", flush=True)
        torch.cuda.empty_cache()
        with open(args.out, "w") as f:      # after every shape: a long sweep that is cut short keeps what it has
            json.dump(table, f, indent=1)
    with open(args.out, "w") as f:
        json.dump(table, f, indent=1)
    print("wrote", args.out)


if __name__ == "__main__":
    main()
