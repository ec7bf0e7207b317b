"""Tile-configuration table for the gfx950 LoRA kernels.

Replaces the reference's ``shape_to_config`` dictionary and ``get_config_a`` / ``get_config_b``
(valora/models/peft/lora_unordered_batch_infer.py:25-172,216-236), which map
``(n_adapters, first_seq_len, K, N)`` to CUTLASS threadblock / warp shapes tuned on an A100 and
fall back to a fixed shape for unknown keys.  Here the key is
``(token bucket, rank bucket, hidden, adapter bucket)`` and the value is what the HIP kernels can
vary: the token height of a shrink tile, the split-K factor of the shrink, who sums the split-K
chunks and the token height of an expand tile.  Entries come from sweeps on MI355X (``tile_table.json`` next to this file);
a width without entries uses those of the nearest measured width, and anything else falls back to a
rule, like the reference's fallback tuple.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass
from typing import Dict

_HERE = os.path.dirname(os.path.abspath(__file__))
TABLE_PATH = os.path.join(_HERE, "tile_table.json")

TOKEN_BUCKETS = (8, 64, 256, 1024, 4096, 16384, 1 << 22)
ADAPTER_BUCKETS = (1, 8, 32, 128, 8192)
RANK_BUCKETS = (16, 32, 64, 128)


@dataclass(frozen=True)
class TileConfig:
    bm_shrink: int   # tokens per shrink tile: 16, 32, 64 (direct loads) or 128 (weights staged in LDS)
    ksplit: int      # K-chunks the shrink is split into (partials summed by the consumer)
    bm_expand: int   # tokens per expand tile: multiple of 16 up to 256
    reduce_in_expand: bool = False  # split-K chunks summed by the expand launch (small batches)
    one_launch: bool = False        # shrink and expand as work items of one grid (decode-like batches, rank <= 64)


def _bucket(v: int, buckets) -> int:
    for b in buckets:
        if v <= b:
            return b
    return buckets[-1]


def key(n_tokens: int, max_rank: int, hidden: int, n_adapters: int) -> str:
    return (f"{_bucket(n_tokens, TOKEN_BUCKETS)}:{_bucket(max_rank, RANK_BUCKETS)}:{hidden}:"
            f"{_bucket(n_adapters, ADAPTER_BUCKETS)}")


def fallback(n_tokens: int, max_rank: int, hidden: int, n_adapters: int) -> TileConfig:
    tokens_per_adapter = n_tokens / max(1, min(n_adapters, n_tokens))
    if n_tokens > 4096 and tokens_per_adapter >= 64:
        bm_s = 128
    else:
        bm_s = 16 if n_tokens <= 1024 else 32
    tiles = max(1, min(n_tokens, -(-n_tokens // bm_s) + min(n_adapters, n_tokens)))
    ksplit = max(1, min(16, hidden // 256, -(-768 // tiles)))
    bm_e = 16 if n_tokens <= 1024 else 32 if n_tokens <= 4096 else 128
    return TileConfig(bm_s, ksplit, bm_e, n_tokens <= 1024)


_table: Dict[str, TileConfig] = {}
_hiddens: list = []      # the widths the table has entries for
_loaded = False


def _load() -> None:
    global _loaded
    _loaded = True
    if os.path.exists(TABLE_PATH):
        with open(TABLE_PATH) as f:
            raw = json.load(f)
        for k, v in raw.get("entries", {}).items():
            _table[k] = TileConfig(int(v["bm_shrink"]), int(v["ksplit"]), int(v["bm_expand"]),
                                   bool(v.get("reduce_in_expand", False)), bool(v.get("one_launch", False)))
        _hiddens[:] = sorted({int(k.split(":")[2]) for k in _table})


def lookup(n_tokens: int, max_rank: int, hidden: int, n_adapters: int) -> TileConfig:
    if not _loaded:
        _load()
    cfg = _table.get(key(n_tokens, max_rank, hidden, n_adapters))
    if cfg is None and _hiddens:
        # a width the table was not measured for: the entry of the nearest measured width (ratio-wise),
        # with the split-K factor cut to what the width can be split into
        near = min(_hiddens, key=lambda h: abs(math.log(h / max(1, hidden))))
        cfg = _table.get(key(n_tokens, max_rank, near, n_adapters))
        if cfg is not None:
            cfg = TileConfig(cfg.bm_shrink, max(1, min(cfg.ksplit, hidden // 128)), cfg.bm_expand,
                             cfg.reduce_in_expand and min(cfg.ksplit, hidden // 128) > 1,
                             cfg.one_launch and hidden >= 256)
    if cfg is None:
        return fallback(n_tokens, max_rank, hidden, n_adapters)
    if max_rank > 64 and cfg.bm_shrink == 64:     # ranks above 64 have no 64-token shrink tile
        cfg = TileConfig(32, cfg.ksplit, cfg.bm_expand, cfg.reduce_in_expand, False)
    return cfg
