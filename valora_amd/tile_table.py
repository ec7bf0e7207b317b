"""Tile-configuration table for the gfx950 LoRA kernels.

Replaces the reference's ``shape_to_config`` dictionary and ``get_config_a`` / ``get_config_b``
(valora/models/peft/lora_unordered_batch_infer.py:25-172,216-236), which map
``(n_adapters, first_seq_len, K, N)`` to CUTLASS threadblock / warp shapes tuned on an A100 and
fall back to a fixed shape for unknown keys.  Here the key is
``(token bucket, rank bucket, hidden, adapter bucket)`` and the value is what the HIP kernels can
vary: the token height of a shrink tile, the split-K factor of the shrink, who sums the split-K
chunks and the token height of an expand tile.  Entries come from sweeps on MI355X (``tile_table.json`` next to this file);
a width without entries uses those of the nearest measured width, and anything else falls back to a
rule, like the reference's fallback tuple.  The look-up itself lives in the library
(``csrc/tiles.hip``, table generated from the JSON file at build time); this module is its Python face.
"""
from __future__ import annotations

import os
from dataclasses import dataclass

_HERE = os.path.dirname(os.path.abspath(__file__))
TABLE_PATH = os.path.join(_HERE, "tile_table.json")

TOKEN_BUCKETS = (8, 64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384, 1 << 22)
ADAPTER_BUCKETS = (1, 8, 32, 64, 128, 8192)
RANK_BUCKETS = (16, 32, 64, 128)


@dataclass(frozen=True)
class TileConfig:
    bm_shrink: int   # tokens per shrink tile: 16, 32, 64 (direct loads), 128 or 256 (weights staged in LDS)
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


def _cfg(c) -> TileConfig:
    from . import _lib
    return TileConfig(int(c.bm_shrink), int(c.ksplit), int(c.bm_expand), bool(c.flags & _lib.REDUCE_IN_EXPAND),
                      bool(c.flags & _lib.ONE_LAUNCH))


def fallback(n_tokens: int, max_rank: int, hidden: int, n_adapters: int) -> TileConfig:
    """The rule a shape without a table entry gets (``mlora_tile_fallback``)."""
    from . import _lib
    c = _lib.TileConfig()
    _lib.check(_lib.lib().mlora_tile_fallback(int(n_tokens), int(max_rank), int(hidden), int(n_adapters), c))
    return _cfg(c)


def lookup(n_tokens: int, max_rank: int, hidden: int, n_adapters: int) -> TileConfig:
    """The configuration ``libmlora.so`` itself uses for this shape (``mlora_tile_lookup``): the table is
    compiled into the library, so the Python host layer and any other caller of the C ABI agree.  After
    ``tune_tiles`` has rewritten ``tile_table.json`` the library has to be rebuilt
    (``python -m valora_amd._build``) for new entries to take effect."""
    from . import _lib
    c = _lib.TileConfig()
    _lib.check(_lib.lib().mlora_tile_lookup(int(n_tokens), int(max_rank), int(hidden), int(n_adapters), c))
    return _cfg(c)
