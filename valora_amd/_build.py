"""Build recipe of ``libmlora.so`` (the HIP kernels + C ABI) for gfx950.

``hipcc`` cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
The library is built in-tree (``valora_amd/libmlora.so``) and links only against the HIP
runtime -- no torch, no pybind.
"""
from __future__ import annotations

import os
import shutil
import subprocess
from typing import List

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
SOURCES = ["api.hip", "tiles.hip", "plan.hip", "shrink.hip", "expand.hip", "decode.hip", "pool.hip", "merge.hip"]
TABLE_JSON = os.path.join(HERE, "tile_table.json")
TABLE_INC = os.path.join(CSRC, "tile_table_gen.inc")
LIB_PATH = os.path.join(HERE, "libmlora.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the ROCm toolchain is required to build libmlora.so")
    return exe


def command() -> List[str]:
    return ([hipcc()] + HIPCC_FLAGS +
            ["-I", os.path.join(ROOT, "include"), "-I", CSRC] +
            [os.path.join(CSRC, s) for s in SOURCES] +
            ["-Wl,-rpath,/opt/rocm/lib", "-o", LIB_PATH])


def generate_tile_table() -> str:
    """``tile_table.json`` (the measured entries, written by ``python -m valora_amd.tune_tiles``) as the C
    initialiser list ``csrc/tiles.hip`` includes: one ``{tokens, rank, hidden, adapters, bm_shrink, ksplit,
    bm_expand, flags}`` row per entry, flags = 1 (expand sums the K chunks) | 2 (one launch)."""
    import json
    with open(TABLE_JSON) as f:
        entries = json.load(f)["entries"]
    rows = []
    for key in sorted(entries, key=lambda k: tuple(int(p) for p in k.split(":"))):
        t, r, h, a = (int(p) for p in key.split(":"))
        v = entries[key]
        flags = (1 if v.get("reduce_in_expand") or v.get("one_launch") else 0) | (2 if v.get("one_launch") else 0)
        rows.append(f"  {{{t}, {r}, {h}, {a}, {int(v['bm_shrink'])}, {int(v['ksplit'])}, {int(v['bm_expand'])}, {flags}}},")
    text = "// generated from valora_amd/tile_table.json by valora_amd/_build.py -- do not edit\n" + "\n".join(rows) + "\n"
    if not os.path.exists(TABLE_INC) or open(TABLE_INC).read() != text:
        with open(TABLE_INC, "w") as f:
            f.write(text)
    return TABLE_INC


def build(verbose: bool = False) -> str:
    generate_tile_table()
    cmd = command()
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is expected
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + err)
    if verbose and err.strip():
        print(err)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
