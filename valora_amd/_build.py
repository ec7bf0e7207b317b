"""Build recipe of ``libmlora.so`` (the HIP kernels + C ABI) for gfx950, and of the torch binding
above it.

``hipcc`` cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
The library is built in-tree (``valora_amd/libmlora.so``) and links only against the HIP
runtime -- no torch, no pybind.  ``valora_amd/_binding.so`` is host code only (``g++``): the
reference's op entry points as a torch extension module that calls the library through its C ABI.
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
BINDING_SRC = os.path.join(CSRC, "binding.cpp")
BINDING_PATH = os.path.join(HERE, "_binding.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first 8 dwords of a kernel's scalar arguments arrive in registers instead of through a load of the
    # argument block (decode_kernel puts what its first dependent loads need there)
    "-mllvm", "-amdgpu-kernarg-preload-count=8",
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


def binding_command() -> List[str]:
    """``g++`` line of the torch binding: torch's and Python's headers, HIP's runtime API header (for the
    stream type), linked against libmlora.so beside it and the torch libraries the process has loaded."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension
    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        raise RuntimeError("g++ not found: it is required to build the torch binding")
    inc = cpp_extension.include_paths() + [sysconfig.get_paths()["include"], "/opt/rocm/include",
                                           os.path.join(ROOT, "include")]
    libdirs = cpp_extension.library_paths()
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    return ([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
             "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_binding",
             f"-D_GLIBCXX_USE_CXX11_ABI={abi}"] +
            [a for d in inc for a in ("-isystem", d)] + [BINDING_SRC] +
            [f"-L{d}" for d in libdirs] + [f"-L{HERE}", "-lmlora", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch",
                                           "-ltorch_python", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN"] +
            [f"-Wl,-rpath,{d}" for d in libdirs] + ["-Wl,-rpath,/opt/rocm/lib", "-o", BINDING_PATH])


def _run(cmd: List[str], what: str, verbose: bool) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; that is expected
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"{what} failed:\n" + " ".join(cmd) + "\n" + err)
    if verbose and err.strip():
        print(err)


def build(verbose: bool = False) -> str:
    generate_tile_table()
    _run(command(), "hipcc", verbose)
    _run(binding_command(), "g++ (torch binding)", verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
