"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares,
its size queries and argument validation work without a GPU, and the Python shims reject what
the reference's extensions reject (valora/csrc/lora_ops.cc:79-98,124-125)."""
import ctypes
import os
import re

import pytest
import torch

from valora_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "mlora.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mlora_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _lib.lib()
    names = _declared()
    assert len(names) >= 16
    for n in names:
        assert hasattr(L, n), n
    assert sorted(_lib.SYMBOLS) == names
    assert L.mlora_version() >= 100


def test_size_queries():
    L = _lib.lib()
    assert L.mlora_plan_bytes(0, 0) > 0
    assert L.mlora_plan_bytes(256, 64) >= (32 + 3 * 256 + 2 * 8 * (16 + 64) + 4 * 64) * 4
    # v (T) + fp32 partials, whose rows are whole 128-byte lines (32 floats for rank 16)
    assert L.mlora_scratch_bytes(256, 16, 8) == 256 * 16 * 2 + 8 * 256 * 32 * 4
    assert L.mlora_scratch_bytes(256, 64, 8) == 256 * 64 * 2 + 8 * 256 * 64 * 4
    assert L.mlora_scratch_bytes(16, 8, 1) == 16 * 16 * 2       # rows padded to 16 columns, no partials
    assert L.mlora_workspace_bytes(256, 64, 16) > L.mlora_plan_bytes(256, 64)
    assert L.mlora_plan_bytes(-1, 3) == 0


def test_argument_validation_needs_no_gpu():
    L = _lib.lib()
    plan = _lib.Plan(None, 0, 0, 0, 0, 0)
    assert L.mlora_build_plan(None, plan, None, 4, None, None, 0, 4, 0, 0) == -1
    assert b"plan buffer is null" in L.mlora_last_error()
    buf = ctypes.create_string_buffer(1 << 16)
    addr = (ctypes.addressof(buf) + 255) & ~255
    plan = _lib.Plan(addr, 64, 0, 0, 0, 0)
    ids = (ctypes.c_int64 * 4)()
    a = (ctypes.c_int64 * 2)()
    rc = L.mlora_build_plan(None, plan, ctypes.addressof(ids), 4, ctypes.addressof(a), ctypes.addressof(a), 2, 4, 16, 32)
    assert rc == -3 and b"plan buffer has 64 bytes" in L.mlora_last_error()
    plan = _lib.Plan(addr, 1 << 15, 0, 0, 0, 0)
    rc = L.mlora_build_plan(None, plan, ctypes.addressof(ids), 4, ctypes.addressof(a), ctypes.addressof(a), 2, 4, 48, 32)
    assert rc == -2 and b"bm_shrink=48" in L.mlora_last_error()
    rc = L.mlora_build_plan(None, plan, ctypes.addressof(ids), 4, ctypes.addressof(a), ctypes.addressof(a), 9000, 4, 16, 32)
    assert rc == -2 and b"n_adapters=9000" in L.mlora_last_error()
    # dims outside what any kernel handles -> the reference's message shape
    pool = _lib.Pool(addr, 8, ctypes.addressof(a), ctypes.addressof(a), ctypes.addressof(a), 2, 2, 4)
    rc = L.mlora_dispatch_bgmv(None, addr, addr, pool, ctypes.addressof(ids), 0, addr, 4, 70000, 16, 0, addr, 1 << 15, None)
    assert rc == -2 and L.mlora_last_error().startswith(b"No suitable kernel. h_in=70000 h_out=16 dtype=Half")
    rc = L.mlora_dispatch_bgmv(None, addr, addr, pool, ctypes.addressof(ids), 0, addr, 4, 4096, 12, 1, addr, 1 << 15, None)
    assert rc == -2 and b"dtype=BFloat16" in L.mlora_last_error()
    rc = L.mlora_dispatch_bgmv(None, addr, addr, pool, ctypes.addressof(ids), 0, addr, 4, 4096, 16, 7, addr, 1 << 15, None)
    assert rc == -2
    rc = L.mlora_dispatch_bgmv(None, addr, addr, pool, ctypes.addressof(ids), 5, addr, 4, 4096, 16, 0, addr, 1 << 15, None)
    assert rc == -1 and b"qkvo=5" in L.mlora_last_error()


def test_shim_rejects_what_the_reference_rejects():
    from valora_amd.kernels import dispatch_bgmv
    y = torch.zeros(4, 16, dtype=torch.float16)
    x = torch.zeros(4, 64, dtype=torch.float16)
    w = torch.zeros(8, 2, 32, dtype=torch.float16)
    i64 = torch.zeros(4, dtype=torch.long)
    with pytest.raises(RuntimeError, match="y must be a CUDA tensor"):
        dispatch_bgmv(y, x, w, i64, i64, i64, i64, 0, y)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmlora.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()


def test_tile_lookup_through_the_c_abi_agrees_with_the_json_table():
    """Every entry of tile_table.json comes back from mlora_tile_lookup for a shape inside its bucket: the
    table compiled into the library is the one the tuner wrote."""
    import json
    from valora_amd import tile_table as tt
    L = _lib.lib()
    with open(tt.TABLE_PATH) as f:
        entries = json.load(f)["entries"]
    assert len(entries) >= 100
    for key, v in entries.items():
        t, r, h, a = (int(p) for p in key.split(":"))
        c = _lib.TileConfig()
        assert L.mlora_tile_lookup(t, r, h, a, c) == 0
        want_flags = (1 if v.get("reduce_in_expand") or v.get("one_launch") else 0) | (2 if v.get("one_launch") and r <= 64 else 0)
        bm_s = 32 if (r > 64 and v["bm_shrink"] == 64) else v["bm_shrink"]
        assert (c.bm_shrink, c.ksplit, c.bm_expand, c.flags) == (bm_s, v["ksplit"], v["bm_expand"], want_flags), key
        assert tt.key(t, r, h, a) == key
    c = _lib.TileConfig()
    assert L.mlora_tile_lookup(-1, 16, 4096, 8, c) == -1 and L.mlora_tile_lookup(8, 16, 4096, 8, None) == -1


def test_tile_table_lookup_and_fallback():
    from valora_amd import tile_table as tt
    cfg = tt.lookup(256, 16, 4096, 64)
    assert cfg.bm_shrink in (16, 32, 64, 128, 256) and 1 <= cfg.ksplit <= 64 and cfg.bm_expand % 16 == 0
    fb = tt.fallback(100000, 128, 4096, 4)          # long runs per adapter -> LDS-staged 128-token tiles
    assert fb.bm_shrink == 128 and fb.ksplit >= 1 and not fb.reduce_in_expand
    fb = tt.fallback(300, 64, 4096, 200)            # decode-like -> direct 16-token tiles, expand sums the chunks
    assert fb.bm_shrink == 16 and fb.reduce_in_expand
    assert tt.key(300, 16, 4096, 64) == "512:16:4096:64" and tt.key(600, 16, 4096, 100) == "1024:16:4096:128"
    assert tt.key(300, 24, 4096, 65) == "512:32:4096:128" and tt.key(1, 8, 4096, 1) == "8:16:4096:1"
    for rank in (8, 40, 128):                       # every table entry is a configuration the kernels take
        for T in (1, 300, 5000, 100000):
            c = tt.lookup(T, rank, 4096, 16)
            assert c.bm_shrink in (16, 32, 64, 128, 256) and not (rank > 64 and c.bm_shrink in (64, 256))
            assert 1 <= c.ksplit <= 64 and c.bm_expand % 16 == 0 and 16 <= c.bm_expand <= 256


def test_install_aliases_registers_the_reference_import_names():
    import importlib
    import sys
    import types
    import valora_amd
    names = ("valora._kernels", "atmm_ops", "valora.models.peft.triton_kernel.lora.lora_prefill")
    saved = {n: sys.modules.pop(n, None) for n in names}
    try:
        valora_amd.install_aliases()
        assert importlib.import_module("atmm_ops").dispatch_bgmv is valora_amd.atmm_ops.dispatch_bgmv
        assert sys.modules["valora._kernels"].dispatch_bgmv is valora_amd.kernels.dispatch_bgmv
        m = sys.modules["valora.models.peft.triton_kernel.lora.lora_prefill"]
        assert m.lora_get_qkvo_fwd_shrink is valora_amd.lora_prefill.lora_get_qkvo_fwd_shrink
        valora_amd.install_aliases()                      # idempotent
        sys.modules["atmm_ops"] = types.ModuleType("atmm_ops")
        with pytest.raises(RuntimeError, match="already imported"):
            valora_amd.install_aliases()
    finally:
        for n, m in saved.items():
            sys.modules.pop(n, None)
            if m is not None:
                sys.modules[n] = m


C_PROGRAM = r"""
#include <stdio.h>
#include <string.h>
#include "mlora.h"
int main(void) {
  mlora_tile_config c;
  mlora_plan plan;
  memset(&plan, 0, sizeof plan);
  if (mlora_version() <= 0) return 1;
  if (mlora_plan_bytes(256, 64) == 0 || mlora_workspace_bytes(256, 64, 16) == 0) return 2;
  if (mlora_tile_lookup(256, 16, 4096, 64, &c) != MLORA_OK || c.bm_shrink <= 0) return 3;
  /* a call the library must refuse before it touches a device */
  if (mlora_build_plan(NULL, &plan, NULL, 8, NULL, NULL, 0, 4, 16, 16) == MLORA_OK) return 4;
  if (mlora_last_error() == NULL || strlen(mlora_last_error()) == 0) return 5;
  printf("ok %d\n", mlora_version());
  return 0;
}
"""


def test_header_is_plain_c_and_a_c_program_links_against_the_library(tmp_path):
    """include/mlora.h is the boundary a foreign-language binding is written against: it has to compile as
    C99 and as C++ without warnings, and a C program has to link against libmlora.so and get answers from the
    calls that need no GPU."""
    import shutil
    import subprocess
    gcc, gxx = shutil.which("gcc"), shutil.which("g++")
    if gcc is None or gxx is None:
        pytest.skip("no host compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    inc = os.path.join(root, "include")
    src = tmp_path / "use_mlora.c"
    src.write_text(C_PROGRAM)
    for cmd in ([gcc, "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", inc, str(src)],
                [gxx, "-std=c++11", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c++", "-I", inc, str(src)]):
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
    exe = tmp_path / "use_mlora"
    libdir = os.path.dirname(_lib.LIB_PATH)
    r = subprocess.run([gcc, "-std=c99", "-I", inc, str(src), "-L", libdir, "-lmlora", f"-Wl,-rpath,{libdir}",
                        "-Wl,-rpath,/opt/rocm/lib", "-o", str(exe)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    r = subprocess.run([str(exe)], capture_output=True, text=True)
    assert r.returncode == 0 and r.stdout.startswith("ok"), (r.returncode, r.stdout, r.stderr)
