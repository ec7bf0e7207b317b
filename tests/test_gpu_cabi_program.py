"""GPU: the C ABI driven by a program that is neither Python nor PyTorch.

``tests/cabi/cabi_gpu_check.c`` is plain C99 over the HIP runtime API and ``include/mlora.h``: it allocates with
hipMalloc, asks the library for the tile configuration, builds the plan, runs the planned op, then the reference's
two-call form (``dispatch_bgmv`` shrink into a caller-visible delta, ``dispatch_bgmv`` expand) with no plan and a
workspace.  This test writes the operands to a file, runs the program and compares what it wrote back with the
oracle -- the same bar as the tests that go through the Python host layer."""
import os
import subprocess

import numpy as np
import pytest
import torch

from oracle import lora_oracle as O
from valora_amd import workloads as W
from tests._util import assert_parity
from tests.cabi import build as cabi_build

pytestmark = pytest.mark.gpu


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy()


@pytest.mark.parametrize("T,h_in,h_out,ranks,n_slots,dtype,style", [
    (256, 4096, 4096, [16] * 64, 4, torch.float16, "zipf"),            # the headline shape (one launch)
    (77, 1024, 2048, [8, 16, 32, 64, 24], 4, torch.bfloat16, "holes"),  # mixed ranks, tokens without adapter
    (1500, 2048, 2048, [64] * 6, 1, torch.bfloat16, "runs"),            # prefill-like, split-K with its own reduce
    (1, 512, 512, [16], 2, torch.float16, "zipf"),
], ids=["decode", "mixed", "prefill", "one-token"])
def test_plain_c_caller(dev, tmp_path, T, h_in, h_out, ranks, n_slots, dtype, style):
    exe = cabi_build.EXE if os.path.exists(cabi_build.EXE) else cabi_build.build()
    g = torch.Generator().manual_seed(T + h_in)
    A, R = len(ranks), max(ranks)
    pool = W.make_pool(ranks, h_in, h_out, dtype, g, True, n_slots=n_slots, std=0.05, heads=1,
                       scalings=[0.5 + 0.25 * (i % 4) for i in range(A)])
    if style == "zipf":
        ids = W.zipf_ids(A, T, 0.6, g)
    elif style == "holes":
        ids = torch.randint(-1, A, (T,), generator=g)
    else:
        ids = torch.repeat_interleave(torch.randint(0, A, ((T + 249) // 250,), generator=g), 250)[:T]
    x = torch.randn(T, h_in, generator=g).to(dtype)
    y0 = torch.randn(T, h_out, generator=g).to(dtype)
    slot = n_slots - 1
    kb = pool.key_buffer.reshape(-1, h_in)
    vb = pool.value_buffer.reshape(-1, h_out)
    header = np.array([T, h_in, h_out, A, R, n_slots, 0 if dtype == torch.float16 else 1, slot, pool.a_loc.numel(),
                       kb.size(0), vb.size(0), 0], dtype=np.int64)
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        header.tofile(f)
        for t in (ids, pool.a_start, pool.a_len, pool.a_loc):
            t.contiguous().numpy().astype(np.int64).tofile(f)
        for t in (pool.a_scaling.to(dtype), x, y0, kb, vb):
            _bits(t).tofile(f)
    r = subprocess.run([exe, str(fin), str(fout)], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stderr
    raw = np.fromfile(fout, dtype=np.int16)
    assert raw.size == 2 * T * h_out + T * R
    as_t = lambda a, shape: torch.from_numpy(a.copy()).view(dtype).reshape(shape)
    y_plan = as_t(raw[:T * h_out], (T, h_out))
    delta = as_t(raw[T * h_out:T * h_out + T * R], (T, R))
    y_bgmv = as_t(raw[T * h_out + T * R:], (T, h_out))
    idx = (pool.a_start, pool.a_len, pool.a_loc)
    want = O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, *idx, ids, slot, pool.a_scaling, n_slots=n_slots)
    assert_parity(y_plan, want, "planned op from C")
    want_delta = O.bgmv_shrink(torch.zeros(T, R, dtype=dtype), x, pool.key_buffer, *idx, ids, slot, n_slots=n_slots)
    assert_parity(delta, want_delta, "dispatch_bgmv shrink from C")
    want2 = O.bgmv_expand(y0, delta, pool.value_buffer, *idx, ids, slot, pool.a_scaling, n_slots=n_slots)
    assert_parity(y_bgmv, want2, "dispatch_bgmv expand from C")
    none = ids < 0
    assert torch.equal(y_plan[none], y0[none]) and torch.equal(y_bgmv[none], y0[none])
