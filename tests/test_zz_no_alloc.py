"""GPU: the entry point that allocates nothing (``mlora_dispatch_bgmv_static``) against
``mlora_dispatch_bgmv`` with a caller-owned workspace and against the oracle: same bits as the former, the
latter's tolerance, two calls in a row on the shared built-in workspace (the second with a smaller batch), and
the size limit."""
import pytest
import torch

from oracle import lora_oracle as O
from tests._util import assert_parity
from valora_amd import _lib, workloads as W

pytestmark = pytest.mark.gpu


def _pair(L, dev, pool, ids, x, narrow, v, y0, slot, dtype):
    """Shrink and expand through both entry points; returns ((delta, y) static, (delta, y) with workspace)."""
    T, h = x.shape
    code = _lib.dtype_code(dtype)
    stream = _lib.current_stream(dev)
    pk = _lib.make_pool(pool.key_buffer, pool.a_start, pool.a_len, pool.a_loc, h, 4)
    pv = _lib.make_pool(pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, h, 4)
    ws = torch.empty(int(L.mlora_workspace_bytes(T, pool.a_start.numel(), narrow)), dtype=torch.uint8, device=dev)
    out = []
    for static in (True, False):
        delta = torch.full((T, narrow), 0.5, dtype=dtype, device=dev)
        y = y0.clone()
        for (yy, xx, p, h_in, h_out) in ((delta, x, pk, h, narrow), (y, v, pv, narrow, h)):
            if static:
                rc = L.mlora_dispatch_bgmv_static(stream, _lib.ptr(yy), _lib.ptr(xx), p, _lib.ptr(ids), slot,
                                                  _lib.ptr(pool.a_scaling), T, h_in, h_out, code)
            else:
                rc = L.mlora_dispatch_bgmv(stream, _lib.ptr(yy), _lib.ptr(xx), p, _lib.ptr(ids), slot,
                                           _lib.ptr(pool.a_scaling), T, h_in, h_out, code, _lib.ptr(ws), ws.numel(), None)
            _lib.check(rc)
        torch.cuda.synchronize()
        out.append((delta.cpu(), y.cpu()))
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_static_workspace_entry_point_matches_dispatch_bgmv(dev, dtype):
    L = _lib.lib()
    g = torch.Generator().manual_seed(7)
    h, ranks = 1024, [16, 8, 32, 16, 64, 8]
    narrow = max(ranks)
    pool = W.make_pool(ranks, h, h, dtype, g, True, std=0.05, scalings=[1.0, 0.5, 2.0, 1.5, 0.25, 1.0]).to(dev)
    # two calls in a row on the same built-in workspace: a large batch, then a smaller one whose plan and
    # partials occupy only the head of what the first call left behind
    for T in (1500, 37):
        ids = torch.randint(-1, len(ranks), (T,), generator=g).to(dev)
        x = torch.randn(T, h, generator=g).to(dtype).to(dev)
        v = torch.randn(T, narrow, generator=g).to(dtype).to(dev)
        y0 = torch.randn(T, h, generator=g).to(dtype).to(dev)
        (d_s, y_s), (d_w, y_w) = _pair(L, dev, pool, ids, x, narrow, v, y0, 2, dtype)
        assert torch.equal(d_s, d_w), f"T={T}: shrink differs"
        assert torch.equal(y_s, y_w), f"T={T}: expand differs"
        assert not torch.equal(y_s, y0.cpu()) and bool((d_s != 0.5).any()), "the calls did something"
        # and the numbers are the operator's (valora/csrc/bgmv/bgmv_impl.cuh:14-207), not merely the sibling's
        pc, idc = pool.to("cpu"), ids.cpu()
        want_d = O.bgmv_shrink(torch.full((T, narrow), 0.5, dtype=dtype), x.cpu(), pc.key_buffer, pc.a_start, pc.a_len,
                               pc.a_loc, idc, 2)
        want_y = O.bgmv_expand(y0.cpu(), v.cpu(), pc.value_buffer, pc.a_start, pc.a_len, pc.a_loc, idc, 2, pc.a_scaling)
        assert_parity(d_s, want_d, f"static workspace, T={T}: shrink vs oracle")
        assert_parity(y_s, want_y, f"static workspace, T={T}: expand vs oracle")


def test_static_workspace_size_limit(dev):
    """A batch whose workspace exceeds the built-in one is refused before anything is launched."""
    L = _lib.lib()
    dtype = torch.float16
    g = torch.Generator().manual_seed(3)
    pool = W.make_pool([128, 128], 256, 256, dtype, g, False, std=0.05).to(dev)
    T = 200000
    assert int(L.mlora_workspace_bytes(T, 2, 128)) > (16 << 20)
    ids = torch.zeros(T, dtype=torch.long, device=dev)
    x = torch.zeros(T, 256, dtype=dtype, device=dev)
    delta = torch.full((T, 128), 3.0, dtype=dtype, device=dev)
    pk = _lib.make_pool(pool.key_buffer, pool.a_start, pool.a_len, pool.a_loc, 256, 4)
    rc = L.mlora_dispatch_bgmv_static(_lib.current_stream(dev), _lib.ptr(delta), _lib.ptr(x), pk, _lib.ptr(ids), 0,
                                      _lib.ptr(pool.a_scaling), T, 256, 128, 0)
    assert rc == -3 and b"needs" in L.mlora_last_error() and b"built-in" in L.mlora_last_error()
    torch.cuda.synchronize()
    assert bool((delta == 3.0).all())
