"""Pins the CPU oracle (oracle/) before anything is compared against it.

The reference ships no golden vectors for this path, so the oracle is fixed by:
  * the reference-held per-token loop of test/kernel/test_kernel_correctness_multi_rank.py:57-116
    restated here with its own shapes (H=1024, ranks [8,16], 128 tokens, 2 adapters);
  * an index-literal fp64 brute force (explicit loops over the flat offsets) on tiny paged pools;
  * the independently written C restatement of the CUDA kernels' indexing (oracle/bgmv_ref.c);
  * algebraic invariants a dropped term / transposed operand / wrong slot would break;
  * hand-derived vectors for the integer segment builder (tests/golden/segments.json).
"""
import itertools
import json
import os

import numpy as np
import pytest
import torch

from oracle import bgmv_ref, lora_oracle as O
from valora_amd import workloads as W

HERE = os.path.dirname(os.path.abspath(__file__))


def _rand_case(seed, T=24, H=64, ranks=(8, 16, 8), dtype=torch.float16, paged=True, n_ids=None):
    g = torch.Generator().manual_seed(seed)
    pool = W.make_pool(list(ranks), H, H, dtype, g, paged, std=0.3)
    ids = torch.randint(0, len(ranks), (T,), generator=g)
    x = torch.randn(T, H, generator=g).to(dtype)
    y0 = torch.randn(T, H, generator=g).to(dtype)
    R = max(ranks)
    v = torch.randn(T, R, generator=g).to(dtype)
    scales = (torch.rand(len(ranks), generator=g) + 0.5).to(dtype)
    return pool, ids, x, y0, v, scales, R


# ------------------------------------------------------------------ 16-bit conversions of the C file
@pytest.mark.parametrize("dt,code", [(torch.float16, 0), (torch.bfloat16, 1)])
def test_c_conversions_match_torch(dt, code):
    lib = bgmv_ref.lib()
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    as_f = bits.view(dt).to(torch.float32)
    step = 37  # every 37th pattern + the edges keeps the ctypes loop short
    picks = list(range(0, 65536, step)) + [0x0001, 0x03ff, 0x0400, 0x7bff, 0x7c00, 0xfc00, 0x8000, 0x7f7f, 0x7f80]
    for b in picks:
        got = lib.bgmv_ref_to_float(b, code)
        want = float(as_f[b])
        assert (np.isnan(got) and np.isnan(want)) or got == want, hex(b)
    g = torch.Generator().manual_seed(5)
    vals = torch.cat([torch.randn(4000, generator=g) * s for s in (1e-7, 1e-4, 1.0, 300.0, 7e4)])
    vals = torch.cat([vals, torch.tensor([0.0, -0.0, 65504.0, 65519.9, 65520.0, 6e-8, 2.98e-8, 2.9802322e-8, 1e-10])])
    want = vals.to(dt).view(torch.int16).to(torch.int32) & 0xffff
    for f, w in zip(vals.tolist(), want.tolist()):
        assert lib.bgmv_ref_from_float(f, code) == w, f


# ------------------------------------------------------------------ reference-held loop
@pytest.mark.parametrize("part", ["A", "B"])
def test_reference_multi_rank_loop(part):
    """Shapes and formula of test_kernel_correctness_multi_rank.py:57-106 (a_loc = arange, scale 1)."""
    g = torch.Generator().manual_seed(42)
    H, R, N, heads = 1024, [8, 16], 128, 32
    max_r = max(R)
    key_buffer = torch.cat([torch.randn(R[0] * 4, heads, H // heads, generator=g),
                            torch.randn(R[1] * 4, heads, H // heads, generator=g)]).to(torch.float16)
    a_len = torch.tensor([R[0] * 4, R[1] * 4])
    a_start = torch.zeros_like(a_len)
    a_start[1:] = torch.cumsum(a_len[:-1], 0)
    a_loc = torch.arange((R[0] + R[1]) * 4)
    a_scaling = torch.tensor([1, 1], dtype=torch.float16)
    bins = torch.cat([torch.tensor([i] * ((N + 1) // 2)) for i in range(2)])[:N]
    qkvo = 0
    if part == "A":
        x = torch.randn(N, H, generator=g).to(torch.float16)
        y0 = torch.zeros(N, max_r, dtype=torch.float16)
    else:
        x = torch.randn(N, max_r, generator=g).to(torch.float16)
        y0 = torch.zeros(N, H, dtype=torch.float16)
    # the loop of :95-106, in fp64 so the yardstick itself has no rounding of its own
    rows = []
    for i in range(N):
        a = int(bins[i])
        a_w = key_buffer[a_start[a] + qkvo * R[a]: a_start[a] + (qkvo + 1) * R[a]].double()
        a_w = a_w.reshape(R[a], H).T if part == "A" else a_w.reshape(H, R[a]).T
        ret = x[i:i + 1, :R[a]].double() @ a_w if part == "B" else x[i:i + 1].double() @ a_w
        rows.append(torch.nn.functional.pad(ret, (0, y0.shape[1] - ret.shape[1])))
    ref = torch.cat(rows)
    got = O.dispatch_bgmv(y0, x, key_buffer, a_start, a_len, a_loc, bins, qkvo, a_scaling)
    assert O.max_abs(got, ref.to(torch.float16)) <= 2 ** -8 * max(1.0, float(ref.abs().max()))
    # and the C restatement agrees with the same yardstick
    c = (bgmv_ref.shrink if part == "A" else
         lambda *a: bgmv_ref.expand(*a, a_scaling))(y0, x, key_buffer, a_start, a_len, a_loc, bins, qkvo)
    assert O.max_abs(c, ref.to(torch.float16)) <= 2 ** -8 * max(1.0, float(ref.abs().max()))


# ------------------------------------------------------------------ index-literal brute force
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("slot", [0, 2, 3])
def test_brute_force_flat_offsets(dtype, slot):
    pool, ids, x, y0, v, scales, R = _rand_case(7 + slot, T=10, H=32, ranks=(8, 16, 8), dtype=dtype)
    H = 32
    kb = pool.key_buffer.reshape(-1, H).double()
    vb = pool.value_buffer.reshape(-1, H).double()
    # shrink: v[t, j] = sum_k x[t,k] * KB[a_loc[a_start + r*slot + j], k]
    want_v = torch.zeros(10, R, dtype=torch.float64)
    keep = torch.ones(10, R, dtype=torch.bool)
    for t in range(10):
        a = int(ids[t]); r = int(pool.a_len[a]) // 4; base = int(pool.a_start[a]) + r * slot
        for j in range(r):
            row = int(pool.a_loc[base + j])
            want_v[t, j] = sum(float(x[t, k]) * float(kb[row, k]) for k in range(H))
            keep[t, j] = False
    y_init = torch.full((10, R), 3.0, dtype=dtype)
    got_v = O.bgmv_shrink(y_init, x, pool.key_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, slot)
    assert torch.equal(got_v[keep], y_init[keep]), "columns >= rank must keep their value"
    assert torch.equal(got_v[~keep], want_v.to(dtype)[~keep])
    # expand: y[t,o] += scale * sum_j v[t,j] * VB[a_loc[base + (o*r+j)//H], (o*r+j)%H]
    want_y = y0.double().clone()
    for t in range(10):
        a = int(ids[t]); r = int(pool.a_len[a]) // 4; base = int(pool.a_start[a]) + r * slot
        for o in range(H):
            acc = 0.0
            for j in range(r):
                f = o * r + j
                acc += float(v[t, j]) * float(vb[int(pool.a_loc[base + f // H]), f % H])
            want_y[t, o] += acc * float(scales[a])
    got_y = O.bgmv_expand(y0, v, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, slot, scales)
    ulp = 2 ** -10 if dtype == torch.float16 else 2 ** -7
    assert O.max_abs(got_y, want_y) <= ulp * float(want_y.abs().max())
    assert (got_y != want_y.to(dtype)).float().mean() < 0.02  # at most rare 1-ulp rounding flips


# ------------------------------------------------------------------ C restatement vs python oracle
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("paged", [False, True])
def test_c_restatement_agrees(dtype, paged):
    pool, ids, x, y0, v, scales, R = _rand_case(11, T=40, H=128, ranks=(8, 16, 32, 8), dtype=dtype, paged=paged)
    for slot in range(4):
        py = O.bgmv_shrink(torch.zeros(40, R, dtype=dtype), x, pool.key_buffer, pool.a_start, pool.a_len,
                           pool.a_loc, ids, slot)
        c = bgmv_ref.shrink(torch.zeros(40, R, dtype=dtype), x, pool.key_buffer, pool.a_start, pool.a_len,
                            pool.a_loc, ids, slot)
        assert (py != c).float().mean() < 0.01 and O.rel_l2(py, c) < 2e-3
        py = O.bgmv_expand(y0, v, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, slot, scales)
        c = bgmv_ref.expand(y0, v, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, slot, scales)
        assert (py != c).float().mean() < 0.01 and O.rel_l2(py, c) < 2e-3


# ------------------------------------------------------------------ invariants
def test_invariants():
    dtype = torch.float16
    pool, ids, x, y0, v, scales, R = _rand_case(3, T=32, H=64, ranks=(8, 16, 8), dtype=dtype)
    args = (pool.a_start, pool.a_len, pool.a_loc, ids)
    base = O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, *args, 1, scales, round_v=False)
    # linearity in the scale (exact-arithmetic variant)
    twice = O.lora_op(y0, x, pool.key_buffer, pool.value_buffer, *args, 1, scales.float() * 2, round_v=False)
    assert torch.allclose(twice - y0.float(), 2 * (base - y0.float()), rtol=1e-5, atol=1e-6)
    # zero scale leaves y untouched, bit for bit
    same = O.bgmv_expand(y0, v, pool.value_buffer, *args, 1, torch.zeros_like(scales))
    assert torch.equal(same, y0)
    # slot isolation: scrambling the rows of slots != 1 does not change slot 1's result
    kb2, vb2 = pool.key_buffer.clone(), pool.value_buffer.clone()
    for a, r in enumerate(pool.ranks):
        st = int(pool.a_start[a])
        other = torch.cat([pool.a_loc[st: st + r], pool.a_loc[st + 2 * r: st + 4 * r]])
        kb2[other] += 1.0
        vb2[other] -= 1.0
    iso = O.lora_op(y0, x, kb2, vb2, *args, 1, scales, round_v=False)
    assert torch.equal(iso, base)
    # page-permutation invariance: move every pool row and rewrite a_loc accordingly
    n = pool.n_rows
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(9))
    kb3 = torch.empty_like(pool.key_buffer); kb3[perm] = pool.key_buffer
    vb3 = torch.empty_like(pool.value_buffer); vb3[perm] = pool.value_buffer
    moved = O.lora_op(y0, x, kb3, vb3, pool.a_start, pool.a_len, perm[pool.a_loc], ids, 1, scales, round_v=False)
    assert torch.equal(moved, base)
    # one-hot A rows make the shrink a column gather: v[t, j] = x[t, col_j]
    kb4 = torch.zeros_like(pool.key_buffer).reshape(n, 64)
    cols = {}
    for a, r in enumerate(pool.ranks):
        st = int(pool.a_start[a]) + r * 1
        for j in range(r):
            c = (7 * a + 3 * j) % 64
            kb4[int(pool.a_loc[st + j]), c] = 1.0
            cols[(a, j)] = c
    vsel = O.bgmv_shrink(torch.zeros(32, R, dtype=dtype), x, kb4.reshape_as(pool.key_buffer), *args, 1)
    for t in range(32):
        a = int(ids[t])
        for j in range(pool.ranks[a]):
            assert vsel[t, j] == x[t, cols[(a, j)]]
    # one-hot B: B[j, o] = [o == j]  ->  y[t, o] += scale * v[t, o] for o < r
    vb5 = torch.zeros(n, 64, dtype=dtype)
    for a, r in enumerate(pool.ranks):
        st = int(pool.a_start[a]) + r * 1
        flat = torch.zeros(64 * r, dtype=dtype)
        for j in range(r):
            flat[j * r + j] = 1.0           # [H_out, r] row-major: flat[o*r + j] = B[j, o]
        vb5[pool.a_loc[st: st + r]] = flat.reshape(r, 64)
    y5 = O.bgmv_expand(torch.zeros(32, 64, dtype=dtype), v, vb5.reshape_as(pool.value_buffer), *args, 1,
                       torch.ones_like(scales))
    for t in range(32):
        r = pool.ranks[int(ids[t])]
        assert torch.equal(y5[t, :r], v[t, :r]) and float(y5[t, r:].abs().max()) == 0.0


def test_per_segment_path_agrees_with_kernel_semantics():
    """lora_bmm_infer.py:342-352 on dense A/B == BGMV shrink+expand over the pool (config 1 shape, small)."""
    w = W.config1(hidden=256, seg_len=16, y0_random=True)
    t = w.targets[0]
    p = t.pool
    dense = [p.dense(a, t.slot) for a in range(p.n_adapters)]
    segs = O.segments_from_ids(w.ids.tolist())
    per_seg = O.per_segment_mm(w.y0["q"], w.x[256], [d[0] for d in dense], [d[1] for d in dense], segs,
                               [float(s) for s in p.a_scaling], compute_dtype=torch.float32)
    kern = O.lora_op(w.y0["q"], w.x[256], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, w.ids,
                     t.slot, p.a_scaling, round_v=False)
    assert O.rel_l2(per_seg, kern) < 1e-3 and O.max_abs(per_seg, kern) < 2e-2
    native = O.per_segment_mm(w.y0["q"], w.x[256], [d[0] for d in dense], [d[1] for d in dense], segs,
                              [float(s) for s in p.a_scaling])
    assert O.rel_l2(native, kern) < 2e-3


def test_triton_style_equals_bgmv_through_repeat_interleave():
    w = W.config3(hidden=128, mlp=256, len_div=16, n_decode=12, targets=("q",))
    t = w.targets[0]; p = t.pool
    R = max(p.ranks)
    x = w.x[128]
    o0 = torch.zeros(w.T, R, dtype=w.dtype)
    tri = O.triton_shrink(x, p.key_buffer.reshape(-1, 128), o0, p.a_loc, p.a_start, p.a_len, w.b_start_loc,
                          w.b_seq_len, w.req_bins, 128, t.slot, R, int(w.b_seq_len.max()))
    bg = O.bgmv_shrink(o0, x, p.key_buffer, p.a_start, p.a_len, p.a_loc, w.ids, t.slot)
    assert torch.equal(tri, bg)  # o0 is zero, so zero-fill and "untouched" coincide
    y0 = w.y0["q"]
    tri = O.triton_expand(bg, p.value_buffer.reshape(-1, 128), y0, p.a_scaling, p.a_loc, p.a_start, p.a_len,
                          w.b_start_loc, w.b_seq_len, w.req_bins, 128, t.slot, R, int(w.b_seq_len.max()))
    be = O.bgmv_expand(y0, bg, p.value_buffer, p.a_start, p.a_len, p.a_loc, w.ids, t.slot, p.a_scaling)
    assert torch.equal(tri, be)


# ------------------------------------------------------------------ Triton launch grid, program by program
def _cdiv(a, b):
    return -(-a // b)


def _int_case(seed, seq, req, ranks, hidden, o_cols, dtype=torch.float16):
    """Small-integer operands: every product and every partial sum is exactly representable in fp16 /
    bf16 / fp32, so any summation order gives the same bits and the comparison can be exact."""
    g = torch.Generator().manual_seed(seed)
    pool = W.make_pool(list(ranks), hidden, hidden, dtype, g, True, std=1.0)
    n = pool.n_rows
    kb = torch.randint(-1, 2, (n, hidden), generator=g).to(dtype)
    vb = torch.randint(-1, 2, (n, hidden), generator=g).to(dtype)
    seq = torch.tensor(seq, dtype=torch.int32)
    start = (torch.cumsum(seq, 0) - seq).to(torch.int32)
    T = int(seq.sum())
    x = torch.randint(-2, 3, (T, hidden), generator=g).to(dtype)
    v = torch.randint(-2, 3, (T, o_cols), generator=g).to(dtype)
    o0 = torch.randint(-3, 4, (T, o_cols), generator=g).to(dtype)
    y0 = torch.randint(-3, 4, (T, hidden), generator=g).to(dtype)
    scale = torch.tensor([0.5, 1.0, 2.0, 1.5][:len(ranks)], dtype=dtype)
    return pool, kb, vb, seq, start, torch.tensor(req), x, v, o0, y0, scale


def _grid_shrink(X, Wt, Out, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies, hidden,
                 qkvo, max_rank, max_input_len):
    """_shrink_fwd_kernel + its launcher (lora_prefill.py:56-102,139-163) on flat arrays: one loop
    iteration per Triton program, masks and offsets as written there."""
    BLOCK_N = 16 if max_rank > 8 else max_rank
    BLOCK_M = 32
    sx, sw, so = X.shape[1], Wt.shape[1], Out.shape[1]
    Xf, Wf, Of = X.reshape(-1).tolist(), Wt.reshape(-1).tolist(), Out.reshape(-1).clone()
    for cur_batch in range(len(b_seq_len)):
        for start_n in range(_cdiv(max_rank, BLOCK_N)):
            for start_m in range(_cdiv(max_input_len, BLOCK_M)):
                ad = int(b_indicies[cur_batch])
                seq_len = int(b_seq_len[cur_batch])
                rank = int(b_lora_ranks[ad]) // 4
                a0 = int(b_lora_start[ad]) + rank * qkvo
                t0 = int(b_start_loc[cur_batch])
                for mi in range(BLOCK_M):
                    m = start_m * BLOCK_M + mi
                    if not m < seq_len:        # store mask (:100); masked x rows load 0.0 and are never stored
                        continue
                    for ni in range(BLOCK_N):
                        nn = start_n * BLOCK_N + ni
                        acc = 0.0
                        if nn < rank:          # weight mask (:89,96): other = 0.0
                            w_loc = int(b_loc[a0 + nn])
                            for k in range(hidden):
                                acc += Xf[(t0 + m) * sx + k] * Wf[w_loc * sw + k]
                        Of[(t0 + m) * so + nn] = acc
    return Of.reshape(Out.shape)


def _grid_expand(X, Wt, Out, scale, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies,
                 feat_out, qkvo, max_rank, max_input_len):
    """_expand_fwd_kernel + its launcher (lora_prefill.py:9-54,105-135), program by program."""
    BLOCK_N, BLOCK_M = 128, 32
    TILE = BLOCK_N
    sx, sw, so = X.shape[1], Wt.shape[1], Out.shape[1]
    Xf, Wf = X.reshape(-1).tolist(), Wt.reshape(-1).tolist()
    Of = Out.reshape(-1).double().clone()
    for cur_batch in range(len(b_seq_len)):
        for cur_tile in range(_cdiv(feat_out, TILE)):
            for start_m in range(_cdiv(max_input_len, BLOCK_M)):
                ad = int(b_indicies[cur_batch])
                seq_len = int(b_seq_len[cur_batch])
                rank = int(b_lora_ranks[ad]) // 4
                a0 = int(b_lora_start[ad]) + rank * qkvo
                t0 = int(b_start_loc[cur_batch])
                sc = float(scale[ad])
                for start_n in range(cur_tile * TILE, (cur_tile + 1) * TILE, BLOCK_N):
                    for ni in range(BLOCK_N):
                        nn = start_n + ni
                        assert nn < feat_out, "the emulation covers widths that are multiples of 128"
                        w_loc = int(b_loc[a0 + (nn * rank) // feat_out])
                        for mi in range(BLOCK_M):
                            m = start_m * BLOCK_M + mi
                            if not m < seq_len:
                                continue
                            acc = 0.0
                            for d in range(max_rank):
                                if d < rank:   # weight mask (:43); x is read for every d < BLOCK_RANK
                                    acc += Xf[(t0 + m) * sx + d] * Wf[w_loc * sw + (nn * rank + d) % feat_out]
                            Of[(t0 + m) * so + nn] += acc * sc
    return Of.reshape(Out.shape)


@pytest.mark.parametrize("max_rank,o_cols", [(8, 8), (8, 16), (24, 32), (16, 16), (32, 40)])
def test_triton_shrink_vs_launch_grid(max_rank, o_cols):
    """Non-zero o, ranks below max_rank (zero fill up to the last column block), a column block that
    ends past max_rank (24 -> 32 columns), max_input_len shorter than the longest request (rows past
    the last 32-row block keep their value), an empty request."""
    ranks = [r for r in (8, 16, 24, 32) if r <= max_rank] or [8]
    seq = [37, 1, 0, 70, 33]
    req = [(i * 3) % len(ranks) for i in range(len(seq))]
    H = 32
    pool, kb, vb, seq, start, req, x, v, o0, y0, scale = _int_case(100 + max_rank, seq, req, ranks, H, o_cols)
    for mx in (int(seq.max()), 40, 1):
        want = _grid_shrink(x.double(), kb.double(), o0.double(), pool.a_loc, pool.a_start, pool.a_len, start,
                            seq, req, H, 1, max_rank, mx)
        got = O.triton_shrink(x, kb, o0, pool.a_loc, pool.a_start, pool.a_len, start, seq, req, H, 1, max_rank, mx)
        assert torch.equal(got.double(), want), f"max_input_len={mx}"
        # the case means something: some rows were left alone, some columns were zero-filled
        if mx == 40:
            assert torch.equal(got[int(start[3]) + 64:int(start[3]) + 70], o0[int(start[3]) + 64:int(start[3]) + 70])
            assert not torch.equal(got[int(start[3]):int(start[3]) + 64], o0[int(start[3]):int(start[3]) + 64])


@pytest.mark.parametrize("max_rank", [8, 16, 24])
def test_triton_expand_vs_launch_grid(max_rank):
    ranks = [r for r in (8, 16, 24) if r <= max_rank]
    seq = [37, 1, 0, 70, 33]
    req = [(i * 2) % len(ranks) for i in range(len(seq))]
    H = 384     # every rank divides it, so an output's r weights never straddle two pool rows
    pool, kb, vb, seq, start, req, x, v, o0, y0, scale = _int_case(200 + max_rank, seq, req, ranks, H, max_rank)
    for mx in (int(seq.max()), 40):
        want = _grid_expand(v.double(), vb.double(), y0, scale, pool.a_loc, pool.a_start, pool.a_len, start, seq,
                            req, H, 2, max_rank, mx)
        got = O.triton_expand(v, vb, y0, scale, pool.a_loc, pool.a_start, pool.a_len, start, seq, req, H, 2,
                              max_rank, mx)
        assert torch.equal(got.double(), want), f"max_input_len={mx}"
        if mx == 40:
            assert torch.equal(got[int(start[3]) + 64:int(start[3]) + 70], y0[int(start[3]) + 64:int(start[3]) + 70])


def test_sgmm_canonical_covered_rows():
    """Rows of the first P segments get the BGMV result, every other row keeps its bits; with P = all
    runs the function is dispatch_bgmv (plain-loop mask, segment tensors with tails of ones)."""
    pool, ids, x, y0, v, scales, R = _rand_case(21, T=40, H=64, ranks=(8, 16, 8))
    ids = torch.repeat_interleave(torch.tensor([2, 0, 0, 1, 2]), torch.tensor([7, 9, 4, 12, 8]))
    oc, rc, li, st = O.count_consecutive_requests(pool.a_len, ids)
    assert oc == [7, 13, 12, 8]
    oc_t = torch.tensor(oc + [1] * 3); st_t = torch.tensor(st + [1] * 3)
    full_s = O.bgmv_shrink(torch.full((40, R), 1.5, dtype=x.dtype), x, pool.key_buffer, pool.a_start, pool.a_len,
                           pool.a_loc, ids, 1)
    full_e = O.bgmv_expand(y0, v, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 1, scales)
    for P in range(0, 5):
        covered = [False] * 40
        for i in range(P):
            for t in range(st[i], st[i] + oc[i]):
                covered[t] = True
        cov = torch.tensor(covered)
        d0 = torch.full((40, R), 1.5, dtype=x.dtype)
        got = O.sgmm_canonical(d0, x, pool.key_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 1, scales, oc_t,
                               st_t, P)
        assert torch.equal(got[cov], full_s[cov]) and torch.equal(got[~cov], d0[~cov])
        got = O.sgmm_canonical(y0, v, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, 1, scales, oc_t,
                               st_t, P)
        assert torch.equal(got[cov], full_e[cov]) and torch.equal(got[~cov], y0[~cov])


# ------------------------------------------------------------------ integer builders
def test_count_consecutive_vs_groupby():
    g = torch.Generator().manual_seed(1)
    lora_rank = torch.tensor([32, 64, 128, 256, 32])
    for T in (1, 2, 5, 64, 65, 300):
        for style in ("random", "runs", "equal", "distinct"):
            if style == "random":
                ids = torch.randint(0, 5, (T,), generator=g)
            elif style == "runs":
                ids = torch.repeat_interleave(torch.randint(0, 5, (T,), generator=g),
                                              torch.randint(1, 9, (T,), generator=g))[:T]
            elif style == "equal":
                ids = torch.full((T,), 3)
            else:
                ids = torch.arange(T) % 5
            oc, rc, li, st = O.count_consecutive_requests(lora_rank, ids)
            runs = [(k, len(list(grp))) for k, grp in itertools.groupby(ids.tolist())]
            assert li == [k for k, _ in runs] and oc == [n for _, n in runs]
            assert rc == [int(lora_rank[k]) // 4 for k, _ in runs]
            assert st == list(np.cumsum([0] + [n for _, n in runs])[:-1])


def _golden():
    with open(os.path.join(HERE, "golden", "segments.json")) as f:
        return json.load(f)["cases"]


@pytest.mark.parametrize("case", _golden(), ids=lambda c: c["name"])
def test_set_sgmm_args_oracle_vs_hand_derived(case):
    out = O.set_sgmm_args(case["dirs"], case["lens"], case["prefill"], case["merged"])
    if case["oc"] is None:
        assert out is None
        return
    oc, lora_ids, st, num_problems = out
    assert oc.tolist() == case["oc"] and st.tolist() == case["st"]
    assert lora_ids.tolist() == [0] * 128 and num_problems == case["num_problems"]
    assert oc.dtype == torch.long and st.dtype == torch.long


@pytest.mark.parametrize("case", _golden(), ids=lambda c: c["name"])
def test_set_sgmm_args_product_vs_hand_derived(case):
    from valora_amd.segments import set_sgmm_args
    out = set_sgmm_args(case["dirs"], case["lens"], case["prefill"], case["merged"])
    if case["oc"] is None:
        assert out is None
        return
    oc, lora_ids, st, num_problems = out
    assert oc.tolist() == case["oc"] and st.tolist() == case["st"]
    assert lora_ids.tolist() == [0] * 128 and num_problems == case["num_problems"]
    assert oc.dtype == torch.long and st.dtype == torch.long and lora_ids.dtype == torch.long


def test_set_sgmm_args_product_vs_oracle_random():
    from valora_amd.segments import set_sgmm_args
    import random
    rng = random.Random(1234)
    names = ["A", "B", "C", "M", None]
    for trial in range(400):
        n = rng.choice([1, 2, 3, 5, 9, 40, 130, 200])
        stick = rng.random()
        dirs = [rng.choice(names)]
        for _ in range(n - 1):
            dirs.append(dirs[-1] if rng.random() < stick else rng.choice(names))
        lens = [rng.randint(1, 50) for _ in range(n)]
        for prefill in (True, False):
            for merged in ("M", "A", None, "absent"):
                want = O.set_sgmm_args(dirs, lens, prefill, merged)
                got = set_sgmm_args(dirs, lens, prefill, merged)
                if want is None:
                    assert got is None
                    continue
                assert got is not None
                for a, b in zip(want[:3], got[:3]):
                    assert torch.equal(a, b)
                assert want[3] == got[3]
                P = want[3][0]
                # invariants of the cumulative sum over the kept counts (the single-request
                # early return leaves start_ids = [0, 1, 1, ...] and is exempt)
                assert n == 1 or all(int(got[2][k + 1] - got[2][k]) == int(got[0][k]) for k in range(min(P, 100)))
