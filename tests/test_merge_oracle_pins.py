"""Pins of the merge / deLoRA restatements in oracle/lora_oracle.py.  CPU only."""
import pytest
import torch

from oracle import lora_oracle as O
from valora_amd import workloads as W


def int_pool(H, ranks, dtype, seed, n_slots=4, paged=True):
    """A pool whose weights are small integers: every product and partial sum below is exact in fp32
    and in the 16-bit formats, so any formulation of the arithmetic must agree bit for bit."""
    g = torch.Generator().manual_seed(seed)
    pool = W.make_pool(ranks, H, H, dtype, g, paged, n_slots=n_slots, heads=8)
    pool.key_buffer.copy_(torch.randint(-2, 3, pool.key_buffer.shape, generator=g).to(dtype))
    pool.value_buffer.copy_(torch.randint(-2, 3, pool.value_buffer.shape, generator=g).to(dtype))
    return pool


def loops_merge(Wm, pool, adapter, slot, scaling, sign):
    """Index-literal: W[i][o] += sign * sum_j key[a_loc[base+j]][i] * (value_flat[o*r+j] * scaling)."""
    r = pool.ranks[adapter]
    base = int(pool.a_start[adapter]) + slot * r
    H_in, H_out = Wm.shape
    kb = pool.key_buffer.reshape(-1, H_in)
    vb = pool.value_buffer.reshape(-1, H_out)
    rows = [int(pool.a_loc[base + j]) for j in range(r)]
    flat = torch.cat([vb[q] for q in rows]).tolist()
    out = Wm.clone()
    for i in range(H_in):
        for o in range(H_out):
            acc = 0.0
            for j in range(r):
                acc += float(kb[rows[j]][i]) * (flat[o * r + j] * scaling)
            out[i][o] = float(Wm[i][o]) + sign * acc
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_merge_exact_integer_cases_vs_loops(dtype):
    H = 16
    pool = int_pool(H, [8, 16, 8], dtype, seed=3)
    g = torch.Generator().manual_seed(4)
    for adapter in range(3):
        for slot in (0, 2, 3):
            Wm = torch.randint(-8, 9, (H, H), generator=g).to(dtype)
            for sign in (1, -1):
                got = O.merge_adapter([Wm], pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc,
                                      adapter, 2.0, slots=(slot,), sign=sign)[0]
                assert torch.equal(got, loops_merge(Wm, pool, adapter, slot, 2.0, sign))


def test_merge_rounding_points_and_fp64():
    g = torch.Generator().manual_seed(5)
    H, r = 64, 16
    for dtype, tol in ((torch.float16, 2 ** -10), (torch.bfloat16, 2 ** -7)):
        Wm = torch.randn(H, H, generator=g).to(dtype)
        A = (torch.randn(H, r, generator=g) * 0.1).to(dtype)
        B = (torch.randn(r, H, generator=g) * 0.1).to(dtype)
        got = O.merge_weight(Wm, A, B, 1.5)
        exact = Wm.double() + A.double() @ (B.double() * 1.5)
        assert ((got.double() - exact).abs() <= tol * (1 + exact.abs())).all()
        # b = B * scaling is rounded to T before the GEMM: a scaling that is not a power of two shows it
        b_T = (B.float() * 1.5).to(dtype)
        assert torch.equal(got, (Wm.float() + (A.float() @ b_T.float()).to(dtype).float()).to(dtype))
        # taking it out again lands within one rounding of the start
        back = O.merge_weight(got, A, B, 1.5, sign=-1)
        assert ((back.double() - Wm.double()).abs() <= tol * (1 + Wm.double().abs())).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_merged_weight_equals_base_plus_lora_and_delora_identity(dtype):
    """x @ W_merged == x @ W + LoRA_m(x) for tokens of the merged adapter, and for every other token
    x @ W_merged + compensate == x @ W + LoRA_own(x) -- to the rounding of the 16-bit tensors."""
    H, T = 64, 40
    g = torch.Generator().manual_seed(6)
    pool = W.make_pool([8, 16, 8, 32], H, H, dtype, g, True, std=0.05, scalings=[2.0, 0.5, 1.0, 0.25], heads=8)
    Wm = (torch.randn(H, H, generator=g) * 0.1).to(dtype)
    x = torch.randn(T, H, generator=g).to(dtype)
    ids = torch.randint(-1, 4, (T,), generator=g)
    merged, slot = 1, 2
    Wmerged = O.merge_adapter([Wm], pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, merged,
                              float(pool.a_scaling[merged]), slots=(slot,))[0]
    zeros = torch.zeros(T, H, dtype=dtype)
    base_plus_lora = x.double() @ Wm.double() + O.lora_op(
        zeros, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids, slot,
        pool.a_scaling, round_v=False).double()
    comp = O.delora_compensate(zeros, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc,
                               ids, merged, slot, pool.a_scaling).double()
    via_merged = x.double() @ Wmerged.double() + comp
    want = base_plus_lora.clone()
    none = ids < 0
    # tokens without adapter see the merged weights uncompensated, exactly as in the reference
    want[none] = (x.double() @ Wmerged.double())[none]
    tol = 3e-2 if dtype == torch.bfloat16 else 4e-3
    assert (via_merged - want).abs().max() <= tol * (1 + want.abs().max())
    assert not comp[ids == merged].any() and not comp[none].any()
