"""Helpers shared by the parity tests: run one target of a workload through each entry point of
the product (always through the C ABI) and through the CPU oracle."""
import torch

from oracle import lora_oracle as O

MAX_ABS = 2e-2   # tolerance stated by the benchmark definition: max-abs error
REL_L2 = 1e-3    # and relative L2 error, both against the reference semantics with fp32 accumulation


def oracle_target(w, name, round_v=True, round_y=True):
    t = w.target(name)
    p = t.pool
    return O.lora_op(w.y0[name], w.x[t.h_in], p_kb(w, name), p.value_buffer, p.a_start, p.a_len, p.a_loc,
                     w.ids, t.slot, p.a_scaling, round_v=round_v, round_y=round_y)


def p_kb(w, name):
    return w.target(name).pool.key_buffer


def max_rank(w):
    return max(w.targets[0].pool.ranks)


def run_bgmv(wd, name):
    """Two dispatch_bgmv calls with a T-typed delta between them, like the reference caller
    (valora/models/peft/lora_unordered_batch_infer.py:632-638)."""
    from valora_amd.kernels import dispatch_bgmv
    t = wd.target(name); p = t.pool
    y = wd.y0[name].clone()
    delta = torch.zeros(wd.T, max_rank(wd), dtype=wd.dtype, device=y.device)
    dispatch_bgmv(delta, wd.x[t.h_in], p.key_buffer, p.a_start, p.a_len, p.a_loc, wd.ids, t.slot, p.a_scaling)
    dispatch_bgmv(y, delta, p.value_buffer, p.a_start, p.a_len, p.a_loc, wd.ids, t.slot, p.a_scaling)
    return y, delta


def run_plan(wd, name, **kw):
    from valora_amd.plan import LoraPlan
    t = wd.target(name); p = t.pool
    plan = LoraPlan(wd.ids, p.a_start, p.a_len, max_rank(wd), hidden=t.h_in, **kw)
    y = wd.y0[name].clone()
    plan.apply(y, wd.x[t.h_in], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)
    return y


def run_multi(wd, names, **kw):
    """Targets that read the same x and live in the same pool, through LoraPlan.apply_multi."""
    from valora_amd.plan import LoraPlan
    ts = [wd.target(n) for n in names]
    p = ts[0].pool
    plan = LoraPlan(wd.ids, p.a_start, p.a_len, max_rank(wd), hidden=ts[0].h_in, **kw)
    ys = [wd.y0[n].clone() for n in names]
    plan.apply_multi(ys, wd.x[ts[0].h_in], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc,
                     [t.slot for t in ts], p.a_scaling)
    return ys


def run_one_launch(wd, name, no_wait=False, ksplit=4):
    """The one-launch op (shrink and expand items of one grid); ``no_wait``: every expand item takes its
    give-up path and computes the tile's partials itself."""
    from valora_amd.plan import LoraPlan
    t = wd.target(name); p = t.pool
    plan = LoraPlan(wd.ids, p.a_start, p.a_len, max_rank(wd), hidden=t.h_in, one_launch=True, ksplit=ksplit,
                    one_launch_no_wait=no_wait)
    y = wd.y0[name].clone()
    plan.apply(y, wd.x[t.h_in], p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)
    return y


def run_sgmm(wd, name):
    from valora_amd.atmm_ops import dispatch_bgmv as dispatch_sgmm
    from valora_amd.segments import count_consecutive_requests
    t = wd.target(name); p = t.pool
    oc, rc, li, st, num = count_consecutive_requests(p.a_len, wd.ids)
    P = int(num.item())
    y = wd.y0[name].clone()
    delta = torch.zeros(wd.T, max_rank(wd), dtype=wd.dtype, device=y.device)
    tmp = torch.zeros(max(P, 1) * 60, dtype=torch.int8, device=y.device)
    for (yy, xx, w) in ((delta, wd.x[t.h_in], p.key_buffer), (y, delta, p.value_buffer)):
        dispatch_sgmm(yy, xx, w, p.a_start, p.a_len, p.a_loc, wd.ids, t.slot, p.a_scaling, oc, rc, li, st,
                      tmp, P, 64, 32, 32, 32, 32, 32)
    return y


def run_prefill(wd, name):
    from valora_amd.lora_prefill import lora_get_qkvo_fwd_expand, lora_get_qkvo_fwd_shrink
    t = wd.target(name); p = t.pool
    R = max_rank(wd)
    y = wd.y0[name].clone()
    delta = torch.zeros(wd.T, R, dtype=wd.dtype, device=y.device)
    mx = int(wd.b_seq_len.max().item())
    lora_get_qkvo_fwd_shrink(wd.x[t.h_in], p.key_buffer.view(-1, t.h_in), delta, p.a_loc, p.a_start, p.a_len,
                             wd.b_start_loc, wd.b_seq_len, wd.req_bins, t.h_in, t.slot, R, mx)
    lora_get_qkvo_fwd_expand(delta, p.value_buffer.view(-1, t.h_out), y, p.a_scaling, p.a_loc, p.a_start,
                             p.a_len, wd.b_start_loc, wd.b_seq_len, wd.req_bins, t.h_out, t.slot, R, mx)
    return y


def ulp(want):
    """Spacing of the 16-bit format at |want| (fp16: 10 mantissa bits, bf16: 7)."""
    bits = 10 if want.dtype == torch.float16 else 7
    mag = want.detach().cpu().double().abs().clamp_min(2.0 ** -14)
    return torch.pow(2.0, torch.floor(torch.log2(mag)) - bits)


# what -> (elements over the strict 2e-2, elements compared); filled by assert_parity
ALLOWANCE = {}


def assert_parity(got, want, what="", unrounded=None):
    """max-abs <= 2e-2 and rel-L2 <= 1e-3.  Both sides are 16-bit tensors, so where one unit in the last
    place of the format is itself larger than 2e-2 (bf16 from |y| >= 4, fp16 from |y| >= 32) two correct
    fp32 accumulations that differ in their last bits can round to neighbouring values.  An element over
    the strict 2e-2 is accepted only if it is such a pair: ``got`` and ``want`` are adjacent values of the
    format (bit patterns differ by one) and, when ``unrounded`` (the oracle's accumulator before its
    last rounding) is given, that value lies between the two.  The number of elements that used the
    allowance is recorded in ``ALLOWANCE[what]``."""
    got, want = got.detach().cpu(), want.detach().cpu()
    err = (got.double() - want.double()).abs()
    ma, rl = float(err.max()) if err.numel() else 0.0, O.rel_l2(got, want)
    over = err > MAX_ABS
    n_over = int(over.sum())
    ALLOWANCE[what] = (n_over, got.numel())
    assert rl <= REL_L2, f"{what}: max_abs={ma:.3e} rel_l2={rl:.3e}"
    if n_over:
        assert want.dtype in (torch.float16, torch.bfloat16) and got.dtype == want.dtype, \
            f"{what}: max_abs={ma:.3e} over {MAX_ABS} on {n_over} elements"
        g, w = got[over], want[over]
        step = (g.view(torch.int16).int() - w.view(torch.int16).int()).abs()
        bad = int((step != 1).sum())
        assert bad == 0, f"{what}: max_abs={ma:.3e}; {bad} of {n_over} elements over {MAX_ABS} are more than one ulp apart"
        if unrounded is not None:
            u = unrounded.detach().cpu().double()[over]
            lo, hi = torch.minimum(g.double(), w.double()), torch.maximum(g.double(), w.double())
            outside = int(((u < lo) | (u > hi)).sum())
            assert outside == 0, f"{what}: {outside} of {n_over} one-ulp differences do not straddle the unrounded value"
    return ma, rl
