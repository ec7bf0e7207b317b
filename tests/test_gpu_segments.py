"""GPU: the reference's real segment chain through the drop-in entry points.

* per-token id builders behind the ATMM / Triton signatures, bit-exact against ``repeat_interleave`` and
  a plain-loop covered-rows mask;
* ``set_sgmm_args(..., device="cuda")`` -> ``dispatch_sgmm`` exactly as the reference's forward pass wires
  them (valora/server/router/model_infer/model_rpc.py:265-375 feeding
  valora/models/peft/lora_unordered_batch_infer.py:188-190,277-283,946-988): 128-long tensors with tails of
  ones, ``start_ids`` of 129 / 128 entries, the leading merged run dropped, ``x`` / ``y`` passed as
  ``[delora_tk_index:]`` views, ``num_problems`` decremented;
* the reference's compensation branch (``:270-276,991-1063``): doubled batch, ``[1:]`` views of the segment
  tensors, ``num_problems - 1``, ``q += d[:de] - d[de:]``.
"""
import pytest
import torch

from oracle import lora_oracle as O
from valora_amd import workloads as W

from tests._util import assert_parity

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------ per-token id builders, bit-exact
@pytest.mark.parametrize("seed", range(6))
def test_ids_from_requests_bit_exact(dev, seed):
    from valora_amd import _lib
    g = torch.Generator().manual_seed(seed)
    n_req = [1, 7, 40, 300, 1000, 64][seed]
    seq = torch.randint(0 if seed % 2 else 1, [5, 90, 600, 40, 9, 2049][seed], (n_req,), generator=g).to(torch.int32)
    req = torch.randint(0, 50, (n_req,), generator=g)
    start = (torch.cumsum(seq, 0) - seq).to(torch.int32)
    T = int(seq.sum())
    pad = 5                                     # rows no request owns (the output is longer than the batch)
    start_d, seq_d, req_d = start.to(dev), seq.to(dev), req.to(dev)
    for max_rows in (1 << 30, 32, 64, 0):
        out = torch.full((T + pad,), 12345, dtype=torch.long, device=dev)
        _lib.check(_lib.lib().mlora_ids_from_requests(
            _lib.current_stream(dev), _lib.ptr(out), _lib.ptr(start_d), _lib.ptr(seq_d), _lib.ptr(req_d), n_req,
            T + pad, max_rows))
        want = torch.full((T + pad,), -1, dtype=torch.long)
        for i in range(n_req):
            s, n = int(start[i]), min(int(seq[i]), max_rows)
            want[s:s + n] = req[i]
        assert torch.equal(out.cpu(), want), f"max_rows={max_rows}"
        if max_rows >= int(seq.max()):
            assert torch.equal(out.cpu()[:T], torch.repeat_interleave(req, seq.long()))


@pytest.mark.parametrize("seed", range(6))
def test_ids_from_segments_bit_exact(dev, seed):
    from valora_amd import _lib
    g = torch.Generator().manual_seed(100 + seed)
    n_runs = [1, 3, 20, 127, 128, 60][seed]
    counts = torch.randint(1, [9, 300, 50, 12, 40, 2][seed], (n_runs,), generator=g)
    T = int(counts.sum())
    ids = torch.randint(-1, 40, (T,), generator=g)
    # the reference's buffers: 128 counts with a tail of ones, 129 starts = [0, running sum]
    oc = torch.ones(128, dtype=torch.long); oc[:n_runs] = counts
    st = torch.cat([torch.zeros(1, dtype=torch.long), torch.cumsum(oc, 0)])
    ids_d, st_d, oc_d = ids.to(dev), st.to(dev), oc.to(dev)
    for P in sorted({0, 1, n_runs // 2, n_runs, min(128, n_runs + 2)}):
        out = torch.full((T,), 777, dtype=torch.long, device=dev)
        _lib.check(_lib.lib().mlora_ids_from_segments(
            _lib.current_stream(dev), _lib.ptr(out), _lib.ptr(ids_d), _lib.ptr(st_d), _lib.ptr(oc_d), P, T))
        want = torch.full((T,), -1, dtype=torch.long)
        for i in range(P):
            for t in range(int(st[i]), min(T, int(st[i]) + int(oc[i]))):   # problems past the batch end are clipped
                want[t] = ids[t]
        assert torch.equal(out.cpu(), want), f"P={P}"


# ------------------------------------------------------------------ set_sgmm_args -> dispatch_sgmm
def _batch(seed, dirs, lens, prefill, ranks, h, dtype):
    """A batch as the server holds it: requests in arrival order, ``adapter_dirs`` per request, the resident
    adapters' directory list (``infer_adapter.adapter_dirs``) naming the pool slots."""
    g = torch.Generator().manual_seed(seed)
    resident = sorted(set(dirs))
    pool = W.make_pool([ranks[d] for d in resident], h, h, dtype, g, True, std=0.05,
                       scalings=[0.5 + 0.25 * i for i in range(len(resident))])
    req_bins = torch.tensor([resident.index(d) for d in dirs])
    seq = torch.tensor(lens if prefill else [1] * len(dirs))
    T = int(seq.sum())
    x = torch.randn(T, h, generator=g).to(dtype)
    q0 = torch.randn(T, h, generator=g).to(dtype)
    return pool, req_bins, seq, T, x, q0


CHAIN_CASES = [
    # name, adapter_dirs, input_lengths, prefill, merged adapter dir
    ("prefill_runs", ["A", "A", "B", "C", "C", "A"], [37, 5, 64, 1, 20, 33], True, None),
    ("prefill_merged_first", ["M", "M", "A", "A", "B"], [5, 7, 3, 2, 9], True, "M"),
    ("prefill_merged_absent", ["A", "B", "B", "M"], [16, 40, 3, 12], True, "M"),
    ("prefill_single_request", ["B"], [50], True, None),
    ("prefill_one_run", ["A", "A", "A"], [9, 30, 2], True, None),
    ("decode_runs", ["A", "B", "B", "A", "C", "C", "C", "B"], [1] * 8, False, None),
    ("decode_merged_first", ["M", "M", "M", "A", "B", "B"], [1] * 6, False, "M"),
    ("decode_distinct", [chr(65 + i % 7) for i in range(90)], [1] * 90, False, None),
    # decode probes the adapter AFTER the first boundary (model_rpc.py:337): the first count is dropped although
    # the leading run is not the merged one, and the problems then cover T - c0 + 1 rows
    ("decode_merged_second", ["A", "M", "M", "B"], [1] * 4, False, "M"),
    ("decode_merged_second_long_first", ["A", "A", "A", "M", "B", "B"], [1] * 6, False, "M"),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CHAIN_CASES, ids=lambda c: c[0])
def test_set_sgmm_args_feeds_dispatch_sgmm(dev, case, dtype):
    from valora_amd.atmm_ops import dispatch_bgmv as dispatch_sgmm
    from valora_amd.segments import set_sgmm_args
    name, dirs, lens, prefill, merged = case
    ranks = {"A": 16, "B": 8, "C": 32, "M": 16, "D": 8, "E": 16, "F": 8, "G": 32}
    h, R = 256, 32
    pool, req_bins, seq, T, x, q0 = _batch(len(name), dirs, lens, prefill, ranks, h, dtype)
    out = set_sgmm_args(dirs, lens, prefill, merged, device=dev)
    want_seg = O.set_sgmm_args(dirs, lens, prefill, merged)
    assert out is not None
    oc, lora_ids, st, num_problems = out
    assert oc.is_cuda and st.is_cuda and lora_ids.is_cuda
    for a, b in zip((oc, lora_ids, st), want_seg[:3]):
        assert torch.equal(a.cpu(), b)
    assert num_problems == want_seg[3]
    assert oc.numel() in (127, 128) and st.numel() == oc.numel() + 1 or len(dirs) == 1

    # what LoraUnorderedBatchInfer.__init__ / forward derive from num_problems (:188-190, :277-283)
    P, (de_req, de_tok) = num_problems[0], num_problems[1]
    if de_req > 0:
        P -= 1
    bins = req_bins[de_req:]
    batch_req_bins = torch.repeat_interleave(bins, seq[de_req:])
    assert batch_req_bins.numel() == T - de_tok
    pd = pool.to(dev)
    idx = (pool.a_start, pool.a_len, pool.a_loc)
    idxd = (pd.a_start, pd.a_len, pd.a_loc)
    rank_counts = torch.full((128,), 64, dtype=torch.long, device=dev)      # req_queue.py:25
    tmp_d = torch.zeros(128 * 60, dtype=torch.int8, device=dev)
    xd, q = x.to(dev), q0.to(dev)
    delta0 = torch.full((T - de_tok, R), 0.75, dtype=dtype)
    delta = delta0.to(dev)
    ids_d = batch_req_bins.to(dev)
    # :946-952 shrink on x[delora_tk_index:], :967-972 expand into q[delora_tk_index:]
    dispatch_sgmm(delta, xd[de_tok:], pd.key_buffer, *idxd, ids_d, 0, pd.a_scaling, oc, rank_counts, lora_ids, st,
                  tmp_d, P, 64, 32, 32, 32, 32, 32)
    want_delta = O.sgmm_canonical(delta0, x[de_tok:], pool.key_buffer, *idx, batch_req_bins, 0, pool.a_scaling,
                                  want_seg[0], want_seg[2], P)
    assert_parity(delta.cpu(), want_delta, f"{name} shrink")
    assert torch.equal(delta.cpu() == 0.75, want_delta == 0.75), "columns past the rank / uncovered rows keep their bits"
    dispatch_sgmm(q[de_tok:], delta, pd.value_buffer, *idxd, ids_d, 0, pd.a_scaling, oc, rank_counts, lora_ids, st,
                  tmp_d, P, 64, 64, 32, 64, 64, 32)
    want_q = q0.clone()
    want_q[de_tok:] = O.sgmm_canonical(q0[de_tok:], want_delta, pool.value_buffer, *idx, batch_req_bins, 0,
                                       pool.a_scaling, want_seg[0], want_seg[2], P)
    assert_parity(q.cpu(), want_q, f"{name} expand")
    assert torch.equal(q.cpu()[:de_tok], q0[:de_tok]), "rows of the merged leading run are not touched"
    # where the problems tile [0, T - de_tok) exactly (every prefill batch but the single-request early
    # return), the result is the plain per-token op on the kept rows
    covered = int(want_seg[0][:P].sum())
    if name == "decode_merged_second_long_first":
        assert covered == T - 2, "the dropped first count leaves the batch's tail uncovered"
        assert torch.equal(q.cpu()[covered:], q0[covered:])
    if len(dirs) > 1 and covered == T - de_tok:
        full = O.lora_op(q0[de_tok:], x[de_tok:], pool.key_buffer, pool.value_buffer, *idx, batch_req_bins, 0,
                         pool.a_scaling)
        assert_parity(q.cpu()[de_tok:], full, f"{name} whole chain")


def test_set_sgmm_args_single_request_quirk(dev):
    """One request: ``start_ids = [0, 1, 1, ...]`` (128 entries, no running sum) and ``num_problems = 1``; the
    one problem covers the whole request (model_rpc.py:279-285)."""
    from valora_amd.atmm_ops import dispatch_bgmv as dispatch_sgmm
    from valora_amd.segments import set_sgmm_args
    dtype, h, R = torch.float16, 128, 16
    pool, req_bins, seq, T, x, q0 = _batch(5, ["A"], [45], True, {"A": 16}, h, dtype)
    oc, lora_ids, st, num_problems = set_sgmm_args(["A"], [45], True, None, device=dev)
    assert st.cpu().tolist() == [0] + [1] * 127 and oc.cpu().tolist() == [45] + [1] * 127 and num_problems == [1, [0, 0]]
    pd = pool.to(dev)
    ids = torch.zeros(T, dtype=torch.long, device=dev)
    delta = torch.zeros(T, R, dtype=dtype, device=dev)
    rc = torch.full((128,), 64, dtype=torch.long, device=dev)
    tmp = torch.zeros(7680, dtype=torch.int8, device=dev)
    q = q0.to(dev)
    dispatch_sgmm(delta, x.to(dev), pd.key_buffer, pd.a_start, pd.a_len, pd.a_loc, ids, 3, pd.a_scaling, oc, rc,
                  lora_ids, st, tmp, 1, 64, 32, 32, 32, 32, 32)
    dispatch_sgmm(q, delta, pd.value_buffer, pd.a_start, pd.a_len, pd.a_loc, ids, 3, pd.a_scaling, oc, rc, lora_ids,
                  st, tmp, 1, 64, 64, 32, 64, 64, 32)
    want = O.lora_op(q0, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, ids.cpu(), 3,
                     pool.a_scaling)
    assert_parity(q.cpu(), want, "single request")


# ------------------------------------------------------------------ the reference's compensation branch
def _doubled_batch(req_bins, seq, de_req):
    """lora_unordered_batch_infer.py:270-276: own adapters | merged adapter (``req_bins[0]``)."""
    sub = req_bins[de_req:]
    rep = sub.repeat(2)
    half = rep.numel() // 2
    rep[half:] = req_bins[0]
    return rep, seq[de_req:].repeat(2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_delora_call_sequence(dev, dtype):
    """The calls of lora_unordered_batch_infer.py:991-1010 made literally: ``cat([sub, sub])`` activations, a
    doubled ``batch_req_bins``, ``output_counts[1:]`` / ``start_ids[1:]`` as fresh offset views and
    ``num_problems - 1``, then ``q[tk:] += d[:de] - d[de:]``.

    The drop-in returns what its documented semantics define for exactly these arguments (checked against
    the oracle).  That result is NOT the compensation: with the tensors ``set_sgmm_args`` emits for a leading
    merged run (first count already dropped), the extra ``[1:]`` skips the first non-merged run and leaves
    all but one row of the merged half uncovered.  The second half of the test shows that the same
    doubled-batch arithmetic through the same entry point does give the compensation once the segment
    tensors cover both halves, and that ``DeLoraPlan`` gives it without the copies."""
    from valora_amd.atmm_ops import dispatch_bgmv as dispatch_sgmm
    from valora_amd.merge import DeLoraPlan
    from valora_amd.segments import set_sgmm_args
    dirs, lens, merged = ["M", "M", "A", "A", "B", "C", "C"], [5, 7, 3, 2, 9, 30, 4], "M"
    ranks = {"A": 16, "B": 8, "C": 32, "M": 16}
    h, R = 256, 32
    pool, req_bins, seq, T, x, q0 = _batch(11, dirs, lens, True, ranks, h, dtype)
    oc, lora_ids, st, num_problems = set_sgmm_args(dirs, lens, True, merged, device=dev)
    P, (de_req, de_tok) = num_problems[0], num_problems[1]
    assert (P, de_req, de_tok) == (4, 2, 12)
    bins2, seq2 = _doubled_batch(req_bins, seq, de_req)
    batch_req_bins = torch.repeat_interleave(bins2, seq2)
    de_length = batch_req_bins.numel() // 2
    assert de_length == T - de_tok
    pd = pool.to(dev)
    idx = (pool.a_start, pool.a_len, pool.a_loc)
    idxd = (pd.a_start, pd.a_len, pd.a_loc)
    rank_counts = torch.full((128,), 64, dtype=torch.long, device=dev)
    tmp_d = torch.zeros(128 * 60, dtype=torch.int8, device=dev)
    xd = x.to(dev)
    ids_d = batch_req_bins.to(dev)

    def reference_sequence(oc_arg, rc_arg, li_arg, st_arg, n_prob):
        q = q0.to(dev)
        delta = torch.zeros(2 * de_length, R, dtype=dtype, device=dev)
        d_lora = torch.zeros(2 * de_length, h, dtype=dtype, device=dev)
        sub = xd[de_tok:]
        expanded = torch.cat([sub, sub], dim=0)
        dispatch_sgmm(delta, expanded, pd.key_buffer, *idxd, ids_d, 0, pd.a_scaling, oc_arg, rc_arg, li_arg, st_arg,
                      tmp_d, n_prob, 64, 32, 32, 32, 32, 32)
        dispatch_sgmm(d_lora, delta, pd.value_buffer, *idxd, ids_d, 0, pd.a_scaling, oc_arg, rc_arg, li_arg, st_arg,
                      tmp_d, n_prob, 64, 64, 32, 64, 64, 32)
        q[de_tok:] += d_lora[:de_length] - d_lora[de_length:]
        return q.cpu(), d_lora.cpu()

    def oracle_sequence(oc_arg, st_arg, n_prob):
        xx = torch.cat([x[de_tok:], x[de_tok:]], dim=0)
        delta = O.sgmm_canonical(torch.zeros(2 * de_length, R, dtype=dtype), xx, pool.key_buffer, *idx, batch_req_bins,
                                 0, pool.a_scaling, oc_arg, st_arg, n_prob)
        d = O.sgmm_canonical(torch.zeros(2 * de_length, h, dtype=dtype), delta, pool.value_buffer, *idx,
                             batch_req_bins, 0, pool.a_scaling, oc_arg, st_arg, n_prob)
        q = q0.clone()
        q[de_tok:] += d[:de_length] - d[de_length:]
        return q, d

    # (1) literally as the reference calls it
    got_q, got_d = reference_sequence(oc[1:], rank_counts[1:], lora_ids[1:], st[1:], P - 1)
    want_q, want_d = oracle_sequence(oc.cpu()[1:], st.cpu()[1:], P - 1)
    assert_parity(got_d, want_d, "literal sequence, expanded deltas")
    assert_parity(got_q, want_q, "literal sequence, q")
    comp = O.delora_compensate(q0, x, pool.key_buffer, pool.value_buffer, *idx,
                               torch.repeat_interleave(req_bins, seq), int(req_bins[0]), 0, pool.a_scaling)
    first_other = slice(de_tok, de_tok + 5)      # the run of adapter A: skipped by the extra [1:]
    assert torch.equal(got_d[:5], torch.zeros(5, h, dtype=dtype))
    assert O.max_abs(got_q[first_other], comp[first_other]) > 5e-2, "the literal call shape is not the compensation"

    # (2) segment tensors that cover both halves: own runs, then one run for the merged half
    runs = O.count_consecutive_requests(pool.a_len, batch_req_bins)
    n_runs = len(runs[0])
    oc2 = torch.ones(128, dtype=torch.long); oc2[:n_runs] = torch.tensor(runs[0])
    st2 = torch.cat([torch.zeros(1, dtype=torch.long), torch.cumsum(oc2, 0)])
    got_q, _ = reference_sequence(oc2.to(dev), rank_counts, lora_ids, st2.to(dev), n_runs)
    want_q, _ = oracle_sequence(oc2, st2, n_runs)
    assert_parity(got_q, want_q, "doubled batch with covering segments")
    # against the y-resident form of the compensation: the doubled batch rounds each half to T, then their
    # difference, then the sum with q -- three more roundings, which bf16's 8 significant bits show
    err = (got_q.double() - comp.double()).abs()
    assert float(err.max()) <= 4e-2 and O.rel_l2(got_q, comp) <= (5e-3 if dtype == torch.bfloat16 else 1e-3)
    assert torch.equal(got_q[:de_tok], q0[:de_tok])

    # (3) the replacement: no copies, no doubled batch
    plan = DeLoraPlan(torch.repeat_interleave(req_bins, seq).to(dev), int(req_bins[0]), pd.a_start, pd.a_len, R,
                      hidden=h)
    q = q0.to(dev)
    plan.apply(q, xd, pd.key_buffer, pd.value_buffer, *idxd, 0, pd.a_scaling)
    assert_parity(q.cpu(), comp, "DeLoraPlan")
