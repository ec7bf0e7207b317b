"""CPU restatement of the reference's multi-LoRA batching operator.  TEST INFRASTRUCTURE ONLY.

Nothing under ``valora_amd/`` may import this module: it is the checker that the HIP
path is compared against (tests, the smoke check and the bench's CPU-baseline leg), never
the thing that is shipped or measured as the product.

Every function cites the reference source it restates (paths relative to the reference
checkout).  Arithmetic is done on CPU torch tensors: 16-bit operands are widened to fp32,
dot products are accumulated in fp32 (fp64 on request) and results are rounded to the
operand dtype ``T`` at exactly the points where the reference kernels store a ``T`` value.

Pinning status of each function (what fixes it besides its own text):

* ``dense_A`` / ``dense_B`` / ``bgmv_shrink`` / ``bgmv_expand`` -- pinned by (1) the
  reference-held per-token loop ``test/kernel/test_kernel_correctness_multi_rank.py:95-106``
  restated with its own shapes, (2) an index-literal fp64 brute force on tiny paged pools,
  (3) the independently written C restatement ``oracle/bgmv_ref.c`` that follows the CUDA
  kernels' flat-offset indexing, (4) algebraic invariants (linearity in scale, slot
  isolation, page-permutation invariance, one-hot adapters).
* ``per_segment_mm`` -- a library routine (``torch.mm``) applied per segment,
  ``valora/models/bmm/lora_bmm_infer.py:342-352``; pinned against ``bgmv_*`` on the same
  operands (they must agree to rounding) and against fp64.
* ``count_consecutive_requests`` -- pinned by brute force against ``itertools.groupby``.
* ``set_sgmm_args`` -- pinned by hand-derived vectors held in ``tests/golden/segments.json``.
* ``sgmm_canonical`` -- ``bgmv_*`` applied to the rows the first P segments cover; pinned by a
  plain-loop covered-rows mask and by ``P = number of runs`` reducing to ``bgmv_*``.  (ATMM's
  literal launch -- adapter from an all-zero tensor, rank from an all-64 tensor, B read as
  ``[r, H_out]``, scaling ignored -- is not restated: nothing is compared against it.)
* ``triton_shrink`` / ``triton_expand`` -- same closed form as ``bgmv_*`` per request;
  pinned by equivalence with ``bgmv_*`` through ``repeat_interleave`` and, for what differs from
  BGMV (zero-filled columns up to the last column block, rows past the grid's last row block
  left alone, accumulation into a non-zero ``o``), by a brute force that walks the Triton launch
  grid program by program with the kernels' own masks and flat offsets on exact-arithmetic
  (small-integer) operands.
* ``merge_weight`` / ``merge_adapter`` -- a library GEMM plus an in-place add in the reference; pinned by
  small-integer cases where every product and sum is exact (bit-exact against plain Python loops
  over the pool indices), by fp64, by ``unmerge(merge(W))`` staying within one rounding of W, and by
  the identity ``x @ merged W == x @ W + lora_op(x)`` to rounding.
* ``delora_compensate`` -- two applications of ``lora_op``; pinned by the identity
  ``x @ W_merged + compensate == x @ W + lora_op`` for every token.
"""
from __future__ import annotations

import itertools
from typing import List, Optional, Sequence, Tuple

import torch

N_SLOTS = 4  # q, k, v, o -- the reference hard-codes ``lora_ranks[a] / 4`` (bgmv_impl.cuh:35)


# --------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------
def _f(t: torch.Tensor, acc=torch.float32) -> torch.Tensor:
    return t.detach().to("cpu").to(acc)


def round_to(t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Round an fp32/fp64 tensor to ``dtype`` (round-to-nearest-even), return it in ``dtype``."""
    return t.to(torch.float32).to(dtype)


def rank_of(a_len: torch.Tensor, a: int, n_slots: int = N_SLOTS) -> int:
    # valora/csrc/bgmv/bgmv_impl.cuh:35,165 ; lora_prefill.py:27,73
    return int(a_len[a]) // n_slots


def slot_rows(a_start, a_len, a_loc, a: int, slot: int, n_slots: int = N_SLOTS) -> torch.Tensor:
    """Pool rows of adapter ``a``'s ``slot``: ``a_loc[a_start[a] + r*slot : + r]``.

    valora/csrc/bgmv/bgmv_impl.cuh:37-38 (shrink), :178 (expand);
    valora/server/router/model_infer/infer_adapter.py:139-147 (how the index is filled).
    """
    r = rank_of(a_len, a, n_slots)
    base = int(a_start[a]) + r * slot
    return a_loc[base: base + r].to(torch.long)


def dense_A(kb2d, a_start, a_len, a_loc, a, slot, n_slots=N_SLOTS, acc=torch.float32):
    """``A_a`` as ``[H_in, r]``: rank-row j is one pool row.

    test/kernel/test_kernel_correctness_multi_rank.py:99-101 ;
    valora/models/peft/lora_single_batch_infer.py:81-90.
    """
    rows = slot_rows(a_start, a_len, a_loc, a, slot, n_slots)
    return _f(kb2d[rows.to(kb2d.device)], acc).T.contiguous()


def dense_B(vb2d, a_start, a_len, a_loc, a, slot, h_out, n_slots=N_SLOTS, acc=torch.float32):
    """``B_a`` as ``[r, H_out]``: the slot's r pool rows, concatenated, hold ``[H_out, r]`` row-major.

    test/kernel/test_kernel_correctness_multi_rank.py:102-103 ;
    valora/models/peft/lora_single_batch_infer.py:91-98 ;
    valora/models/peft/layer_weights/lora_layer_weight.py:450,511-514.
    The pool row width must equal ``h_out`` (the kernels index ``W + row*feat_out``,
    valora/csrc/bgmv/bgmv_impl.cuh:191).
    """
    rows = slot_rows(a_start, a_len, a_loc, a, slot, n_slots)
    r = rows.numel()
    blk = _f(vb2d[rows.to(vb2d.device)], acc)
    assert blk.shape[1] == h_out, "pool row width must equal the wide dimension of the call"
    return blk.reshape(h_out, r).T.contiguous()


# --------------------------------------------------------------------------------------
# BGMV semantics (valora/csrc/bgmv/bgmv_impl.cuh)
# --------------------------------------------------------------------------------------
def bgmv_shrink(y, x, w, a_start, a_len, a_loc, ids, slot, n_slots=N_SLOTS, acc=torch.float32):
    """``y[t, :r] = T( sum_k f32(x[t,k]) * f32(A[j,k]) )``; columns ``>= r`` keep their old value.

    valora/csrc/bgmv/bgmv_impl.cuh:14-148 (one block per (j, t); ``if (j >= lora_rank) return``
    at :36; overwrite at :147).  Returns a new tensor; ``y`` is not modified.
    """
    T = x.dtype
    out = y.detach().to("cpu").clone()
    xw = _f(x, acc)
    w2 = w.reshape(-1, x.shape[1])
    ids_l = ids.to("cpu").tolist()
    for a in sorted(set(ids_l)):
        if a < 0:
            continue
        r = rank_of(a_len, a, n_slots)
        if r == 0:
            continue
        A = dense_A(w2, a_start, a_len, a_loc, a, slot, n_slots, acc)     # [H_in, r]
        sel = torch.tensor([i for i, v in enumerate(ids_l) if v == a], dtype=torch.long)
        out[sel, :r] = round_to(xw[sel] @ A, T)
    return out


def bgmv_expand(y, x, w, a_start, a_len, a_loc, ids, slot, scales, n_slots=N_SLOTS,
                acc=torch.float32, round_y=True):
    """``y[t,o] = T( f32(y[t,o]) + sum_{j<r} f32(x[t,j]) * f32(B[j,o]) * f32(scale[a]) )``.

    valora/csrc/bgmv/bgmv_impl.cuh:152-207: lanes with ``j >= r`` contribute zero (:186-188),
    scale is read as T and widened (:180,197), the read-modify-write rounds once (:205-207).
    ``round_y=False`` returns the accumulator before that last rounding (what the tolerance
    accounting of the parity tests places between two neighbouring T values).
    """
    T = y.dtype
    h_out = y.shape[1]
    out = _f(y, acc).clone()
    xv = _f(x, acc)
    w2 = w.reshape(-1, h_out)
    ids_l = ids.to("cpu").tolist()
    for a in sorted(set(ids_l)):
        if a < 0:
            continue
        r = rank_of(a_len, a, n_slots)
        if r == 0:
            continue
        B = dense_B(w2, a_start, a_len, a_loc, a, slot, h_out, n_slots, acc)  # [r, H_out]
        sel = torch.tensor([i for i, v in enumerate(ids_l) if v == a], dtype=torch.long)
        s = _f(scales, acc)[a]
        out[sel] += (xv[sel, :r] @ B) * s
    return round_to(out, T) if round_y else out


def dispatch_bgmv(y, x, w, a_start, a_len, a_loc, ids, qkvo, scales):
    """The 9-argument entry point: direction chosen by ``h_in < h_out``.

    valora/csrc/lora_ops.cc:76-126 (checks), valora/csrc/bgmv/bgmv_impl.cuh:221 (direction).
    Returns the new ``y``.
    """
    if y.dim() != 2 or x.dim() != 2:
        raise RuntimeError("y and x must be 2D tensors")
    if w.dim() != 3:
        raise RuntimeError("w must be a 3D tensor")
    if ids.dim() != 1:
        raise RuntimeError("indicies must be a 1D tensor")
    if ids.shape[0] != x.shape[0] or y.shape[0] != x.shape[0]:
        raise RuntimeError("CHECK_EQ failed")
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"No suitable kernel. h_in={x.shape[1]} h_out={y.shape[1]} dtype={x.dtype}")
    if x.shape[1] < y.shape[1]:
        return bgmv_expand(y, x, w, a_start, a_len, a_loc, ids, qkvo, scales)
    return bgmv_shrink(y, x, w, a_start, a_len, a_loc, ids, qkvo)


def lora_op(y, x, kb, vb, a_start, a_len, a_loc, ids, slot, scales, n_slots=N_SLOTS,
            acc=torch.float32, round_v=True, round_y=True):
    """Shrink then expand with the intermediate held exactly as the reference holds it.

    The reference stores ``delta`` as a T tensor between the two launches
    (valora/models/peft/lora_unordered_batch_infer.py:304-308, 632-638), so ``round_v=True``
    rounds v to T.  ``round_v=False`` keeps v in the accumulator type (a tighter bound used to
    report how far both implementations are from exact arithmetic).
    """
    T = x.dtype
    R = max([rank_of(a_len, a, n_slots) for a in set(ids.tolist()) if a >= 0] + [8])
    if round_v:
        v = torch.zeros(x.shape[0], R, dtype=T)
        v = bgmv_shrink(v, x, kb, a_start, a_len, a_loc, ids, slot, n_slots, acc)
        return bgmv_expand(y, v, vb, a_start, a_len, a_loc, ids, slot, scales, n_slots, acc, round_y)
    out = _f(y, acc).clone()
    ids_l = ids.tolist()
    for a in sorted(set(ids_l)):
        if a < 0 or rank_of(a_len, a, n_slots) == 0:
            continue
        A = dense_A(kb.reshape(-1, x.shape[1]), a_start, a_len, a_loc, a, slot, n_slots, acc)
        B = dense_B(vb.reshape(-1, y.shape[1]), a_start, a_len, a_loc, a, slot, y.shape[1], n_slots, acc)
        sel = torch.tensor([i for i, v_ in enumerate(ids_l) if v_ == a], dtype=torch.long)
        out[sel] += (_f(x, acc)[sel] @ A) @ B * _f(scales, acc)[a]
    return out  # not rounded: exact-arithmetic yardstick


# --------------------------------------------------------------------------------------
# PyTorch per-segment path (valora/models/bmm/lora_bmm_infer.py)
# --------------------------------------------------------------------------------------
def per_segment_mm(y, x, A_list, B_list, seg_bounds: Sequence[Tuple[int, int, int]], scalings,
                   compute_dtype: Optional[torch.dtype] = None):
    """``y[s:e] += mm(mm(x[s:e], A_i), B_i) * scaling_i`` for each ``(s, e, i)``.

    valora/models/bmm/lora_bmm_infer.py:342-352 (q), :354-379 (k, v), :425-435 (o).  Dense
    ``A_i [H_in, R]``, ``B_i [R, H_out]`` (zero-padded to the max rank at :34-48).  With
    ``compute_dtype=None`` the matmuls run in the tensors' own dtype on CPU exactly like the
    reference's tensors would (intermediates rounded to T by ``torch.mm``); pass
    ``torch.float32`` to run fp32 arithmetic on the T-rounded inputs.  This is also what the
    bench times as the CPU baseline.
    """
    out = y.clone()
    for (s, e, i) in seg_bounds:
        if e <= s:
            continue
        xs = x[s:e]
        if compute_dtype is None:
            out[s:e] += torch.mm(torch.mm(xs, A_list[i]), B_list[i]) * scalings[i]
        else:
            d = torch.mm(torch.mm(xs.to(compute_dtype), A_list[i].to(compute_dtype)),
                         B_list[i].to(compute_dtype)) * float(scalings[i])
            out[s:e] = (out[s:e].to(compute_dtype) + d).to(y.dtype)
    return out


def segments_from_ids(ids: Sequence[int]) -> List[Tuple[int, int, int]]:
    """Maximal runs of equal adapter id as ``(start, end, adapter)`` -- how the reference's bmm
    path sees a batch after ``adapter_sep`` compression
    (valora/server/router/model_infer/model_rpc.py:415-428)."""
    out, s = [], 0
    for a, grp in itertools.groupby(ids):
        n = len(list(grp))
        out.append((s, s + n, int(a)))
        s += n
    return out


# --------------------------------------------------------------------------------------
# Triton-style per-request entry points (valora/models/peft/triton_kernel/lora/lora_prefill.py)
# --------------------------------------------------------------------------------------
def _ids_from_requests(total_rows, b_start_loc, b_seq_len, b_indicies):
    ids = torch.full((total_rows,), -1, dtype=torch.long)
    for i in range(len(b_seq_len)):
        s, n = int(b_start_loc[i]), int(b_seq_len[i])
        ids[s: s + n] = int(b_indicies[i])
    return ids


def triton_shrink(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies,
                  hidden_size, qkvo, max_rank, max_input_len):
    """lora_prefill.py:56-102,139-163.  Differences from BGMV shrink that are observable: every
    column ``< max_rank`` of a covered row is stored, columns ``>= r`` as zero (the weight load
    is masked, the store is not, :89,96-100); rows beyond ``max_input_len`` of a request are
    not visited (grid z, :147)."""
    out = o.clone()
    for i in range(len(b_seq_len)):
        a = int(b_indicies[i])
        r = int(b_lora_ranks[a]) // N_SLOTS
        s = int(b_start_loc[i])
        n = min(int(b_seq_len[i]), -(-max_input_len // 32) * 32)
        if n <= 0:
            continue
        A = dense_A(w.reshape(-1, hidden_size), b_lora_start, b_lora_ranks, b_loc, a, qkvo)
        block_n = 16 if max_rank > 8 else max_rank
        width = -(-max_rank // block_n) * block_n
        width = min(width, o.shape[1])
        v = torch.zeros(n, width, dtype=torch.float32)
        v[:, :min(r, width)] = (_f(x)[s: s + n] @ A)[:, :min(r, width)]
        out[s: s + n, :width] = round_to(v, o.dtype)
    return out


def triton_expand(x, w, o, scale, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len,
                  b_indicies, feat_out, qkvo, max_rank, max_input_len):
    """lora_prefill.py:9-54,105-135: ``out += dot(x, w) * scale[a]`` per request tile."""
    acc = _f(o).clone()
    for i in range(len(b_seq_len)):
        a = int(b_indicies[i])
        r = int(b_lora_ranks[a]) // N_SLOTS
        s = int(b_start_loc[i])
        n = min(int(b_seq_len[i]), -(-max_input_len // 32) * 32)
        if n <= 0 or r == 0:
            continue
        B = dense_B(w.reshape(-1, feat_out), b_lora_start, b_lora_ranks, b_loc, a, qkvo, feat_out)
        acc[s: s + n] += (_f(x)[s: s + n, :r] @ B) * _f(scale)[a]
    return round_to(acc, o.dtype)


# --------------------------------------------------------------------------------------
# ATMM (atmm/valora/csrc/bgmv/bgmv_impl.cuh)
# --------------------------------------------------------------------------------------
def sgmm_canonical(y, x, w, a_start, a_len, a_loc, ids, qkvo, scales, output_counts, start_ids,
                   num_problems):
    """Segmented op with the canonical layouts: rows of problems ``i < P`` are processed with
    the adapter of their per-token id; rows outside every problem are untouched.  Direction as
    in ``dispatch_bgmv``.  (Signature: atmm/valora/csrc/lora_ops.cc:115-122.)"""
    T_rows = x.shape[0]
    eff = torch.full((T_rows,), -1, dtype=torch.long)
    for i in range(int(num_problems)):
        s, n = int(start_ids[i]), int(output_counts[i])
        e = min(s + n, T_rows)
        if s < T_rows and n > 0:
            eff[s:e] = ids[s:e]
    if x.shape[1] < y.shape[1]:
        return bgmv_expand(y, x, w, a_start, a_len, a_loc, eff, qkvo, scales)
    return bgmv_shrink(y, x, w, a_start, a_len, a_loc, eff, qkvo)


def count_consecutive_requests(lora_rank: torch.Tensor, indicies: torch.Tensor):
    """Run-length encoding of the per-token adapter ids.

    atmm/valora/csrc/bgmv/bgmv_impl.cuh:39-72: single-thread loop; for run k it writes
    ``output_counts[k]`` (length), ``rank_counts[k] = lora_rank[id]/4``, ``lora_ids[k] = id``,
    ``start_ids[k]`` (first token).  Returns the four lists (only the written prefix)."""
    ids = indicies.tolist()
    n = len(ids)
    oc, rc, li, st = [], [], [], []
    cur, start = 1, 0
    for i in range(1, n):
        if ids[i] == ids[i - 1]:
            cur += 1
        else:
            oc.append(cur); rc.append(int(lora_rank[ids[i - 1]]) // 4); li.append(ids[i - 1]); st.append(start)
            start = i
            cur = 1
    oc.append(cur); rc.append(int(lora_rank[ids[n - 1]]) // 4); li.append(ids[n - 1]); st.append(start)
    return oc, rc, li, st


# --------------------------------------------------------------------------------------
# host segment builder (valora/server/router/model_infer/model_rpc.py:265-375)
# --------------------------------------------------------------------------------------
def set_sgmm_args(adapter_dirs: Sequence[str], input_lengths: Sequence[int], is_prefill: bool,
                  merged_adapter_dir: Optional[str]):
    """Literal loop restatement.  Returns ``(output_counts, lora_ids, start_ids, num_problems)``
    as int64 tensors + the python list, or ``None`` where the reference's ``except`` swallows an
    error (more than 128 runs overflow the fixed buffers, model_rpc.py:267-270,373-374)."""
    N = 128
    output_counts = torch.ones(N, dtype=torch.long)
    lora_ids = torch.zeros(N, dtype=torch.long)
    start_ids = torch.ones(N, dtype=torch.long)
    n = len(adapter_dirs)
    try:
        current_count = 0
        de_lora = 1
        flag = True
        num_problems = [0, [0, 0]]

        def L(i):
            return int(input_lengths[i]) if is_prefill else 1

        req_len = L(0)
        if n == 1:
            output_counts[current_count] = req_len
            start_ids[current_count] = 0
            num_problems[0] = 1
            return output_counts, lora_ids, start_ids, num_problems
        for i in range(1, n):
            if adapter_dirs[i - 1] == adapter_dirs[i]:
                req_len += L(i)
                de_lora += 1
            else:
                probe = adapter_dirs[i - 1] if is_prefill else adapter_dirs[i]   # :292 vs :337
                if probe == merged_adapter_dir and flag:
                    num_problems[1][0] = de_lora
                    num_problems[1][1] = req_len
                flag = False
                num_problems[0] += 1
                output_counts[current_count] = req_len
                req_len = L(i)
                current_count += 1
        if adapter_dirs[-1] == merged_adapter_dir and flag:
            num_problems[1][0] = de_lora
            num_problems[1][1] = req_len
        num_problems[0] += 1
        output_counts[current_count] = req_len
        if num_problems[1][1] > 0:
            output_counts = output_counts[1:]
        start_ids = torch.cat((torch.tensor([0], dtype=torch.long), torch.cumsum(output_counts, dim=0)))
        if not is_prefill:
            num_problems[1][0] = 0
            num_problems[1][1] = 0
        return output_counts, lora_ids, start_ids, num_problems
    except Exception:  # the reference prints and falls through to an implicit ``return None``
        return None


def batch_req_bins(req_bins: torch.Tensor, b_seq_len: torch.Tensor) -> torch.Tensor:
    """valora/models/peft/lora_unordered_batch_infer.py:291-293."""
    return torch.repeat_interleave(req_bins.to(torch.long), b_seq_len.to(torch.long))


# --------------------------------------------------------------------------------------
# error metrics used by the parity tests
# --------------------------------------------------------------------------------------
def max_abs(a, b) -> float:
    return float((_f(a, torch.float64) - _f(b, torch.float64)).abs().max()) if a.numel() else 0.0


def rel_l2(a, b) -> float:
    a64, b64 = _f(a, torch.float64), _f(b, torch.float64)
    den = float(b64.norm())
    return float((a64 - b64).norm()) / den if den > 0 else float((a64 - b64).norm())


def merge_weight(W: torch.Tensor, A: torch.Tensor, B: torch.Tensor, scaling: float, sign: int = 1) -> torch.Tensor:
    """``W +- bmm(A, B * scaling)`` with the reference's rounding points: ``b = B * scaling`` is a T
    tensor, the GEMM accumulates in fp32 and stores T, ``add_`` / ``sub_`` round once more.
    ``W [H_in, H_out]``, ``A [H_in, r]``, ``B [r, H_out]``.

    valora/models/peft/lora_single_batch_infer.py:113-123 (merge), :137-146 (unmerge).
    """
    T = W.dtype
    b = (B.to(torch.float32) * float(scaling)).to(T)
    ab = (A.to(torch.float32) @ b.to(torch.float32)).to(T)
    return (W.to(torch.float32) + float(sign) * ab.to(torch.float32)).to(T)


def merge_adapter(weights, kb, vb, a_start, a_len, a_loc, adapter, scaling, slots=(0, 1, 2, 3), n_slots=N_SLOTS,
                  sign: int = 1):
    """The four (or fewer) weights of one layer with adapter ``adapter`` merged in (or taken out): A and
    B of each slot are read back from the pool as the reference does
    (lora_single_batch_infer.py:81-98: ``key_buffer[loc[s*r:(s+1)*r]].reshape(r, H).T`` and
    ``value_buffer[...].reshape(H, r).T``).  Returns new tensors."""
    r = int(a_len[adapter]) // n_slots
    start = int(a_start[adapter])
    out = []
    for W, slot in zip(weights, slots):
        rows = a_loc[start + slot * r: start + (slot + 1) * r]
        h_in, h_out = W.shape
        A = kb.reshape(-1, h_in)[rows].reshape(r, h_in).transpose(0, 1)
        B = vb.reshape(-1, h_out)[rows].reshape(h_out, r).transpose(0, 1)
        out.append(merge_weight(W, A, B, scaling, sign))
    return out


def delora_compensate(y, x, kb, vb, a_start, a_len, a_loc, ids, merged, slot, scales, n_slots=N_SLOTS):
    """While adapter ``merged`` sits in the base weights, tokens of the other adapters get
    ``+ LoRA(own) - LoRA(merged)``; tokens of the merged adapter and tokens without adapter are
    left alone.  valora/models/peft/lora_unordered_batch_infer.py:991-1063 (the reference runs the
    two halves as one doubled batch and adds ``first half - second half``)."""
    ids = torch.as_tensor(ids, dtype=torch.long)
    other = (ids != merged) & (ids >= 0) & (ids < a_start.numel())
    own_ids = torch.where(other, ids, torch.full_like(ids, -1))
    mrg_ids = torch.where(other, torch.full_like(ids, merged), torch.full_like(ids, -1))
    y1 = lora_op(y, x, kb, vb, a_start, a_len, a_loc, own_ids, slot, scales, n_slots=n_slots)
    return lora_op(y1, x, kb, vb, a_start, a_len, a_loc, mrg_ids, slot, -scales, n_slots=n_slots)
