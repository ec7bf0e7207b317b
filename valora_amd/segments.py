"""Segment / adapter-index tensors that drive the multi-LoRA op.

* ``set_sgmm_args``            host-side segment builder, same outputs as the reference's
                               ``ModelRpcServer.set_sgmm_args``
                               (valora/server/router/model_infer/model_rpc.py:265-375)
* ``count_consecutive_requests`` run-length encoding of per-token ids on the GPU, same outputs
                               as the reference's device kernel
                               (atmm/valora/csrc/bgmv/bgmv_impl.cuh:39-72)
* ``batch_req_bins``           per-token ids from per-request ids
                               (valora/models/peft/lora_unordered_batch_infer.py:291-293)
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _lib

SGMM_BUFFER_LEN = 128  # model_rpc.py:267


def set_sgmm_args(adapter_dirs: Sequence[str], input_lengths: Sequence[int], is_prefill: bool,
                  merged_adapter_dir: Optional[str], device="cpu"
                  ) -> Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor, List]]:
    """Run-length encode consecutive requests that share an adapter.

    Returns ``(output_counts, lora_ids, start_ids, num_problems)`` with
    ``num_problems = [n_runs, [requests_in_leading_merged_run, tokens_in_it]]`` or ``None`` when
    the batch has more runs than the fixed 128-entry buffers hold (the reference swallows the
    resulting IndexError and returns None, model_rpc.py:373-374).

    Behaviours kept on purpose because callers depend on the exact tensors:
    buffers are 128 long and pre-filled with ones (``lora_ids`` with zeros and never written);
    a single request returns early with ``start_ids = [0, 1, 1, ...]``; when the leading run
    belongs to the merged adapter the first count is dropped before the cumulative sum; prefill
    tests the adapter *before* the first boundary and decode the one *after* it; decode reports
    ``[0, 0]`` for the merged run after having used it.
    """
    n = len(adapter_dirs)
    if n == 0:
        return None  # input_lengths[0] raises in the reference
    N = SGMM_BUFFER_LEN
    lens = (np.asarray(list(input_lengths)[:n], dtype=np.int64) if is_prefill
            else np.ones(n, dtype=np.int64))
    oc = np.ones(N, dtype=np.int64)
    lora_ids = torch.zeros(N, dtype=torch.long, device=device)
    if n == 1:
        oc[0] = lens[0]
        st = np.ones(N, dtype=np.int64)
        st[0] = 0
        return (torch.from_numpy(oc).to(device), lora_ids, torch.from_numpy(st).to(device), [1, [0, 0]])

    # intern the directory names, then find run boundaries
    table = {}
    codes = np.fromiter((table.setdefault(d, len(table)) for d in adapter_dirs), dtype=np.int64, count=n)
    heads = np.flatnonzero(np.concatenate(([True], codes[1:] != codes[:-1])))
    P = int(heads.size)
    if P > N:
        return None
    run_tokens = np.add.reduceat(lens, heads)
    oc[:P] = run_tokens
    merged = [0, 0]
    merged_code = table.get(merged_adapter_dir, -1)  # a None directory compares equal to None, as in Python
    first_run_reqs = int(heads[1]) if P > 1 else n
    if P == 1:
        if codes[-1] == merged_code:
            merged = [n, int(run_tokens[0])]
    else:
        probe = codes[heads[1] - 1] if is_prefill else codes[heads[1]]
        if probe == merged_code:
            merged = [first_run_reqs, int(run_tokens[0])]
    if merged[1] > 0:
        oc = oc[1:]
    st = np.concatenate(([0], np.cumsum(oc)))
    if not is_prefill:
        merged = [0, 0]
    return (torch.from_numpy(oc.copy()).to(device), lora_ids, torch.from_numpy(st).to(device), [P, merged])


def batch_req_bins(req_bins: torch.Tensor, b_seq_len: torch.Tensor) -> torch.Tensor:
    return torch.repeat_interleave(req_bins.to(torch.long), b_seq_len.to(torch.long))


def count_consecutive_requests(lora_rank: torch.Tensor, indicies: torch.Tensor):
    """GPU run-length encoding.  ``lora_rank`` holds ``4 * r`` per adapter (the ``a_len`` tensor).

    Returns ``(output_counts, rank_counts, lora_ids, start_ids, num_runs)``: four int64 device
    tensors of length ``T`` of which the first ``num_runs`` entries are meaningful, and the run
    count as a 1-element device tensor (no host synchronisation happens here).
    """
    if not indicies.is_cuda or not lora_rank.is_cuda:
        raise RuntimeError("indicies and lora_rank must be CUDA tensors")
    if indicies.dtype != torch.long or lora_rank.dtype != torch.long:
        raise RuntimeError("expected scalar type Long")
    if not indicies.is_contiguous() or not lora_rank.is_contiguous():
        raise RuntimeError("indicies and lora_rank must be contiguous")
    T = indicies.numel()
    dev = indicies.device
    out = torch.zeros(4, max(T, 1), dtype=torch.long, device=dev)
    num = torch.zeros(1, dtype=torch.long, device=dev)
    _lib.check(_lib.lib().mlora_count_consecutive(
        _lib.current_stream(dev), _lib.ptr(lora_rank), lora_rank.numel(), _lib.ptr(indicies), T,
        _lib.ptr(out[0]), _lib.ptr(out[1]), _lib.ptr(out[2]), _lib.ptr(out[3]), _lib.ptr(num)))
    return out[0], out[1], out[2], out[3], num
