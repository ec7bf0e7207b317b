"""Writes tests/golden/segments.json: known-answer vectors for the host segment builder.

Every case was derived BY HAND from the text of the reference's ``set_sgmm_args``
(valora/server/router/model_infer/model_rpc.py:265-375) -- walking the loop on paper -- and is
recorded here as the hand-derived prefix plus the rule for the untouched tail of the fixed
128-entry buffers (``output_counts`` tail = 1, ``start_ids`` tail = previous + 1 after the
cumulative sum, or 1 on the single-request early return).  No oracle or product code is used.
"""
import json
import os

N = 128


def oc_full(prefix, length):
    return list(prefix) + [1] * (length - len(prefix))


def st_cumsum(oc):
    out, s = [0], 0
    for v in oc:
        s += v
        out.append(s)
    return out


cases = []

# (i) a single prefill request: early return, start_ids = [0, 1, 1, ...]
cases.append(dict(name="single_prefill", dirs=["A"], lens=[7], prefill=True, merged=None,
                  oc=oc_full([7], N), st=[0] + [1] * (N - 1), num_problems=[1, [0, 0]]))
cases.append(dict(name="single_decode", dirs=["A"], lens=[7], prefill=False, merged="A",
                  oc=oc_full([1], N), st=[0] + [1] * (N - 1), num_problems=[1, [0, 0]]))

# (ii) all requests on one adapter
oc = oc_full([15], N)
cases.append(dict(name="all_same_prefill", dirs=["A", "A", "A"], lens=[5, 7, 3], prefill=True, merged=None,
                  oc=oc, st=st_cumsum(oc), num_problems=[1, [0, 0]]))
# ... and that adapter is the merged one: the only count is dropped before the cumulative sum
oc = oc_full([], N - 1)
cases.append(dict(name="all_same_merged_prefill", dirs=["A", "A", "A"], lens=[5, 7, 3], prefill=True, merged="A",
                  oc=oc, st=st_cumsum(oc), num_problems=[1, [3, 15]]))

# (iii) A A B B C, prefill lengths 5 7 3 2 9
oc = oc_full([12, 5, 9], N)
cases.append(dict(name="aabbc_prefill", dirs=["A", "A", "B", "B", "C"], lens=[5, 7, 3, 2, 9], prefill=True,
                  merged=None, oc=oc, st=st_cumsum(oc), num_problems=[3, [0, 0]]))

# (iv) leading run is the merged adapter (prefill tests the adapter BEFORE the boundary)
oc = oc_full([3, 2], N - 1)
cases.append(dict(name="leading_merged_prefill", dirs=["M", "M", "B", "C"], lens=[4, 6, 3, 2], prefill=True,
                  merged="M", oc=oc, st=st_cumsum(oc), num_problems=[3, [2, 10]]))
# merged adapter appears later only: nothing is dropped
oc = oc_full([4, 9, 2], N)
cases.append(dict(name="late_merged_prefill", dirs=["B", "M", "M", "C"], lens=[4, 6, 3, 2], prefill=True,
                  merged="M", oc=oc, st=st_cumsum(oc), num_problems=[3, [0, 0]]))

# (v) decode tests the adapter AFTER the first boundary: A | M M | B with merged = M drops the
#     first count although the leading run is A, then reports [0, 0]
oc = oc_full([2, 1], N - 1)
cases.append(dict(name="decode_quirk_second_run_merged", dirs=["A", "M", "M", "B"], lens=[9, 9, 9, 9],
                  prefill=False, merged="M", oc=oc, st=st_cumsum(oc), num_problems=[3, [0, 0]]))
# decode with the leading run merged: the probe looks at B, nothing dropped
oc = oc_full([2, 1], N)
cases.append(dict(name="decode_leading_merged", dirs=["M", "M", "B"], lens=[3, 3, 3], prefill=False,
                  merged="M", oc=oc, st=st_cumsum(oc), num_problems=[2, [0, 0]]))

# (vi) exactly 128 runs fit; 129 runs overflow the buffers -> the reference returns None
dirs128 = ["A" if i % 2 == 0 else "B" for i in range(128)]
oc = [2] * 128
cases.append(dict(name="128_runs_prefill", dirs=dirs128, lens=[2] * 128, prefill=True, merged=None,
                  oc=oc, st=st_cumsum(oc), num_problems=[128, [0, 0]]))
dirs129 = ["A" if i % 2 == 0 else "B" for i in range(129)]
cases.append(dict(name="129_runs_prefill", dirs=dirs129, lens=[2] * 129, prefill=True, merged=None,
                  oc=None, st=None, num_problems=None))

here = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(here, "segments.json"), "w") as f:
    json.dump(dict(source="hand-derived from valora/server/router/model_infer/model_rpc.py:265-375",
                   cases=cases), f)
print(len(cases), "cases")
