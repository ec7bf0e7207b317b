"""Writes tests/golden/pool_index.json: known-answer vectors for the pool row allocator and the
adapter index tensors.

Every case was worked out BY HAND from the text of the reference
(valora/common/mem_allocator.py:30-75,203-217 and
valora/server/router/model_infer/infer_adapter.py:94-256): the row states are written as strings
('1' = free, '0' = taken), the expected results are literals.  No oracle or product code is used.
"""
import json
import os

alloc_cases = [
    # first fit takes the first `need` free rows in index order
    dict(name="fresh", state="11111111", op="alloc", need=3, index=[0, 1, 2], after="00011111"),
    dict(name="holes", state="01001101", op="alloc", need=3, index=[1, 4, 5], after="00000001"),
    dict(name="all_free_rows", state="01001101", op="alloc", need=4, index=[1, 4, 5, 7], after="00000000"),
    dict(name="zero", state="0110", op="alloc", need=0, index=[], after="0110"),
    dict(name="last_row_only", state="00000001", op="alloc", need=1, index=[7], after="00000000"),
    # contiguous: the first window of `need` free rows; None (state untouched) when there is none
    dict(name="contig_first_window", state="11011101", op="alloc_contiguous", need=3, start=3, index=[3, 4, 5],
         after="11000001"),
    dict(name="contig_prefers_earliest", state="11101111", op="alloc_contiguous", need=2, start=0, index=[0, 1],
         after="00101111"),
    dict(name="contig_at_end", state="01010011", op="alloc_contiguous", need=2, start=6, index=[6, 7],
         after="01010000"),
    dict(name="contig_none", state="11011011", op="alloc_contiguous", need=3, start=None, index=None,
         after="11011011"),
    dict(name="contig_whole_pool", state="1111", op="alloc_contiguous", need=4, start=0, index=[0, 1, 2, 3],
         after="0000"),
    dict(name="contig_one", state="0010", op="alloc_contiguous", need=1, start=2, index=[2], after="0000"),
    # free marks rows free again, duplicates and already-free rows are harmless
    dict(name="free_some", state="00000000", op="free", index=[5, 1, 1, 6], after="01000110"),
]

# A residency history on a pool of 40 rows, n_slots = 4.  Adapters: X r=2 (8 rows), Y r=1 (4 rows),
# Z r=3 (12 rows), W r=2 (8 rows).
#  1. load [X, Y, Z]: one alloc(24) -> rows 0..23; a_start = [0, 8, 12], a_len = [8, 4, 12].
#  2. offload keeping [X, Z]: Y's rows 8..11 are freed; a_loc = rows 0..7 then 12..23,
#     a_start = [0, 8], a_len = [8, 12]; free rows: 8..11 and 24..39 (20 rows).
#  3. load [W, X]: X is resident, W needs 8 rows -> first fit takes 8, 9, 10, 11, 24, 25, 26, 27;
#     a_start = [0, 8, 20], a_len = [8, 12, 8]; a_loc gains those 8 rows at the end.
#  4. offload keeping [W]: X and Z go; a_loc = W's rows, a_start = [0], a_len = [8];
#     free rows = 40 - 8 = 32.
#  5. offload keeping []: everything is freed.
history = dict(
    tot_size=40, n_slots=4,
    adapters=dict(X=dict(r=2, scaling=2.0), Y=dict(r=1, scaling=0.5), Z=dict(r=3, scaling=1.0),
                  W=dict(r=2, scaling=4.0)),
    steps=[
        dict(op="load", dirs=["X", "Y", "Z"],
             adapter_dirs=["X", "Y", "Z"], a_start=[0, 8, 12], a_len=[8, 4, 12], a_loc=list(range(24)),
             a_scaling=[2.0, 0.5, 1.0], free=16),
        dict(op="offload", reserve=["X", "Z"],
             adapter_dirs=["X", "Z"], a_start=[0, 8], a_len=[8, 12], a_loc=list(range(8)) + list(range(12, 24)),
             a_scaling=[2.0, 1.0], free=20),
        dict(op="load", dirs=["W", "X"],
             adapter_dirs=["X", "Z", "W"], a_start=[0, 8, 20], a_len=[8, 12, 8],
             a_loc=list(range(8)) + list(range(12, 24)) + [8, 9, 10, 11, 24, 25, 26, 27],
             a_scaling=[2.0, 1.0, 4.0], free=12),
        dict(op="offload", reserve=["W"],
             adapter_dirs=["W"], a_start=[0], a_len=[8], a_loc=[8, 9, 10, 11, 24, 25, 26, 27],
             a_scaling=[4.0], free=32),
        dict(op="offload", reserve=[],
             adapter_dirs=[], a_start=[], a_len=[], a_loc=[], a_scaling=[], free=40),
    ])

# Prefetch tags (infer_adapter.py:101-113,199-206): a prefetch flips cur_tag and tags every adapter
# it names; an offload keeps adapters tagged by the LATEST prefetch even when they are not reserved.
#  pool 24 rows; P r=1, Q r=1, R r=1 (4 rows each).
#  1. load [P] (normal).  2. prefetch [Q, R] -> cur_tag = 1, tags Q = R = 1.
#  3. offload reserve [P, Q]: P, Q reserved, R kept by its tag -> nothing leaves
#     (3 names kept == 3 resident; the early return on equal lengths does not fire since 2 != 3).
#  4. prefetch [P] -> cur_tag = 0, tag P = 0; Q, R still carry tag 1.
#  5. offload reserve [Q, X?]: lengths differ from 3 -> scan: P kept by tag 0 == cur_tag, Q reserved, R leaves.
prefetch_history = dict(
    tot_size=24, n_slots=4,
    adapters=dict(P=dict(r=1, scaling=1.0), Q=dict(r=1, scaling=2.0), R=dict(r=1, scaling=3.0)),
    steps=[
        dict(op="load", dirs=["P"], adapter_dirs=["P"], a_start=[0], a_len=[4], a_loc=[0, 1, 2, 3],
             a_scaling=[1.0], free=20),
        dict(op="prefetch", dirs=["Q", "R"], adapter_dirs=["P", "Q", "R"], a_start=[0, 4, 8], a_len=[4, 4, 4],
             a_loc=list(range(12)), a_scaling=[1.0, 2.0, 3.0], free=12),
        dict(op="offload", reserve=["P", "Q"], adapter_dirs=["P", "Q", "R"], a_start=[0, 4, 8], a_len=[4, 4, 4],
             a_loc=list(range(12)), a_scaling=[1.0, 2.0, 3.0], free=12),
        dict(op="prefetch", dirs=["P"], adapter_dirs=["P", "Q", "R"], a_start=[0, 4, 8], a_len=[4, 4, 4],
             a_loc=list(range(12)), a_scaling=[1.0, 2.0, 3.0], free=12),
        dict(op="offload", reserve=["Q", "not-resident"], adapter_dirs=["P", "Q"], a_start=[0, 4], a_len=[4, 4],
             a_loc=list(range(8)), a_scaling=[1.0, 2.0], free=16),
    ])

out = dict(alloc_cases=alloc_cases, history=history, prefetch_history=prefetch_history)
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "pool_index.json")
with open(path, "w") as f:
    json.dump(out, f, indent=1)
print("wrote", path)
