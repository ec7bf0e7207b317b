/* mlora.h -- C ABI of the MI355X (gfx950) multi-LoRA batching operator.
 *
 * Plain pointers and sizes only; every pointer marked "device" is device memory owned by the
 * caller, every launch goes on the caller's stream, the library allocates nothing and keeps no
 * state between calls.  Every function returns MLORA_OK (0) or a negative mlora_status;
 * mlora_last_error() then returns a message for the calling thread.
 *
 * Citations name the reference interface each entry point replaces (paths relative to the
 * mi150/VaLoRA checkout).
 */
#ifndef MLORA_H_
#define MLORA_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { MLORA_F16 = 0, MLORA_BF16 = 1 } mlora_dtype;

#define MLORA_MAX_TARGETS 4   /* targets one mlora_lora_apply_multi call can take */

typedef enum {
  MLORA_OK = 0,
  MLORA_ERR_INVALID = -1,     /* bad argument (null pointer, negative size, misaligned base) */
  MLORA_ERR_NO_KERNEL = -2,   /* "No suitable kernel." -- valora/csrc/lora_ops.cc:124-125 */
  MLORA_ERR_WORKSPACE = -3,   /* workspace or plan buffer too small */
  MLORA_ERR_LAUNCH = -4       /* the HIP runtime refused a launch */
} mlora_status;

/* Behaviour switches of the shrink store (see mlora_shrink). */
enum {
  MLORA_SHRINK_OVERWRITE = 0, /* y[t,:r] = v, columns >= r untouched (BGMV, bgmv_impl.cuh:36,147) */
  MLORA_SHRINK_ZERO_PAD = 1,  /* y[t,:width] = v, zero for columns >= r (Triton, lora_prefill.py:89,96-100) */
  MLORA_SHRINK_ACCUMULATE = 2 /* y[t,:r] += v (ATMM beta = 1, atmm/.../bgmv_impl.cuh:174) */
};

/* flags of mlora_shrink / mlora_expand / mlora_lora_apply */
enum {
  MLORA_REDUCE_IN_EXPAND = 1, /* split-K chunks are summed by the expand launch instead of by a
                                 separate reduce launch: one launch fewer for small batches, more
                                 re-reads for large ones.  Must be given to both launches of a pair,
                                 with the same ksplit.                                            */
  MLORA_ONE_LAUNCH = 2,       /* mlora_lora_apply / mlora_lora_apply_multi only: shrink and expand are
                                 work items of ONE grid; an expand item requests its B and y operands,
                                 then waits (bounded: 30 us) for its tile's K-chunk partials and computes
                                 them itself if they do not come.  For decode-like batches: needs a plan
                                 cut with bm_shrink = bm_expand = 16 and max_rank <= 64; ksplit is raised
                                 to 2 if smaller and cut so that ksplit * n_targets <= 16; scratch of
                                 mlora_one_launch_scratch_bytes(), 128-byte aligned (the partials are
                                 handed over in cache lines that belong to one tile each; a scratch
                                 buffer aligned to less, an empty index or an empty pool make the call
                                 run as two launches, and so does a call with more than 16 expand items
                                 per tile -- 512-column chunks (256 above rank 32) x targets -- where two
                                 launches measured faster).  Any batch size: items the device cannot
                                 hold from the start take part in the hand-off like the others.
                                 Bit-identical to the two-launch op with MLORA_REDUCE_IN_EXPAND and the
                                 same ksplit.  Launches that share a plan must not overlap in time.  */
  MLORA_ONE_LAUNCH_NO_WAIT = 4, /* with MLORA_ONE_LAUNCH: expand items do not wait at all and always
                                 compute their tile's partials themselves (the give-up path made
                                 testable; same results, slower)                                  */
  MLORA_SHRINK_RECOMPUTE = 8, /* a split-K shrink of a small batch (tiles up to 64 tokens) sums its K
                                 chunks inside the launch: the chunk of a tile that finishes last reads
                                 the others' partials out of the L2 it shares with them, or -- when they
                                 did not all run on its XCD -- computes them itself.  This flag makes
                                 every tile take the second path (made testable; same results, slower) */
  MLORA_EXPAND_COLUMN_LOOP = 16, /* expand of a plan with 16-token expand tiles: a workgroup walks over two
                                 256-column chunks of its tile instead of owning one.  The library does
                                 this by itself where the grid would otherwise be several times what the
                                 device holds (decode batches with many targets or wide outputs); the flag
                                 forces it for any size (made testable; same results)                    */
  MLORA_ONE_LAUNCH_NEVER_READY = 32  /* with MLORA_ONE_LAUNCH: expand items look for a stamp that no shrink item
                                 leaves, so every one of them waits out its bound (30 us) and then computes
                                 its tile's partials itself: the way out of the bounded wait made testable
                                 and measurable from the host; every kernel still ends normally, same
                                 results, slower                                                          */
};

/* What the kernels can vary per batch shape (see mlora_tile_lookup). */
typedef struct {
  int32_t bm_shrink;        /* tokens per shrink tile: 16, 32, 64 (direct loads), 128 or 256 (LDS-staged) */
  int32_t ksplit;           /* K chunks the shrink is split into                                      */
  int32_t bm_expand;        /* tokens per expand tile: multiple of 16 up to 256                       */
  int32_t flags;            /* MLORA_REDUCE_IN_EXPAND | MLORA_ONE_LAUNCH                              */
} mlora_tile_config;

/* Pool + adapter index operands shared by all op entry points (device pointers).
 * Semantics: valora/server/router/model_infer/infer_adapter.py:14-17,128-148.            */
typedef struct {
  const void *w;            /* pool rows, 16-bit elements, row stride = the call's wide dim     */
  int64_t w_rows;           /* number of pool rows (rows named by a_loc outside it are skipped) */
  const int64_t *a_start;   /* [n_adapters] offset into a_loc                                   */
  const int64_t *a_len;     /* [n_adapters] n_slots * rank                                      */
  const int64_t *a_loc;     /* [a_loc_len] pool row per (adapter, slot, rank row)               */
  int64_t n_adapters;
  int64_t a_loc_len;
  int32_t n_slots;          /* 4 in the reference (q,k,v,o): bgmv_impl.cuh:35                   */
} mlora_pool;

/* Host-side handle of a plan: the device buffer (caller-owned, mlora_plan_bytes() bytes) plus
 * the shape it was built for.  mlora_build_plan fills every field but dev and bytes.          */
typedef struct {
  void *dev;
  size_t bytes;
  int64_t T;
  int64_t n_adapters;
  int32_t bm_shrink;        /* tile heights in tokens the two tile lists were cut with          */
  int32_t bm_expand;
  int32_t n_slots;          /* slots per adapter of the index the plan was cut for; the op entry
                               points reject a pool whose n_adapters or n_slots differ           */
} mlora_plan;

const char *mlora_last_error(void);
int mlora_version(void);

/* ---- sizing ------------------------------------------------------------------------------ */
/* Bytes of a plan for T tokens and n_adapters adapters.                                       */
size_t mlora_plan_bytes(int64_t T, int64_t n_adapters);
/* Bytes of the scratch buffer that carries v = x*A^T from mlora_shrink to mlora_expand (a T-typed
 * [T, max_rank] matrix plus, for ksplit > 1, the fp32 split-K partials).                       */
size_t mlora_scratch_bytes(int64_t T, int64_t max_rank, int32_t ksplit);
/* Bytes of scratch a call with MLORA_ONE_LAUNCH needs (its K-chunk partials are laid out tile by tile, in
 * whole cache lines per tile, which takes more room than mlora_scratch_bytes gives).             */
size_t mlora_one_launch_scratch_bytes(int64_t T, int64_t n_adapters, int64_t max_rank, int32_t ksplit,
                                      int32_t n_targets);
/* Bytes of scratch the one-call entry points (dispatch_bgmv, dispatch_sgmm, prefill_*) need.
 * Replaces sgmm_tmp_size (atmm/valora/csrc/bgmv/bgmv_impl.cuh:128-132).                       */
size_t mlora_workspace_bytes(int64_t T, int64_t n_adapters, int64_t max_rank);

/* ---- tile selection ------------------------------------------------------------------------- */
/* The tile configuration measured for this batch shape on MI355X: key (token bucket, rank bucket,
 * hidden = wide dim of the shrink, adapter bucket); a width without entries takes those of the
 * nearest measured width, anything else a rule.  Replaces shape_to_config / get_config_a /
 * get_config_b (valora/models/peft/lora_unordered_batch_infer.py:25-172,216-236).  The one-call
 * entry points use it themselves; callers of mlora_build_plan / mlora_lora_apply pass its answer
 * on (bm_* to the plan, ksplit and flags to the op).                                          */
int mlora_tile_lookup(int64_t n_tokens, int64_t max_rank, int64_t hidden, int64_t n_adapters,
                      mlora_tile_config *out);
/* The rule alone (what a shape without table entry gets): the counterpart of the reference's
 * fixed fallback tuples (lora_unordered_batch_infer.py:224,235).                              */
int mlora_tile_fallback(int64_t n_tokens, int64_t max_rank, int64_t hidden, int64_t n_adapters,
                        mlora_tile_config *out);

/* ---- index / segment builders ------------------------------------------------------------- */
/* Adapter-grouped work tiles from per-token adapter ids (device int64[T]; an id outside
 * [0, n_adapters) or an adapter of rank 0 marks a token that gets no LoRA).  Stable counting
 * sort of the tokens by adapter + one tile list per tile height.  Replaces the host-side
 * grouping done by precompute_sgmm_args_* (atmm/valora/csrc/bgmv/bgmv_impl.cuh:76-125).
 * bm_shrink, bm_expand: tile heights in tokens (16, 32, 64, 128 or 256 -- 256 up to rank 64 -- / any multiple of 16 up to 256);
 * 0 lets the library choose.                                                                 */
int mlora_build_plan(void *stream, mlora_plan *plan, const int64_t *ids, int64_t T,
                     const int64_t *a_start, const int64_t *a_len, int64_t n_adapters,
                     int32_t n_slots, int32_t bm_shrink, int32_t bm_expand);

/* Run-length encoding of per-token ids, bit-exact with count_consecutive_requests
 * (atmm/valora/csrc/bgmv/bgmv_impl.cuh:39-72).  Outputs are device int64 arrays with room for
 * T entries; only the first *num_runs entries are written.  num_runs: device int64[1].        */
int mlora_count_consecutive(void *stream, const int64_t *lora_rank, int64_t n_adapters,
                            const int64_t *indicies, int64_t T, int64_t *output_counts,
                            int64_t *rank_counts, int64_t *lora_ids, int64_t *start_ids,
                            int64_t *num_runs);

/* ids_out[t] = ids_in[t] for rows covered by problems i < P (rows start_ids[i] ..
 * start_ids[i] + output_counts[i]), -1 elsewhere.  Turns the ATMM segment tensors
 * (atmm/valora/csrc/lora_ops.cc:115-122) into per-token ids.                                  */
int mlora_ids_from_segments(void *stream, int64_t *ids_out, const int64_t *ids_in,
                            const int64_t *start_ids, const int64_t *output_counts, int64_t P,
                            int64_t T);

/* ids_out[b_start_loc[i] + m] = b_indicies[i] for m < min(b_seq_len[i], max_rows), -1 elsewhere
 * (per-request operands of valora/models/peft/triton_kernel/lora/lora_prefill.py:105,139).    */
int mlora_ids_from_requests(void *stream, int64_t *ids_out, const int32_t *b_start_loc,
                            const int32_t *b_seq_len, const int64_t *b_indicies, int64_t n_req,
                            int64_t T, int64_t max_rows);

/* ---- planned op: shrink / expand / fused ---------------------------------------------------- */
/* v[row, j] = T( sum_k x[t, k] * A_a[j, k] ) for j < r_a, fp32 accumulation, one rounding.
 * out == NULL : v goes to `scratch` (rows in the plan's sorted order) for mlora_expand.
 * out != NULL : the caller's matrix [T, out_stride] is written in token order; `mode` is one of
 *               MLORA_SHRINK_* and `width` the number of columns ZERO_PAD fills.
 * ksplit: K-chunks computed by separate workgroups (0 = library default); the chunks are summed
 * in index order by a small second launch (or by mlora_expand, see MLORA_REDUCE_IN_EXPAND), so
 * results do not depend on scheduling.
 * Kernel semantics: valora/csrc/bgmv/bgmv_impl.cuh:14-148.                                    */
int mlora_shrink(void *stream, const mlora_plan *plan, void *scratch, size_t scratch_bytes,
                 const void *x, int64_t T, int64_t h_in, int64_t max_rank, const mlora_pool *pool,
                 int32_t slot, int32_t ksplit, void *out, int64_t out_stride, int32_t mode,
                 int32_t width, int32_t flags, mlora_dtype dtype);

/* y[t,:] = T( y[t,:] + scale[a] * v[t,:r] * B_a ), fp32 accumulation, one rounding.
 * v == NULL : v is read from `scratch` as written by mlora_shrink(out = NULL) -- pass that call's
 *             ksplit and flags.
 * v != NULL : a T matrix [T, v_stride] in token order (the reference's `delta` tensor).
 * Kernel semantics: valora/csrc/bgmv/bgmv_impl.cuh:152-207.                                   */
int mlora_expand(void *stream, const mlora_plan *plan, void *y, int64_t T, int64_t h_out,
                 const void *scratch, const void *v, int64_t v_stride, int64_t max_rank,
                 const mlora_pool *pool, int32_t slot, const void *scales, int32_t ksplit,
                 int32_t flags, mlora_dtype dtype);

/* Shrink + expand of one target in one call (two launches, v stays in `scratch`).  pool_a holds
 * the A rows (row width h_in), pool_b the B rows (row width h_out); they share the index.     */
int mlora_lora_apply(void *stream, const mlora_plan *plan, void *scratch, size_t scratch_bytes,
                     void *y, const void *x, int64_t T, int64_t h_in, int64_t h_out,
                     int64_t max_rank, const mlora_pool *pool_a, const mlora_pool *pool_b,
                     int32_t slot, const void *scales, int32_t ksplit, int32_t flags,
                     mlora_dtype dtype);

/* One output of a multi-target call: y += scale * v_slot * B_slot. */
typedef struct {
  void *y;                  /* [T, h_out], updated in place                                      */
  const void *w_b;          /* value buffer holding this target's B rows (row width h_out)        */
  int64_t w_b_rows;
  int32_t slot;             /* slot of the adapter index this target uses (A rows and B rows)     */
} mlora_target;

/* Shrink + expand for several targets that read the same x (q, k, v of one layer; gate and up):
 * one shrink launch for all targets, one expand launch for all targets.  The targets share h_in,
 * h_out, the key buffer and the adapter index of pool_a; each has its own y, value buffer and slot.
 * Replaces the reference's 3 + 3 launches per attention block
 * (valora/models/peft/lora_unordered_batch_infer.py:946-988).  scratch_bytes must be at least
 * n_targets * mlora_scratch_bytes(T, max_rank, ksplit).  Results are identical to n_targets
 * separate mlora_lora_apply calls.                                                              */
int mlora_lora_apply_multi(void *stream, const mlora_plan *plan, void *scratch, size_t scratch_bytes,
                           const void *x, int64_t T, int64_t h_in, int64_t h_out, int64_t max_rank,
                           const mlora_pool *pool_a, int32_t n_targets, const mlora_target *targets,
                           const void *scales, int32_t ksplit, int32_t flags, mlora_dtype dtype);

/* ---- the reference's entry points, one call each -------------------------------------------- */
/* Each of the four takes an optional `plan`.  NULL: the call sorts the tokens and cuts the tiles
 * itself, in `workspace` (mlora_workspace_bytes), with the tile table's configuration for the shape
 * -- one extra launch per call.  The reference passes the same per-token ids to the 8 calls of a
 * layer and to all layers of a forward pass (lora_unordered_batch_infer.py:946-1063), so a binding
 * should build ONE plan per batch (mlora_tile_lookup + mlora_build_plan on the ids the calls would
 * get; for the segment / per-request signatures on the output of mlora_ids_from_segments /
 * mlora_ids_from_requests) and pass it to every call: then `indicies` / the segment operands are
 * not read, an expand needs no workspace, and a shrink only mlora_scratch_bytes of it.          */
/* dispatch_bgmv(y, x, w, start_indicies, lora_ranks, loc_indicies, indicies, qkvo, lora_scales)
 * valora/csrc/lora_ops.cc:76-126.  Direction: h_in < h_out => expand, else shrink
 * (valora/csrc/bgmv/bgmv_impl.cuh:221).                                                       */
int mlora_dispatch_bgmv(void *stream, void *y, const void *x, const mlora_pool *pool,
                        const int64_t *indicies, int64_t qkvo, const void *lora_scales, int64_t T,
                        int64_t h_in, int64_t h_out, mlora_dtype dtype, void *workspace,
                        size_t workspace_bytes, const mlora_plan *plan);

/* mlora_dispatch_bgmv for callers that cannot allocate device memory and have no workspace to
 * bring: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  Same arguments, checks, kernels and results as
 * mlora_dispatch_bgmv, but the plan and the split-K partials live in a workspace of
 * MLORA_STATIC_WORKSPACE_BYTES that is part of the library's device image (one copy per GPU, held
 * until the process ends).  A call whose mlora_workspace_bytes(T, n_adapters, min(h_in, h_out))
 * exceeds that size fails with MLORA_ERR_WORKSPACE and touches nothing.  The call allocates and
 * frees nothing; the first call on each device looks the workspace's address up once (make that
 * call outside a graph capture).  All calls on one GPU share the workspace: calls that overlap in
 * time on one GPU (two streams, two threads) race, whereas calls queued on one stream are safe.   */
#define MLORA_STATIC_WORKSPACE_BYTES (16u << 20)
int mlora_dispatch_bgmv_static(void *stream, void *y, const void *x, const mlora_pool *pool,
                               const int64_t *indicies, int64_t qkvo, const void *lora_scales,
                               int64_t T, int64_t h_in, int64_t h_out, mlora_dtype dtype);

/* dispatch_bgmv of the ATMM extension (imported as dispatch_sgmm)
 * atmm/valora/csrc/lora_ops.cc:115-186.  Rows of problems i < num_problems are processed with
 * the adapter named by their per-token id; tile arguments tb_* / wp_* are accepted and ignored
 * (tile selection is the library's own table).  shrink_mode: MLORA_SHRINK_OVERWRITE or
 * MLORA_SHRINK_ACCUMULATE.                                                                     */
int mlora_dispatch_sgmm(void *stream, void *y, const void *x, const mlora_pool *pool,
                        const int64_t *indicies, int64_t qkvo, const void *lora_scales,
                        const int64_t *output_counts, const int64_t *start_ids,
                        int64_t num_problems, int64_t T, int64_t h_in, int64_t h_out,
                        mlora_dtype dtype, int32_t shrink_mode, void *workspace,
                        size_t workspace_bytes, const mlora_plan *plan);

/* lora_get_qkvo_fwd_shrink / lora_get_qkvo_fwd_expand
 * valora/models/peft/triton_kernel/lora/lora_prefill.py:139-163 / :105-135.                   */
int mlora_prefill_shrink(void *stream, void *o, const void *x, const mlora_pool *pool,
                         const int32_t *b_start_loc, const int32_t *b_seq_len,
                         const int64_t *b_indicies, int64_t n_req, int64_t T, int64_t hidden,
                         int64_t o_stride, int64_t qkvo, int64_t max_rank, int64_t max_input_len,
                         mlora_dtype dtype, void *workspace, size_t workspace_bytes,
                         const mlora_plan *plan);
int mlora_prefill_expand(void *stream, void *o, const void *x, const mlora_pool *pool,
                         const void *scale, const int32_t *b_start_loc, const int32_t *b_seq_len,
                         const int64_t *b_indicies, int64_t n_req, int64_t T, int64_t x_stride,
                         int64_t feat_out, int64_t qkvo, int64_t max_rank, int64_t max_input_len,
                         mlora_dtype dtype, void *workspace, size_t workspace_bytes,
                         const mlora_plan *plan);

/* ---------------------------------------------------------------------------------------------
 * Adapter residency: the row allocator of the paged pool, loading / reading back an adapter's rows
 * and re-indexing when adapters are dropped.  All tensors are device memory; every call only
 * launches kernels on `stream` (no allocation, no synchronisation).  Integer results are
 * bit-exact with the reference's tensor code.
 *
 * mem_state: one byte per pool row, 1 = free, 0 = taken (the storage of the reference's torch.bool
 * tensor, valora/common/mem_allocator.py:247).  status: device int32[2] written by the call.
 * ------------------------------------------------------------------------------------------- */

/* MemoryAllocator.alloc (valora/common/mem_allocator.py:30-56): hands out the first `need` free rows
 * in index order, writes them ascending to out_index[need] and marks them taken.  The caller keeps
 * the count of free rows on the host, as the reference does (can_use_mem_size), and only asks for
 * what is free; status[0] = rows granted (== need then), status[1] = free rows seen by the scan. */
int mlora_pool_alloc(void *stream, void *mem_state, int64_t tot_size, int64_t need, int64_t *out_index,
                     int32_t *status);

/* MemoryAllocator.alloc_contiguous (mem_allocator.py:59-75): the first run of `need` consecutive
 * free rows.  status[0] = first row of the run, or -1 if there is none (state untouched; the
 * reference returns None). */
int mlora_pool_alloc_contiguous(void *stream, void *mem_state, int64_t tot_size, int64_t need,
                                int64_t *out_index, int32_t *status);

/* MemoryAllocator.free (mem_allocator.py:203-217): mem_state[index[i]] = 1. */
int mlora_pool_free(void *stream, void *mem_state, int64_t tot_size, const int64_t *index, int64_t n);

/* MemoryAllocator.free_all / reset (mem_allocator.py:219-221,246): every row free (or taken). */
int mlora_pool_fill(void *stream, void *mem_state, int64_t tot_size, int32_t is_free);

/* InferAdapter.load_lora_A / load_lora_B (valora/server/router/model_infer/infer_adapter.py:45-91):
 * `buffer[layer][loc[i]] = w[layer][i]` for every layer in ONE launch (the reference issues one
 * indexed assignment per layer and buffer).  pool: [n_layers][pool_rows][row_bytes] with
 * pool_layer_stride_bytes between layers; packed: [n_layers][n][row_bytes].  Rows and strides are
 * multiples of 16 bytes.  loc entries outside [0, pool_rows) are skipped. */
int mlora_pool_scatter_rows(void *stream, void *pool, int64_t pool_rows, int64_t pool_layer_stride_bytes,
                            const void *packed, int64_t packed_layer_stride_bytes, const int64_t *loc,
                            int64_t n, int64_t row_bytes, int32_t n_layers);

/* The inverse: `w[layer][i] = buffer[layer][loc[i]]`, the read-back the reference does row-group by
 * row-group when it densifies an adapter (valora/models/peft/lora_single_batch_infer.py:81-98).
 * Rows whose loc is outside the pool read as zeros. */
int mlora_pool_gather_rows(void *stream, const void *pool, int64_t pool_rows, int64_t pool_layer_stride_bytes,
                           void *packed, int64_t packed_layer_stride_bytes, const int64_t *loc, int64_t n,
                           int64_t row_bytes, int32_t n_layers);

/* InferAdapter.offload_adapters' re-indexing (infer_adapter.py:218-251 and the var_len_copy kernel
 * :263-284).  keep[n_keep] = indices of the surviving adapters in the old tensors, ascending.
 * new_len = old_len[keep]; new_start = exclusive running sum of new_len; new_scaling =
 * old_scaling[keep] (16-bit elements); new_loc = the surviving a_loc segments, concatenated.  When
 * mem_state is not null the pool rows of every dropped adapter are freed as well
 * (infer_adapter.py:214-223).  status[0] = 1 if keep[] held an index outside [0, n_old);
 * status[1] = entries written to new_loc. */
int mlora_index_compact(void *stream, const int32_t *keep, int32_t n_keep, int32_t n_old,
                        const int64_t *old_start, const int64_t *old_len, const int64_t *old_loc,
                        int64_t old_loc_len, const void *old_scaling, int64_t *new_start, int64_t *new_len,
                        int64_t *new_loc, int64_t new_loc_len, void *new_scaling, void *mem_state,
                        int64_t tot_size, int32_t *status);

/* ---------------------------------------------------------------------------------------------
 * Merging one adapter into the base weights of a layer and taking it out again
 * (valora/models/peft/lora_single_batch_infer.py:103-149, merge_adapter / unmerge_adapter):
 *
 *     w[k][i, o] = T( w[k][i, o] + sign * T( sum_j A[i, j] * T(B[j, o] * scaling) ) ),  k < n_targets
 *
 * with A / B the blocks of slot slots[k] of `adapter`, read in place from the key / value pool of
 * the layer (the reference first copies them into dense matrices, :81-98, and runs a batched GEMM
 * into a temporary).  w[k] is the [h_in, h_out] row-major weight the base model multiplies with
 * (x @ W), `ld` elements between rows.  The three rounding points of the reference (scaled B, the
 * GEMM result, the in-place add) are kept; the accumulation is fp32.  sign = +1 merges, -1
 * unmerges.  max_rank bounds the adapter's rank (multiple of 8, <= 128).  One launch for all
 * targets; each weight element is read once and written once. */
int mlora_merge_adapter(void *stream, void *const *w, const int32_t *slots, int32_t n_targets, int64_t ld,
                        int64_t h_in, int64_t h_out, const mlora_pool *pool_a, const mlora_pool *pool_b,
                        int64_t adapter, int64_t max_rank, float scaling, int32_t sign, mlora_dtype dtype);

#ifdef __cplusplus
}
#endif
#endif /* MLORA_H_ */
