// C ABI of libmlora: argument validation, workspace carving and kernel dispatch.
// The checks mirror the reference's host-side checks (valora/csrc/lora_ops.cc:79-98,124-125);
// failures come back as a status code plus a thread-local message instead of a C++ exception.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "mlora_internal.h"

namespace mlora {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MLORA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return MLORA_OK;
}

int expand_bn();
int decode_bn(int max_rank);   // output columns per expand item of the one-launch op

// How long an expand item of the one-launch op waits for its tile's shrink items before it computes the tile's
// partials itself, in ticks of the device's 100 MHz clock: 30 us.  The shrink items are started before the expand
// items that wait for them and run for a few microseconds, so a healthy launch never gets near the bound; it only
// limits how long a workgroup holds its slot when the producers are held up (a device shared with other work).
constexpr int ONE_LAUNCH_WAIT_TICKS = 3000;
// expand items per tile up to which a call that asks for one launch gets it (see mlora_lora_apply_multi)
constexpr int ONE_LAUNCH_MAX_EXPAND_ITEMS = 16;

namespace {

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned128(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 127u) == 0; }

const char *dtype_name(mlora_dtype dt) { return dt == MLORA_F16 ? "Half" : "BFloat16"; }

int check_dtype(mlora_dtype dt, int64_t h_in, int64_t h_out) {
  if (dt != MLORA_F16 && dt != MLORA_BF16)
    return fail(MLORA_ERR_NO_KERNEL, "No suitable kernel. h_in=%lld h_out=%lld dtype=%d", (long long)h_in,
                (long long)h_out, (int)dt);
  return MLORA_OK;
}

int check_pool(const mlora_pool *pool, const char *who) {
  if (!pool) return fail(MLORA_ERR_INVALID, "%s: pool is null", who);
  if (pool->n_adapters < 0 || pool->a_loc_len < 0 || pool->w_rows < 0)
    return fail(MLORA_ERR_INVALID, "%s: negative pool size", who);
  if (pool->n_adapters > 0 && (!pool->a_start || !pool->a_len))
    return fail(MLORA_ERR_INVALID, "%s: a_start / a_len is null", who);
  if (pool->a_loc_len > 0 && !pool->a_loc) return fail(MLORA_ERR_INVALID, "%s: a_loc is null", who);
  if (pool->w_rows > 0 && !pool->w) return fail(MLORA_ERR_INVALID, "%s: w is null", who);
  if (!aligned16(pool->w)) return fail(MLORA_ERR_INVALID, "%s: w must be 16-byte aligned", who);
  if (pool->n_slots < 1) return fail(MLORA_ERR_INVALID, "%s: n_slots must be >= 1", who);
  if (pool->n_adapters > MAX_ADAPTERS)
    return fail(MLORA_ERR_NO_KERNEL, "%s: more than %lld adapters", who, (long long)MAX_ADAPTERS);
  // the tile records and the kernels' address set-up keep index positions and pool rows in 32 bits
  if (pool->a_loc_len > 0x7fffffff || pool->w_rows > 0x7fffffff)
    return fail(MLORA_ERR_NO_KERNEL, "%s: more than 2^31 - 1 index entries or pool rows", who);
  return MLORA_OK;
}

// the plan must have been cut for the pool index it is used with
int check_plan_pool(const mlora_plan *plan, const mlora_pool *pool, const char *who) {
  if (plan->n_adapters != pool->n_adapters || plan->n_slots != pool->n_slots)
    return fail(MLORA_ERR_INVALID, "%s: plan was built for %lld adapters with %d slots, the pool has %lld with %d (a plan "
                "does not outlive a change of the adapter index)", who, (long long)plan->n_adapters, plan->n_slots,
                (long long)pool->n_adapters, pool->n_slots);
  return MLORA_OK;
}

int check_plan(const mlora_plan *plan, int64_t T, const char *who) {
  if (!plan || !plan->dev) return fail(MLORA_ERR_INVALID, "%s: plan is null", who);
  if (plan->T != T) return fail(MLORA_ERR_INVALID, "%s: plan was built for T=%lld, call has T=%lld", who,
                                (long long)plan->T, (long long)T);
  if (plan->bytes < (size_t)plan_layout(plan->T, plan->n_adapters).total_words * 4)
    return fail(MLORA_ERR_WORKSPACE, "%s: plan buffer too small", who);
  return MLORA_OK;
}

// narrow (rank / scratch) and wide dims as the reference's compiled table bounds them:
// dims < 65536 (valora/csrc/lora_ops.cc:98), 16-byte vectors (bgmv_impl.cuh:166-168).
int check_dims(int64_t T, int64_t wide, int64_t narrow, int64_t h_in, int64_t h_out, mlora_dtype dt) {
  if (T < 0 || T > MAX_TOKENS) return fail(MLORA_ERR_INVALID, "T=%lld out of range", (long long)T);
  if (wide <= 0 || wide >= 65536 || narrow <= 0 || narrow > MAX_RANK || (wide % 8) != 0 || (narrow % 8) != 0)
    return fail(MLORA_ERR_NO_KERNEL, "No suitable kernel. h_in=%lld h_out=%lld dtype=%s", (long long)h_in,
                (long long)h_out, dtype_name(dt));
  return MLORA_OK;
}

}  // namespace

size_t scratch_bytes(int64_t T, int64_t max_rank, int ksplit) {
  const int64_t rp = partial_stride(max_rank);
  size_t n = (size_t)align_up(T * rp * 2, 256);
  // the partials' rows are whole 128-byte lines when the shrink sums them itself (128-token tiles)
  if (ksplit > 1) n += (size_t)ksplit * (size_t)T * (size_t)partial_stride_lines(max_rank) * 4;
  return n < 256 ? 256 : n;
}

namespace {

PoolDev pool_dev(const mlora_pool *p) {
  PoolDev d;
  d.w = static_cast<const uint16_t *>(p->w);
  d.w_rows = p->w_rows;
  d.a_loc = p->a_loc;
  d.a_loc_len = p->a_loc_len;
  return d;
}

// Small tiles (direct-load shrink, up to 64 tokens) of small batches sum their K chunks inside the launch: the
// last chunk of a tile to finish reads the others' partials out of the L2 they share.  One workgroup then reads
// ksplit x tile x rank x 4 bytes at L2 latency, which beats a separate reduce launch (about 3.7 us with the gap
// between the launches) only while that is a few tens of KB (64 KB: 1 us faster on a 1152-token batch; 256 KB,
// the 128-token tiles at rank 64: 5 us slower); those and large batches keep the reduce launch (or leave the
// sum to the expand).
void set_reduce_here(ShrinkArgs &a, const mlora_plan *plan, const PlanLayout &L, int64_t max_rank, int flags) {
  const int64_t tile_bytes = (int64_t)a.ksplit * plan->bm_shrink * partial_stride_lines(max_rank) * 4;
  // (the partials' rows must really begin on 128-byte lines: a scratch buffer that is only 16-byte aligned keeps the
  // reduce launch)
  const bool small = plan->bm_shrink <= 64 && tile_bytes <= 65536 && plan->T <= 4096 && aligned128(a.partial);
  a.reduce_here = (small && a.ksplit > 1 && !a.partial_only) ? ((flags & MLORA_SHRINK_RECOMPUTE) ? 2 : 1) : 0;
  a.prp = (int)partial_stride_lines(max_rank);
  a.n_tiles = (int)tiles_upper(plan->T, plan->n_adapters, plan->bm_shrink);
  a.arrive = reinterpret_cast<unsigned long long *>(static_cast<int32_t *>(plan->dev) + L.off_arrive);
}

struct Carver {
  char *p;
  size_t left;
  void *take(size_t n) {
    n = (n + 255) & ~(size_t)255;
    if (n > left) return nullptr;
    void *r = p;
    p += n;
    left -= n;
    return r;
  }
};

}  // namespace
}  // namespace mlora

using namespace mlora;

extern "C" {

const char *mlora_last_error(void) { return g_err; }
int mlora_version(void) { return 100; }

size_t mlora_plan_bytes(int64_t T, int64_t n_adapters) {
  if (T < 0 || n_adapters < 0) return 0;
  return (size_t)plan_layout(T, n_adapters).total_words * 4;
}

size_t mlora_scratch_bytes(int64_t T, int64_t max_rank, int32_t ksplit) {
  if (T < 0 || max_rank < 0 || ksplit < 1) return 0;
  return scratch_bytes(T, max_rank, ksplit);
}

size_t mlora_one_launch_scratch_bytes(int64_t T, int64_t n_adapters, int64_t max_rank, int32_t ksplit,
                                      int32_t n_targets) {
  if (T < 0 || n_adapters < 0 || max_rank < 0 || n_targets < 1) return 0;
  if (ksplit < 2) ksplit = 2;
  if (ksplit * n_targets > DECODE_MAX_PRODUCERS) ksplit = DECODE_MAX_PRODUCERS / n_targets;
  const int64_t rp = partial_stride(max_rank);
  return (size_t)align_up(T * rp * 2, 256) +
         4 * decode_partial_floats(tiles_upper(T, n_adapters, 16), n_targets, ksplit, rp);
}

size_t mlora_workspace_bytes(int64_t T, int64_t n_adapters, int64_t max_rank) {
  if (T < 0 || n_adapters < 0 || max_rank < 0) return 0;
  auto up = [](size_t n) { return (n + 255) & ~(size_t)255; };
  const int ks = tile_max_ksplit(T, max_rank, n_adapters);
  return up(mlora_plan_bytes(T, n_adapters)) + up(scratch_bytes(T, max_rank, ks)) + up((size_t)T * 8 + 8) + 256;
}

int mlora_build_plan(void *stream, mlora_plan *plan, const int64_t *ids, int64_t T, const int64_t *a_start,
                     const int64_t *a_len, int64_t n_adapters, int32_t n_slots, int32_t bm_shrink,
                     int32_t bm_expand) {
  if (!plan || !plan->dev) return fail(MLORA_ERR_INVALID, "build_plan: plan buffer is null");
  if (T < 0 || T > MAX_TOKENS) return fail(MLORA_ERR_INVALID, "build_plan: T=%lld out of range", (long long)T);
  if (n_adapters < 0 || n_adapters > MAX_ADAPTERS)
    return fail(MLORA_ERR_NO_KERNEL, "build_plan: n_adapters=%lld out of range (max %lld)", (long long)n_adapters,
                (long long)MAX_ADAPTERS);
  if (T > 0 && !ids) return fail(MLORA_ERR_INVALID, "build_plan: ids is null");
  if (n_adapters > 0 && (!a_start || !a_len)) return fail(MLORA_ERR_INVALID, "build_plan: a_start / a_len is null");
  if (n_slots < 1) return fail(MLORA_ERR_INVALID, "build_plan: n_slots must be >= 1");
  if (bm_shrink == 0 || bm_expand == 0) {   // neither rank nor width is known here: the rule's tile heights
    const mlora_tile_config c = tile_fallback(T, 16, 4096, n_adapters);
    if (bm_shrink == 0) bm_shrink = c.bm_shrink;
    if (bm_expand == 0) bm_expand = c.bm_expand;
  }
  if (bm_shrink != 16 && bm_shrink != 32 && bm_shrink != 64 && bm_shrink != 128 && bm_shrink != 256)
    return fail(MLORA_ERR_NO_KERNEL, "build_plan: bm_shrink=%d not in {16,32,64,128,256}", bm_shrink);
  if (bm_expand < 16 || bm_expand > 256 || (bm_expand % 16) != 0)
    return fail(MLORA_ERR_NO_KERNEL, "build_plan: bm_expand=%d not a multiple of 16 in [16,256]", bm_expand);
  const PlanLayout L = plan_layout(T, n_adapters);
  if (plan->bytes < (size_t)L.total_words * 4)
    return fail(MLORA_ERR_WORKSPACE, "build_plan: plan buffer has %zu bytes, needs %zu", plan->bytes,
                (size_t)L.total_words * 4);
  if (!aligned16(plan->dev)) return fail(MLORA_ERR_INVALID, "build_plan: plan buffer must be 16-byte aligned");
  plan->T = T;
  plan->n_adapters = n_adapters;
  plan->n_slots = n_slots;
  plan->bm_shrink = bm_shrink;
  plan->bm_expand = bm_expand;
  return launch_plan((hipStream_t)stream, static_cast<int32_t *>(plan->dev), L, ids, a_start, a_len, n_slots,
                     bm_shrink, bm_expand);
}

int mlora_count_consecutive(void *stream, const int64_t *lora_rank, int64_t n_adapters, const int64_t *indicies,
                            int64_t T, int64_t *output_counts, int64_t *rank_counts, int64_t *lora_ids,
                            int64_t *start_ids, int64_t *num_runs) {
  if (T < 0 || T > MAX_TOKENS) return fail(MLORA_ERR_INVALID, "count_consecutive: T=%lld out of range", (long long)T);
  if (!num_runs) return fail(MLORA_ERR_INVALID, "count_consecutive: num_runs is null");
  if (T > 0 && (!indicies || !output_counts || !rank_counts || !lora_ids || !start_ids || !lora_rank))
    return fail(MLORA_ERR_INVALID, "count_consecutive: null pointer");
  return launch_count_consecutive((hipStream_t)stream, lora_rank, n_adapters, indicies, T, output_counts,
                                  rank_counts, lora_ids, start_ids, num_runs);
}

int mlora_ids_from_segments(void *stream, int64_t *ids_out, const int64_t *ids_in, const int64_t *start_ids,
                            const int64_t *output_counts, int64_t P, int64_t T) {
  if (T < 0 || P < 0) return fail(MLORA_ERR_INVALID, "ids_from_segments: negative size");
  if (T > 0 && (!ids_out || !ids_in)) return fail(MLORA_ERR_INVALID, "ids_from_segments: null pointer");
  if (P > 0 && (!start_ids || !output_counts)) return fail(MLORA_ERR_INVALID, "ids_from_segments: null segments");
  return launch_ids_from_segments((hipStream_t)stream, ids_out, ids_in, start_ids, output_counts, P, T);
}

int mlora_ids_from_requests(void *stream, int64_t *ids_out, const int32_t *b_start_loc, const int32_t *b_seq_len,
                            const int64_t *b_indicies, int64_t n_req, int64_t T, int64_t max_rows) {
  if (T < 0 || n_req < 0) return fail(MLORA_ERR_INVALID, "ids_from_requests: negative size");
  if (T > 0 && !ids_out) return fail(MLORA_ERR_INVALID, "ids_from_requests: null pointer");
  if (n_req > 0 && (!b_start_loc || !b_seq_len || !b_indicies))
    return fail(MLORA_ERR_INVALID, "ids_from_requests: null request operands");
  return launch_ids_from_requests((hipStream_t)stream, ids_out, b_start_loc, b_seq_len, b_indicies, n_req, T,
                                  max_rows);
}

int mlora_shrink(void *stream, const mlora_plan *plan, void *scratch, size_t scratch_nbytes, const void *x, int64_t T,
                 int64_t h_in, int64_t max_rank, const mlora_pool *pool, int32_t slot, int32_t ksplit, void *out,
                 int64_t out_stride, int32_t mode, int32_t width, int32_t flags, mlora_dtype dtype) {
  if (int rc = check_dtype(dtype, h_in, max_rank)) return rc;
  if (int rc = check_dims(T, h_in, max_rank, h_in, max_rank, dtype)) return rc;
  if (int rc = check_plan(plan, T, "shrink")) return rc;
  if (int rc = check_pool(pool, "shrink")) return rc;
  if (int rc = check_plan_pool(plan, pool, "shrink")) return rc;
  if (T == 0) return MLORA_OK;
  if (!x || !scratch) return fail(MLORA_ERR_INVALID, "shrink: null pointer");
  if (!aligned16(x) || !aligned16(scratch)) return fail(MLORA_ERR_INVALID, "shrink: x and scratch must be 16-byte aligned");
  if (slot < 0 || slot >= pool->n_slots) return fail(MLORA_ERR_INVALID, "shrink: slot %d outside [0,%d)", slot, pool->n_slots);
  if (ksplit == 0) ksplit = tile_ksplit_for(T, max_rank, h_in, plan->n_adapters, plan->bm_shrink);
  if (ksplit < 1 || ksplit > 64) return fail(MLORA_ERR_INVALID, "shrink: ksplit=%d outside [1,64]", ksplit);
  if (scratch_nbytes < scratch_bytes(T, max_rank, ksplit))
    return fail(MLORA_ERR_WORKSPACE, "shrink: scratch has %zu bytes, needs %zu", scratch_nbytes,
                scratch_bytes(T, max_rank, ksplit));
  if (mode < 0 || mode > 2) return fail(MLORA_ERR_INVALID, "shrink: bad mode %d", mode);
  if (out && (out_stride < 1 || (mode == MLORA_SHRINK_ZERO_PAD && width > out_stride)))
    return fail(MLORA_ERR_INVALID, "shrink: width %d exceeds row stride %lld", width, (long long)out_stride);
  const PlanLayout L = plan_layout(plan->T, plan->n_adapters);
  const int64_t rp = partial_stride(max_rank);
  ShrinkArgs a;
  a.plan = static_cast<const int32_t *>(plan->dev);
  a.off_perm = L.off_perm;
  a.off_tiles = L.off_tiles_s;
  a.off_prank = L.off_prank;
  a.partial = reinterpret_cast<float *>(static_cast<char *>(scratch) + align_up(T * rp * 2, 256));
  a.x = static_cast<const uint16_t *>(x);
  a.pool = pool_dev(pool);
  a.T = (int)T;
  a.h_in = (int)h_in;
  a.rp = (int)rp;
  a.slot = slot;
  a.ksplit = ksplit;
  a.kchunk = (int)align_up((h_in + ksplit - 1) / ksplit, 128);
  a.partial_only = (!out && ksplit > 1 && (flags & MLORA_REDUCE_IN_EXPAND)) ? 1 : 0;
  a.n_targets = 1;
  for (int i = 0; i < MLORA_MAX_TARGETS; ++i) a.slots[i] = slot;
  a.out_tstride = 0;
  a.partial_tstride = 0;
  if (out) {
    a.out = static_cast<uint16_t *>(out);
    a.out_stride = out_stride;
    a.out_by_token = 1;
    a.mode = mode;
    a.width = width;
    a.ncols = (int)(max_rank < out_stride ? max_rank : out_stride);
  } else {
    a.out = static_cast<uint16_t *>(scratch);
    a.out_stride = rp;
    a.out_by_token = 0;
    a.mode = MLORA_SHRINK_OVERWRITE;
    a.width = 0;
    a.ncols = (int)rp;
  }
  set_reduce_here(a, plan, L, max_rank, flags);
  if (int rc = launch_shrink((hipStream_t)stream, a, plan->bm_shrink, (int)max_rank,
                             tiles_upper(T, plan->n_adapters, plan->bm_shrink), dtype))
    return rc;
  if (ksplit > 1 && !a.partial_only && !a.reduce_here) return launch_shrink_reduce((hipStream_t)stream, a, dtype);
  return MLORA_OK;
}

int mlora_expand(void *stream, const mlora_plan *plan, void *y, int64_t T, int64_t h_out, const void *scratch,
                 const void *v, int64_t v_stride, int64_t max_rank, const mlora_pool *pool, int32_t slot,
                 const void *scales, int32_t ksplit, int32_t flags, mlora_dtype dtype) {
  if (int rc = check_dtype(dtype, max_rank, h_out)) return rc;
  if (int rc = check_dims(T, h_out, max_rank, max_rank, h_out, dtype)) return rc;
  if (int rc = check_plan(plan, T, "expand")) return rc;
  if (int rc = check_pool(pool, "expand")) return rc;
  if (int rc = check_plan_pool(plan, pool, "expand")) return rc;
  if (T == 0) return MLORA_OK;
  if (!y || !scales) return fail(MLORA_ERR_INVALID, "expand: null pointer");
  if (!scratch && !v) return fail(MLORA_ERR_INVALID, "expand: neither scratch nor v given");
  if (!aligned16(y) || !aligned16(scratch) || !aligned16(v))
    return fail(MLORA_ERR_INVALID, "expand: y, scratch and v must be 16-byte aligned");
  if (v && (v_stride < max_rank || (v_stride % 8) != 0))
    return fail(MLORA_ERR_NO_KERNEL, "No suitable kernel. h_in=%lld h_out=%lld dtype=%s", (long long)v_stride,
                (long long)h_out, dtype_name(dtype));
  if (slot < 0 || slot >= pool->n_slots) return fail(MLORA_ERR_INVALID, "expand: slot %d outside [0,%d)", slot, pool->n_slots);
  const PlanLayout L = plan_layout(plan->T, plan->n_adapters);
  ExpandArgs a;
  a.plan = static_cast<const int32_t *>(plan->dev);
  a.off_perm = L.off_perm;
  a.off_tiles = L.off_tiles_e;
  a.y = static_cast<uint16_t *>(y);
  a.v = static_cast<const uint16_t *>(v ? v : scratch);
  a.v_stride = v ? v_stride : partial_stride(max_rank);
  a.v_by_pos = v ? 0 : 1;
  a.partial = nullptr;
  a.ksplit = 1;
  a.rp = (int)partial_stride(max_rank);
  if (!v && ksplit > 1 && (flags & MLORA_REDUCE_IN_EXPAND)) {
    if (ksplit > 64) return fail(MLORA_ERR_INVALID, "expand: ksplit=%d outside [1,64]", ksplit);
    a.partial = reinterpret_cast<const float *>(static_cast<const char *>(scratch) + align_up(T * a.rp * 2, 256));
    a.ksplit = ksplit;
  }
  a.pool = pool_dev(pool);
  a.scales = static_cast<const uint16_t *>(scales);
  a.T = (int)T;
  a.h_out = (int)h_out;
  a.kmax = (int)max_rank;
  a.slot = slot;
  a.n_ochunks = (int)((h_out + expand_bn() - 1) / expand_bn());
  a.column_loop = (flags & MLORA_EXPAND_COLUMN_LOOP) ? 1 : 0;
  a.n_targets = 1;
  for (int i = 0; i < MLORA_MAX_TARGETS; ++i) {
    a.slots[i] = slot;
    a.ys[i] = a.y;
    a.ws[i] = a.pool.w;
    a.w_rows_t[i] = a.pool.w_rows;
  }
  a.v_tstride = 0;
  a.partial_tstride = 0;
  return launch_expand((hipStream_t)stream, a, (int)max_rank, tiles_upper(T, plan->n_adapters, plan->bm_expand),
                       plan->bm_expand, dtype);
}

int mlora_lora_apply(void *stream, const mlora_plan *plan, void *scratch, size_t scratch_nbytes, void *y,
                     const void *x, int64_t T, int64_t h_in, int64_t h_out, int64_t max_rank,
                     const mlora_pool *pool_a, const mlora_pool *pool_b, int32_t slot, const void *scales,
                     int32_t ksplit, int32_t flags, mlora_dtype dtype) {
  if (!plan) return fail(MLORA_ERR_INVALID, "lora_apply: plan is null");
  if (flags & MLORA_ONE_LAUNCH) {
    if (int rc = check_pool(pool_b, "lora_apply")) return rc;
    mlora_target tg;
    tg.y = y;
    tg.w_b = pool_b->w;
    tg.w_b_rows = pool_b->w_rows;
    tg.slot = slot;
    return mlora_lora_apply_multi(stream, plan, scratch, scratch_nbytes, x, T, h_in, h_out, max_rank, pool_a, 1, &tg,
                                  scales, ksplit, flags, dtype);
  }
  if (ksplit == 0) ksplit = tile_ksplit_for(T, max_rank, h_in, plan->n_adapters, plan->bm_shrink);
  if (int rc = mlora_shrink(stream, plan, scratch, scratch_nbytes, x, T, h_in, max_rank, pool_a, slot, ksplit, nullptr,
                            0, MLORA_SHRINK_OVERWRITE, 0, flags, dtype))
    return rc;
  return mlora_expand(stream, plan, y, T, h_out, scratch, nullptr, 0, max_rank, pool_b, slot, scales, ksplit, flags,
                      dtype);
}

int mlora_lora_apply_multi(void *stream, const mlora_plan *plan, void *scratch, size_t scratch_nbytes, const void *x,
                           int64_t T, int64_t h_in, int64_t h_out, int64_t max_rank, const mlora_pool *pool_a,
                           int32_t n_targets, const mlora_target *targets, const void *scales, int32_t ksplit,
                           int32_t flags, mlora_dtype dtype) {
  if (int rc = check_dtype(dtype, h_in, h_out)) return rc;
  if (int rc = check_dims(T, h_in, max_rank, h_in, h_out, dtype)) return rc;
  if (int rc = check_dims(T, h_out, max_rank, h_in, h_out, dtype)) return rc;
  if (int rc = check_plan(plan, T, "lora_apply_multi")) return rc;
  if (int rc = check_pool(pool_a, "lora_apply_multi")) return rc;
  if (int rc = check_plan_pool(plan, pool_a, "lora_apply_multi")) return rc;
  if (n_targets < 1 || n_targets > MLORA_MAX_TARGETS || !targets)
    return fail(MLORA_ERR_INVALID, "lora_apply_multi: n_targets=%d outside [1,%d]", n_targets, MLORA_MAX_TARGETS);
  if (T == 0) return MLORA_OK;
  if (!x || !scratch || !scales) return fail(MLORA_ERR_INVALID, "lora_apply_multi: null pointer");
  if (!aligned16(x) || !aligned16(scratch)) return fail(MLORA_ERR_INVALID, "lora_apply_multi: x and scratch must be 16-byte aligned");
  for (int i = 0; i < n_targets; ++i) {
    if (!targets[i].y || !targets[i].w_b || !aligned16(targets[i].y) || !aligned16(targets[i].w_b))
      return fail(MLORA_ERR_INVALID, "lora_apply_multi: target %d has a null or misaligned pointer", i);
    if (targets[i].slot < 0 || targets[i].slot >= pool_a->n_slots)
      return fail(MLORA_ERR_INVALID, "lora_apply_multi: target %d slot %d outside [0,%d)", i, targets[i].slot, pool_a->n_slots);
    for (int j = 0; j < i; ++j)
      if (targets[j].y == targets[i].y) return fail(MLORA_ERR_INVALID, "lora_apply_multi: targets %d and %d share y", j, i);
  }
  if (ksplit == 0) ksplit = tile_ksplit_for(T, max_rank, h_in, plan->n_adapters, plan->bm_shrink);
  const bool one_launch = (flags & MLORA_ONE_LAUNCH) != 0;
  if (one_launch) {
    if (plan->bm_shrink != 16 || plan->bm_expand != 16)
      return fail(MLORA_ERR_NO_KERNEL, "lora_apply: the one-launch op needs a plan cut with bm_shrink = bm_expand = 16 (has %d / %d)",
                  plan->bm_shrink, plan->bm_expand);
    if (max_rank > 64) return fail(MLORA_ERR_NO_KERNEL, "lora_apply: max_rank=%lld > 64 uses the two-launch op", (long long)max_rank);
    if (ksplit < 2) ksplit = 2;   // the hand-off carries fp32 K-chunk partials
    if (ksplit * n_targets > DECODE_MAX_PRODUCERS) ksplit = DECODE_MAX_PRODUCERS / n_targets;
  }
  // The one-launch op hands the K-chunk partials over inside the launch, through lines of the scratch buffer that
  // belong to one tile each (128-byte aligned), and its expand items read element 0 of the index and of every
  // target's pool where they have nothing to fetch: a call that cannot offer that runs as two launches with the
  // same ksplit, which gives the same bits.
  bool use_decode = one_launch && aligned128(scratch) && pool_a->a_loc_len > 0 && pool_a->w_rows > 0;
  for (int i = 0; use_decode && i < n_targets; ++i) use_decode = targets[i].w_b_rows > 0;
  // Where the one-launch op pays is a matter of the expand items per tile (column chunks x targets), measured on 256
  // decode tokens over 64 adapters: up to 16 of them (one or two 4096-wide targets, an 11008 -> 4096 one) it is
  // 2 - 2.5 us faster than two launches, with more (q+k+v: 24, one 4096 -> 11008 target: 22) the expand half is the
  // longer one and the column-looping expand launch does it 3 us faster than these items do.
  if (use_decode) {
    const int64_t bn = decode_bn((int)max_rank);
    use_decode = (h_out + bn - 1) / bn * n_targets <= ONE_LAUNCH_MAX_EXPAND_ITEMS;
  }
  if (ksplit < 1 || ksplit > 64) return fail(MLORA_ERR_INVALID, "lora_apply_multi: ksplit=%d outside [1,64]", ksplit);
  const size_t per_target = scratch_bytes(T, max_rank, ksplit);
  const size_t scratch_need = use_decode ? mlora_one_launch_scratch_bytes(T, plan->n_adapters, max_rank, ksplit, n_targets)
                                         : per_target * (size_t)n_targets;
  if (scratch_nbytes < scratch_need)
    return fail(MLORA_ERR_WORKSPACE, "lora_apply_multi: scratch has %zu bytes, needs %zu", scratch_nbytes, scratch_need);
  const PlanLayout L = plan_layout(plan->T, plan->n_adapters);
  const int64_t rp = partial_stride(max_rank);
  const int64_t v_bytes = align_up(T * rp * 2, 256);
  const bool rie = one_launch || (ksplit > 1 && (flags & MLORA_REDUCE_IN_EXPAND));
  ShrinkArgs a;
  a.plan = static_cast<const int32_t *>(plan->dev);
  a.off_perm = L.off_perm;
  a.off_tiles = L.off_tiles_s;
  a.off_prank = L.off_prank;
  a.partial = reinterpret_cast<float *>(static_cast<char *>(scratch) + v_bytes);
  a.x = static_cast<const uint16_t *>(x);
  a.pool = pool_dev(pool_a);
  a.T = (int)T;
  a.h_in = (int)h_in;
  a.rp = (int)rp;
  a.slot = targets[0].slot;
  a.ksplit = ksplit;
  a.kchunk = (int)align_up((h_in + ksplit - 1) / ksplit, 128);
  a.out = static_cast<uint16_t *>(scratch);
  a.out_stride = rp;
  a.out_by_token = 0;
  a.mode = MLORA_SHRINK_OVERWRITE;
  a.width = 0;
  a.ncols = (int)rp;
  a.partial_only = rie ? 1 : 0;
  a.n_targets = n_targets;
  for (int i = 0; i < MLORA_MAX_TARGETS; ++i) a.slots[i] = targets[i < n_targets ? i : 0].slot;
  a.out_tstride = (int64_t)(per_target / 2);
  a.partial_tstride = (int64_t)(per_target / 4);
  set_reduce_here(a, plan, L, max_rank, flags);
  if (!use_decode) {
    if (int rc = launch_shrink((hipStream_t)stream, a, plan->bm_shrink, (int)max_rank,
                               tiles_upper(T, plan->n_adapters, plan->bm_shrink), dtype))
      return rc;
    if (ksplit > 1 && !rie && !a.reduce_here)
      if (int rc = launch_shrink_reduce((hipStream_t)stream, a, dtype)) return rc;
  }

  ExpandArgs e;
  e.plan = a.plan;
  e.off_perm = L.off_perm;
  e.off_tiles = L.off_tiles_e;
  e.y = static_cast<uint16_t *>(targets[0].y);
  e.v = static_cast<const uint16_t *>(scratch);
  e.v_stride = rp;
  e.v_by_pos = 1;
  e.partial = rie ? a.partial : nullptr;
  e.ksplit = rie ? ksplit : 1;
  e.rp = (int)rp;
  e.pool = pool_dev(pool_a);
  e.scales = static_cast<const uint16_t *>(scales);
  e.T = (int)T;
  e.h_out = (int)h_out;
  e.kmax = (int)max_rank;
  e.slot = targets[0].slot;
  e.n_ochunks = (int)((h_out + expand_bn() - 1) / expand_bn());
  e.column_loop = (flags & MLORA_EXPAND_COLUMN_LOOP) ? 1 : 0;
  e.n_targets = n_targets;
  for (int i = 0; i < MLORA_MAX_TARGETS; ++i) {
    const mlora_target &t = targets[i < n_targets ? i : 0];
    e.slots[i] = t.slot;
    e.ys[i] = static_cast<uint16_t *>(t.y);
    e.ws[i] = static_cast<const uint16_t *>(t.w_b);
    e.w_rows_t[i] = t.w_b_rows;
  }
  e.v_tstride = a.out_tstride;
  e.partial_tstride = a.partial_tstride;
  if (use_decode) {
    const int64_t tiles = tiles_upper(T, plan->n_adapters, 16);
    int32_t *words = static_cast<int32_t *>(plan->dev);
    DecodeArgs d;
    d.s = a;
    d.e = e;
    d.done = reinterpret_cast<uint32_t *>(words + L.off_counters);
    d.stamps = reinterpret_cast<uint32_t *>(words + L.off_stamps);
    d.n_tiles = (int)tiles;
    d.e.n_ochunks = (int)((h_out + decode_bn((int)max_rank) - 1) / decode_bn((int)max_rank));
    d.n_producers = ksplit * n_targets;
    d.n_consumers = d.e.n_ochunks * n_targets;
    d.spin_limit = (flags & MLORA_ONE_LAUNCH_NO_WAIT) ? 0 : ONE_LAUNCH_WAIT_TICKS;
    d.never_ready = (flags & MLORA_ONE_LAUNCH_NEVER_READY) ? 1 : 0;
    return launch_decode((hipStream_t)stream, d, (int)max_rank, dtype);
  }
  return launch_expand((hipStream_t)stream, e, (int)max_rank, tiles_upper(T, plan->n_adapters, plan->bm_expand),
                       plan->bm_expand, dtype);
}

// ---- one-call entry points ------------------------------------------------------------------------

// `given`: the caller's plan for exactly these per-token ids (then nothing is built here and the tile heights
// are the plan's), or null: a plan is built in the workspace with the table's tiles for this shape.
static int one_call(void *stream, void *y, const void *x, const mlora_pool *pool, const int64_t *ids, int64_t qkvo,
                    const void *scales, int64_t T, int64_t h_in, int64_t h_out, mlora_dtype dtype, int shrink_mode,
                    int shrink_width, int64_t narrow_stride, Carver &ws, const mlora_plan *given, const char *who) {
  if (int rc = check_pool(pool, who)) return rc;
  if (qkvo < 0 || qkvo >= pool->n_slots) return fail(MLORA_ERR_INVALID, "%s: qkvo=%lld outside [0,%d)", who, (long long)qkvo, pool->n_slots);
  const bool expand = h_in < h_out;  // valora/csrc/bgmv/bgmv_impl.cuh:221
  const int64_t narrow = expand ? h_in : h_out;
  const int64_t wide = expand ? h_out : h_in;
  if (int rc = check_dims(T, wide, narrow, h_in, h_out, dtype)) return rc;
  if (T == 0) return MLORA_OK;
  mlora_plan built;
  const mlora_plan *plan = given;
  int ksplit;
  if (given) {
    if (int rc = check_plan(given, T, who)) return rc;
    if (int rc = check_plan_pool(given, pool, who)) return rc;
    ksplit = tile_ksplit_for(T, narrow, wide, pool->n_adapters, given->bm_shrink);
  } else {
    const mlora_tile_config cfg = tile_lookup(T, narrow, wide, pool->n_adapters);
    built.bytes = mlora_plan_bytes(T, pool->n_adapters);
    built.dev = ws.take(built.bytes);
    if (!built.dev) return fail(MLORA_ERR_WORKSPACE, "%s: workspace too small (needs %zu bytes)", who,
                                mlora_workspace_bytes(T, pool->n_adapters, narrow));
    if (int rc = mlora_build_plan(stream, &built, ids, T, pool->a_start, pool->a_len, pool->n_adapters, pool->n_slots,
                                  cfg.bm_shrink, cfg.bm_expand))
      return rc;
    plan = &built;
    ksplit = cfg.ksplit;
  }
  if (expand) {
    if (narrow_stride == 0) narrow_stride = h_in;
    return mlora_expand(stream, plan, y, T, h_out, nullptr, x, narrow_stride, narrow, pool, (int32_t)qkvo, scales, 1,
                        0, dtype);
  }
  const size_t sbytes = scratch_bytes(T, narrow, ksplit);
  void *scratch = ws.take(sbytes);
  if (!scratch) return fail(MLORA_ERR_WORKSPACE, "%s: workspace too small (needs %zu bytes)", who,
                            mlora_workspace_bytes(T, pool->n_adapters, narrow));
  if (narrow_stride == 0) narrow_stride = h_out;
  return mlora_shrink(stream, plan, scratch, sbytes, x, T, h_in, narrow, pool, (int32_t)qkvo, ksplit, y,
                      narrow_stride, shrink_mode, shrink_width, 0, dtype);
}

int mlora_dispatch_bgmv(void *stream, void *y, const void *x, const mlora_pool *pool, const int64_t *indicies,
                        int64_t qkvo, const void *lora_scales, int64_t T, int64_t h_in, int64_t h_out,
                        mlora_dtype dtype, void *workspace, size_t workspace_bytes, const mlora_plan *plan) {
  if (int rc = check_dtype(dtype, h_in, h_out)) return rc;
  if (T > 0 && (!y || !x || (!indicies && !plan))) return fail(MLORA_ERR_INVALID, "dispatch_bgmv: null pointer");
  const bool needs_ws = !(plan && h_in < h_out);   // an expand on a caller-held plan needs no scratch at all
  if (T > 0 && needs_ws && (!workspace || !aligned16(workspace)))
    return fail(MLORA_ERR_WORKSPACE, "dispatch_bgmv: workspace missing or misaligned");
  if (T > 0 && h_in < h_out && !lora_scales) return fail(MLORA_ERR_INVALID, "dispatch_bgmv: lora_scales is null");
  Carver ws{static_cast<char *>(workspace), workspace_bytes};
  return one_call(stream, y, x, pool, indicies, qkvo, lora_scales, T, h_in, h_out, dtype, MLORA_SHRINK_OVERWRITE, 0, 0,
                  ws, plan, "dispatch_bgmv");
}

int mlora_dispatch_sgmm(void *stream, void *y, const void *x, const mlora_pool *pool, const int64_t *indicies,
                        int64_t qkvo, const void *lora_scales, const int64_t *output_counts,
                        const int64_t *start_ids, int64_t num_problems, int64_t T, int64_t h_in, int64_t h_out,
                        mlora_dtype dtype, int32_t shrink_mode, void *workspace, size_t workspace_bytes,
                        const mlora_plan *plan) {
  if (int rc = check_dtype(dtype, h_in, h_out)) return rc;
  if (T < 0 || T > MAX_TOKENS) return fail(MLORA_ERR_INVALID, "dispatch_sgmm: T=%lld out of range", (long long)T);
  if (num_problems < 0) return fail(MLORA_ERR_INVALID, "dispatch_sgmm: num_problems < 0");
  if (shrink_mode != MLORA_SHRINK_OVERWRITE && shrink_mode != MLORA_SHRINK_ACCUMULATE)
    return fail(MLORA_ERR_INVALID, "dispatch_sgmm: bad shrink_mode %d", shrink_mode);
  if (T == 0) return MLORA_OK;
  if (!y || !x || (!indicies && !plan)) return fail(MLORA_ERR_INVALID, "dispatch_sgmm: null pointer");
  if (!(plan && (h_in < h_out)) && (!workspace || !aligned16(workspace)))
    return fail(MLORA_ERR_WORKSPACE, "dispatch_sgmm: workspace missing or misaligned");
  if (h_in < h_out && !lora_scales) return fail(MLORA_ERR_INVALID, "dispatch_sgmm: lora_scales is null");
  Carver ws{static_cast<char *>(workspace), workspace_bytes};
  int64_t *ids_eff = nullptr;
  if (!plan) {   // a caller-held plan was cut from the covered rows' ids already
    ids_eff = static_cast<int64_t *>(ws.take((size_t)T * 8));
    if (!ids_eff) return fail(MLORA_ERR_WORKSPACE, "dispatch_sgmm: workspace too small");
    if (int rc = mlora_ids_from_segments(stream, ids_eff, indicies, start_ids, output_counts, num_problems, T)) return rc;
  }
  return one_call(stream, y, x, pool, ids_eff, qkvo, lora_scales, T, h_in, h_out, dtype, shrink_mode, 0, 0, ws, plan,
                  "dispatch_sgmm");
}

// ---- dispatch_bgmv for callers that cannot allocate --------------------------------------------
// The workspace of mlora_dispatch_bgmv (plan + split-K partials) lives in this array instead of in
// memory the caller brings.  Every device that loads the library holds its own copy until the
// process ends.  Host code must never pass the array's name to a kernel (it is a host-side stand-in,
// not a device address): the address is looked up once per device and kept in g_static_ws.
constexpr size_t STATIC_WS_BYTES = (size_t)MLORA_STATIC_WORKSPACE_BYTES;
constexpr int STATIC_WS_MAX_DEVICES = 64;
static __device__ __align__(256) unsigned char scratch[STATIC_WS_BYTES];
static std::atomic<void *> g_static_ws[STATIC_WS_MAX_DEVICES];

// Device address of `scratch` on the current device (looked up on the first call per device).
static int static_workspace(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(MLORA_ERR_LAUNCH, "dispatch_bgmv_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= STATIC_WS_MAX_DEVICES)
    return fail(MLORA_ERR_INVALID, "dispatch_bgmv_static: device %d outside [0,%d)", dev, STATIC_WS_MAX_DEVICES);
  void *p = g_static_ws[dev].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(MLORA_ERR_LAUNCH, "dispatch_bgmv_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_static_ws[dev].store(p, std::memory_order_release);   // every thread gets the same address for a device
  }
  *out = p;
  return MLORA_OK;
}

int mlora_dispatch_bgmv_static(void *stream, void *y, const void *x, const mlora_pool *pool, const int64_t *indicies,
                               int64_t qkvo, const void *lora_scales, int64_t T, int64_t h_in, int64_t h_out,
                               mlora_dtype dtype) {
  if (int rc = check_dtype(dtype, h_in, h_out)) return rc;
  if (int rc = check_pool(pool, "dispatch_bgmv_static")) return rc;
  if (T < 0 || T > MAX_TOKENS) return fail(MLORA_ERR_INVALID, "dispatch_bgmv_static: T=%lld out of range", (long long)T);
  if (T > 0 && (!y || !x || !indicies)) return fail(MLORA_ERR_INVALID, "dispatch_bgmv_static: null pointer");
  if (T > 0 && h_in < h_out && !lora_scales) return fail(MLORA_ERR_INVALID, "dispatch_bgmv_static: lora_scales is null");
  const int64_t narrow = h_in < h_out ? h_in : h_out;
  const size_t need = mlora_workspace_bytes(T, pool->n_adapters, narrow);
  if (need > STATIC_WS_BYTES)
    return fail(MLORA_ERR_WORKSPACE,
                "dispatch_bgmv_static: T=%lld with %lld adapters and rank %lld needs %zu bytes of workspace, the "
                "built-in one has %zu; use mlora_dispatch_bgmv with a workspace of your own",
                (long long)T, (long long)pool->n_adapters, (long long)narrow, need, STATIC_WS_BYTES);
  void *ws_dev = nullptr;
  if (int rc = static_workspace(&ws_dev)) return rc;
  // nothing in the workspace has to start at zero: the plan kernel writes every word the later
  // kernels read, and every split-K partial is written before it is summed
  Carver ws{static_cast<char *>(ws_dev), STATIC_WS_BYTES};
  return one_call(stream, y, x, pool, indicies, qkvo, lora_scales, T, h_in, h_out, dtype, MLORA_SHRINK_OVERWRITE, 0, 0,
                  ws, nullptr, "dispatch_bgmv_static");
}

int mlora_prefill_shrink(void *stream, void *o, const void *x, const mlora_pool *pool, const int32_t *b_start_loc,
                         const int32_t *b_seq_len, const int64_t *b_indicies, int64_t n_req, int64_t T,
                         int64_t hidden, int64_t o_stride, int64_t qkvo, int64_t max_rank, int64_t max_input_len,
                         mlora_dtype dtype, void *workspace, size_t workspace_bytes, const mlora_plan *plan) {
  if (int rc = check_dtype(dtype, hidden, max_rank)) return rc;
  if (T < 0 || T > MAX_TOKENS || n_req < 0) return fail(MLORA_ERR_INVALID, "prefill_shrink: bad size");
  if (T == 0 || n_req == 0) return MLORA_OK;
  if (!o || !x) return fail(MLORA_ERR_INVALID, "prefill_shrink: null pointer");
  if (!workspace || !aligned16(workspace))
    return fail(MLORA_ERR_WORKSPACE, "prefill_shrink: workspace missing or misaligned");
  if (max_rank <= 0 || max_rank > MAX_RANK) return fail(MLORA_ERR_NO_KERNEL, "prefill_shrink: max_rank=%lld", (long long)max_rank);
  Carver ws{static_cast<char *>(workspace), workspace_bytes};
  int64_t *ids_eff = nullptr;
  if (!plan) {
    ids_eff = static_cast<int64_t *>(ws.take((size_t)T * 8));
    if (!ids_eff) return fail(MLORA_ERR_WORKSPACE, "prefill_shrink: workspace too small");
    // rows visited per request: grid z covers cdiv(max_input_len, 32) blocks of 32 rows (lora_prefill.py:147)
    const int64_t max_rows = (max_input_len + 31) / 32 * 32;
    if (int rc = mlora_ids_from_requests(stream, ids_eff, b_start_loc, b_seq_len, b_indicies, n_req, T, max_rows)) return rc;
  }
  // columns stored: cdiv(max_rank, BLOCK_N) blocks of BLOCK_N = 16 (or max_rank when <= 8) (lora_prefill.py:142,147)
  const int64_t block_n = max_rank > 8 ? 16 : max_rank;
  int64_t width = (max_rank + block_n - 1) / block_n * block_n;
  if (width > o_stride) width = o_stride;
  const int64_t narrow = align_up(max_rank, 8);
  return one_call(stream, o, x, pool, ids_eff, qkvo, nullptr, T, hidden, narrow, dtype, MLORA_SHRINK_ZERO_PAD,
                  (int)width, o_stride, ws, plan, "prefill_shrink");
}

int mlora_prefill_expand(void *stream, void *o, const void *x, const mlora_pool *pool, const void *scale,
                         const int32_t *b_start_loc, const int32_t *b_seq_len, const int64_t *b_indicies,
                         int64_t n_req, int64_t T, int64_t x_stride, int64_t feat_out, int64_t qkvo,
                         int64_t max_rank, int64_t max_input_len, mlora_dtype dtype, void *workspace,
                         size_t workspace_bytes, const mlora_plan *plan) {
  if (int rc = check_dtype(dtype, max_rank, feat_out)) return rc;
  if (T < 0 || T > MAX_TOKENS || n_req < 0) return fail(MLORA_ERR_INVALID, "prefill_expand: bad size");
  if (T == 0 || n_req == 0) return MLORA_OK;
  if (!o || !x || !scale) return fail(MLORA_ERR_INVALID, "prefill_expand: null pointer");
  if (!plan && (!workspace || !aligned16(workspace)))
    return fail(MLORA_ERR_WORKSPACE, "prefill_expand: workspace missing or misaligned");
  if (max_rank <= 0 || max_rank > MAX_RANK || max_rank >= feat_out)
    return fail(MLORA_ERR_NO_KERNEL, "prefill_expand: max_rank=%lld", (long long)max_rank);
  Carver ws{static_cast<char *>(workspace), workspace_bytes};
  int64_t *ids_eff = nullptr;
  if (!plan) {
    ids_eff = static_cast<int64_t *>(ws.take((size_t)T * 8));
    if (!ids_eff) return fail(MLORA_ERR_WORKSPACE, "prefill_expand: workspace too small");
    const int64_t max_rows = (max_input_len + 31) / 32 * 32;
    if (int rc = mlora_ids_from_requests(stream, ids_eff, b_start_loc, b_seq_len, b_indicies, n_req, T, max_rows)) return rc;
  }
  return one_call(stream, o, x, pool, ids_eff, qkvo, scale, T, align_up(max_rank, 8), feat_out, dtype,
                  MLORA_SHRINK_OVERWRITE, 0, x_stride, ws, plan, "prefill_expand");
}

}  // extern "C"
