// Internal declarations shared by the kernel translation units of libmlora (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mlora.h"

namespace mlora {

// ---- plan buffer layout (int32 words) ------------------------------------------------------
//   hdr[32] | perm[T] | padapter[T] | prank[T] | tiles_s[max_tiles][8] | tiles_e[max_tiles][8]
//   | done[max_tiles] | stamps[max_tiles][DECODE_MAX_PRODUCERS] | arrive[max_tiles][2 * MLORA_MAX_TARGETS]
//   | scratch: cnt[A] gstart[A] toff_s[A] toff_e[A]
// perm[p]     token index at sorted position p (tokens grouped by adapter, original order kept
//             inside a group); positions >= hdr[H_NACTIVE] are unused
// padapter[p] adapter of position p;  prank[p] its rank
// tile        {adapter, rank, first position, token count, a_start[adapter], 0, 0, 0}
// done, stamps  the hand-off words of the one-launch op (csrc/decode.hip): per tile a word that numbers the launches
//             on this plan, and one stamp per shrink item; zeroed by the plan kernel
// arrive      the arrival words of the shrink's own split-K sum (csrc/shrink.hip): one 64-bit word per tile and
//             target, zeroed by the plan kernel and back at zero after every launch
constexpr int HDR_WORDS = 32;
constexpr int TILE_WORDS = 8;
constexpr int32_t PLAN_MAGIC = 0x4d4c5241;
enum Hdr {
  H_MAGIC = 0, H_T = 1, H_NADAPTERS = 2, H_NTILES_S = 3, H_NTILES_E = 4, H_NGROUPS = 5,
  H_MAXRANK = 6, H_RESERVED = 7, H_BM_S = 8, H_BM_E = 9, H_NACTIVE = 10
};

constexpr int64_t MAX_ADAPTERS = 8192;   // per-wave histograms live in LDS
constexpr int64_t MAX_TOKENS = 1 << 22;
constexpr int MAX_RANK = 128;
constexpr int DECODE_MAX_PRODUCERS = 16;   // shrink items per tile (K chunks x targets) of the one-launch op
// What one launch of the one-launch op adds to a tile's `done` word, all items of the tile together; the word
// divided by it numbers the launches on the plan (csrc/decode.hip).  More than the shrink items of a tile (16).
constexpr uint32_t DECODE_TAG_SHIFT = 12;
constexpr uint32_t DECODE_LAUNCH_WEIGHT = 1u << DECODE_TAG_SHIFT;
constexpr int ONE_LAUNCH_MAX_POLLS = 4096;   // hard cap on the polls of a bounded wait, whatever the clock says

struct PlanLayout {
  int64_t T, A, max_tiles;
  int64_t off_perm, off_padapter, off_prank, off_tiles_s, off_tiles_e, off_counters, off_stamps, off_arrive, off_scratch,
      total_words;
};

static inline __host__ __device__ int64_t align_up(int64_t v, int64_t a) { return (v + a - 1) / a * a; }

static inline PlanLayout plan_layout(int64_t T, int64_t A) {
  PlanLayout L;
  L.T = T;
  L.A = A;
  L.max_tiles = (T + 15) / 16 + (A < T ? A : T);
  L.off_perm = HDR_WORDS;
  L.off_padapter = align_up(L.off_perm + T, 8);
  L.off_prank = align_up(L.off_padapter + T, 8);
  L.off_tiles_s = align_up(L.off_prank + T, 8);
  L.off_tiles_e = L.off_tiles_s + L.max_tiles * TILE_WORDS;
  L.off_counters = L.off_tiles_e + L.max_tiles * TILE_WORDS;
  L.off_stamps = align_up(L.off_counters + L.max_tiles, 32);
  L.off_arrive = align_up(L.off_stamps + L.max_tiles * DECODE_MAX_PRODUCERS, 8);
  L.off_scratch = align_up(L.off_arrive + L.max_tiles * 2 * MLORA_MAX_TARGETS, 8);
  L.total_words = L.off_scratch + 4 * A + 8;
  return L;
}

// upper bound of the tile count for tile height bm (what the grids are sized with)
static inline int64_t tiles_upper(int64_t T, int64_t A, int bm) {
  return (T + bm - 1) / bm + (A < T ? A : T);
}

static inline int64_t partial_stride(int64_t max_rank) { return align_up(max_rank, 16); }
// row stride of the split-K partials when the shrink sums them itself: every row owns whole 128-byte lines, so
// no line holds rows of two tiles
static inline int64_t partial_stride_lines(int64_t max_rank) { return align_up(max_rank, 32); }

// ---- error reporting (api.hip) ---------------------------------------------------------------
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);

// ---- tile table (tiles.hip) --------------------------------------------------------------------
mlora_tile_config tile_lookup(int64_t T, int64_t max_rank, int64_t hidden, int64_t A);
mlora_tile_config tile_fallback(int64_t T, int64_t max_rank, int64_t hidden, int64_t A);
int tile_ksplit_for(int64_t T, int64_t max_rank, int64_t hidden, int64_t A, int bm);
int tile_max_ksplit(int64_t T, int64_t max_rank, int64_t A);

// ---- kernel launchers ------------------------------------------------------------------------
struct PoolDev {
  const uint16_t *w;
  int64_t w_rows;
  const int64_t *a_loc;
  int64_t a_loc_len;
};

struct ShrinkArgs {
  const int32_t *plan;
  int64_t off_perm, off_tiles, off_prank;
  float *partial;             // [ksplit][T][rp] fp32, used when ksplit > 1
  const uint16_t *x;
  PoolDev pool;
  uint16_t *out;              // v: [T positions][out_stride] or the caller's y: [T tokens][out_stride]
  int64_t out_stride;
  int T, h_in, rp, slot, ksplit, kchunk;
  int out_by_token, mode, width, ncols;
  int partial_only;           // leave the K-chunk partials for the expand to sum (no reduce launch)
  // several targets that share x in one launch (grid z = target): slot, v buffer and partials per target
  int n_targets;
  int slots[MLORA_MAX_TARGETS];
  int64_t out_tstride, partial_tstride;   // elements / floats between consecutive targets
  // split-K summed inside the launch by the last K chunk of a tile to arrive (small tiles, csrc/shrink.hip)
  int reduce_here;            // 0 off, 1 on, 2 on with every sum taking the recompute path (tests)
  int prp;                    // row stride of the partials in that mode: whole 128-byte lines per row
  int n_tiles;                // upper bound of the tile count
  unsigned long long *arrive; // [tiles][MLORA_MAX_TARGETS] arrival words, zero between launches
};

struct ExpandArgs {
  const int32_t *plan;
  int64_t off_perm, off_tiles;
  uint16_t *y;
  const uint16_t *v;          // narrow operand, T dtype
  int64_t v_stride;
  int v_by_pos;               // rows indexed by sorted position (internal buffer) or by token
  const float *partial;       // when set: v = T(sum_s partial[s][pos][:]) with ksplit chunks of T*rp floats
  int ksplit, rp;
  // several targets in one launch (grid y = target)
  int n_targets;
  int slots[MLORA_MAX_TARGETS];
  uint16_t *ys[MLORA_MAX_TARGETS];
  const uint16_t *ws[MLORA_MAX_TARGETS];
  int64_t w_rows_t[MLORA_MAX_TARGETS];
  int64_t v_tstride, partial_tstride;
  PoolDev pool;
  const uint16_t *scales;
  int T, h_out, kmax, slot, n_ochunks;
  int column_loop;            // force the column-looping kernel for 16-token tiles (tests); else by grid size
};


// one-launch op: shrink items and expand items of one grid (csrc/decode.hip)
struct DecodeArgs {
  ShrinkArgs s;               // partial-only shrink: s.partial, s.ksplit >= 2, tile height 16
  ExpandArgs e;               // expand that sums the chunks: e.partial == s.partial, e.ksplit == s.ksplit
  uint32_t *done;             // [tiles] DECODE_LAUNCH_WEIGHT per finished launch on this plan (only ever counts up)
  uint32_t *stamps;           // [tiles][DECODE_MAX_PRODUCERS] (launch tag, XCD) left by each shrink item
  int n_tiles;                // upper bound of the tile count (records past the last tile are zero)
  int n_producers;            // shrink items per tile: ksplit * targets
  int n_consumers;            // expand items per tile: column chunks * targets
  int never_ready;            // tests: expand items look for a stamp nobody leaves and wait out their bound
  int spin_limit;             // 10 ns ticks an expand item waits for its tile's stamps before it computes the partials itself
};
int launch_decode(hipStream_t st, const DecodeArgs &a, int max_rank, mlora_dtype dt);
int decode_bn(int max_rank);   // output columns per expand item of the one-launch op
size_t decode_partial_floats(int64_t n_tiles, int n_targets, int ksplit, int64_t rp);
int launch_plan(hipStream_t st, int32_t *plan, const PlanLayout &L, const int64_t *ids,
                const int64_t *a_start, const int64_t *a_len, int n_slots, int bm_s, int bm_e);
size_t scratch_bytes(int64_t T, int64_t max_rank, int ksplit);
int launch_count_consecutive(hipStream_t st, const int64_t *lora_rank, int64_t n_adapters,
                             const int64_t *indicies, int64_t T, int64_t *output_counts,
                             int64_t *rank_counts, int64_t *lora_ids, int64_t *start_ids,
                             int64_t *num_runs);
int launch_ids_from_segments(hipStream_t st, int64_t *ids_out, const int64_t *ids_in,
                             const int64_t *start_ids, const int64_t *output_counts, int64_t P,
                             int64_t T);
int launch_ids_from_requests(hipStream_t st, int64_t *ids_out, const int32_t *b_start_loc,
                             const int32_t *b_seq_len, const int64_t *b_indicies, int64_t n_req,
                             int64_t T, int64_t max_rows);
int launch_shrink(hipStream_t st, const ShrinkArgs &a, int bm, int max_rank, int64_t grid_tiles,
                  mlora_dtype dt);
int launch_shrink_reduce(hipStream_t st, const ShrinkArgs &a, mlora_dtype dt);
int launch_expand(hipStream_t st, const ExpandArgs &a, int max_rank, int64_t grid_tiles, int bm_expand,
                  mlora_dtype dt);

}  // namespace mlora
