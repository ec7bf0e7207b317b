// Tile-configuration table of the gfx950 LoRA kernels, host side.
//
// Replaces the reference's `shape_to_config` dictionary and `get_config_a` / `get_config_b`
// (valora/models/peft/lora_unordered_batch_infer.py:25-172,216-236), which map
// (n_adapters, first_seq_len, K, N) to CUTLASS threadblock / warp shapes tuned on an A100 and fall back to a
// fixed shape for unknown keys.  Here the key is (token bucket, rank bucket, hidden, adapter bucket) and the
// value is what the HIP kernels can vary: shrink tile height, split-K factor, who sums the split-K chunks,
// expand tile height, and whether the whole op runs as one launch.  The entries are measured on MI355X and
// live in valora_amd/tile_table.json; the build step turns that file into tile_table_gen.inc, so every caller
// of the C ABI -- not only the Python host layer -- gets the tuned tiles.
#include "mlora_internal.h"

namespace mlora {

namespace {

struct Entry {
  int32_t tokens, rank, hidden, adapters;   // bucket upper bounds (hidden: exact width)
  int32_t bm_shrink, ksplit, bm_expand, flags;
};

const Entry kTable[] = {
#include "tile_table_gen.inc"
};
constexpr int kEntries = (int)(sizeof(kTable) / sizeof(kTable[0]));

const int64_t kTokenBuckets[] = {8, 64, 128, 256, 512, 1024, 2048, 4096, 8192, 16384, (int64_t)1 << 22};
const int64_t kAdapterBuckets[] = {1, 8, 32, 64, 128, 8192};
const int64_t kRankBuckets[] = {16, 32, 64, 128};

template <int N>
int64_t bucket(int64_t v, const int64_t (&b)[N]) {
  for (int i = 0; i < N; ++i)
    if (v <= b[i]) return b[i];
  return b[N - 1];
}

const Entry *find(int64_t tb, int64_t rb, int64_t hidden, int64_t ab) {
  for (int i = 0; i < kEntries; ++i)
    if (kTable[i].tokens == tb && kTable[i].rank == rb && kTable[i].hidden == hidden && kTable[i].adapters == ab)
      return &kTable[i];
  return nullptr;
}

}  // namespace

// The rule for shapes the table has no entry for (the reference's counterpart is its fixed fallback tuple,
// lora_unordered_batch_infer.py:224,235): 128-token LDS-staged shrink tiles once adapters own long runs of
// tokens, otherwise direct tiles; enough K chunks for about 768 workgroups.
int rule_ksplit(int64_t T, int64_t A, int bm, int64_t hidden) {
  int64_t tiles = tiles_upper(T, A, bm);
  if (tiles > T) tiles = T;
  if (tiles < 1) tiles = 1;
  int64_t ks = (768 + tiles - 1) / tiles;
  int64_t kmax = hidden / 256;
  if (kmax < 1) kmax = 1;
  if (ks > kmax) ks = kmax;
  if (ks > 16) ks = 16;
  if (ks < 1) ks = 1;
  return (int)ks;
}

mlora_tile_config tile_fallback(int64_t T, int64_t max_rank, int64_t hidden, int64_t A) {
  (void)max_rank;
  mlora_tile_config c;
  const int64_t groups = A < T ? (A > 0 ? A : 1) : (T > 0 ? T : 1);
  if (T > 4096 && T / groups >= 64) c.bm_shrink = 128;
  else c.bm_shrink = T <= 1024 ? 16 : 32;
  const int ks = rule_ksplit(T, A, c.bm_shrink, hidden);
  c.ksplit = (int32_t)ks;
  c.bm_expand = T <= 1024 ? 16 : T <= 4096 ? 32 : 128;
  c.flags = (T <= 1024 && ks > 1) ? MLORA_REDUCE_IN_EXPAND : 0;
  return c;
}

static bool table_lookup(int64_t max_rank, int64_t hidden, int64_t tb, int64_t rb, int64_t ab, mlora_tile_config &c);

// The table is scanned linearly; a serving loop asks for the same few shapes call after call, so each thread
// remembers its last answers.  (T and the rank enter the answer beyond their buckets only through max_rank > 64,
// which the rank bucket already tells.)
mlora_tile_config tile_lookup(int64_t T, int64_t max_rank, int64_t hidden, int64_t A) {
  const int64_t tb = bucket(T, kTokenBuckets), rb = bucket(max_rank, kRankBuckets), ab = bucket(A, kAdapterBuckets);
  struct Memo {
    int64_t tb, rb, hidden, ab;
    mlora_tile_config cfg;
    bool valid;
  };
  constexpr int N_MEMO = 8;
  static thread_local Memo memo[N_MEMO];
  static thread_local int next = 0;
  // what depends on T itself rather than on its bucket: a 256-token shrink tile needs a batch that fills the device
  // with such tiles (one workgroup per compute unit); the low end of a bucket takes 128-token tiles with the same split
  auto finish = [T](mlora_tile_config c) {
    if (c.bm_shrink == 256 && (T + 255) / 256 * c.ksplit < 224) c.bm_shrink = 128;
    return c;
  };
  for (int i = 0; i < N_MEMO; ++i)
    if (memo[i].valid && memo[i].tb == tb && memo[i].rb == rb && memo[i].hidden == hidden && memo[i].ab == ab)
      return finish(memo[i].cfg);
  mlora_tile_config c;
  // the rule for shapes without an entry looks at T and A themselves, not at their buckets: not remembered
  // an adapter bucket without entries takes those of the next larger measured one, else of the next smaller
  bool found = table_lookup(max_rank, hidden, tb, rb, ab, c);
  constexpr int NA = (int)(sizeof(kAdapterBuckets) / sizeof(kAdapterBuckets[0]));
  for (int i = 0; i < NA && !found; ++i)
    if (kAdapterBuckets[i] > ab) found = table_lookup(max_rank, hidden, tb, rb, kAdapterBuckets[i], c);
  for (int i = NA - 1; i >= 0 && !found; --i)
    if (kAdapterBuckets[i] < ab) found = table_lookup(max_rank, hidden, tb, rb, kAdapterBuckets[i], c);
  if (!found) return tile_fallback(T, max_rank, hidden, A);
  memo[next] = Memo{tb, rb, hidden, ab, c, true};
  next = (next + 1) % N_MEMO;
  return finish(c);
}

// the entry of the shape's buckets (of the nearest measured width, if this one has none); false: no entry
static bool table_lookup(int64_t max_rank, int64_t hidden, int64_t tb, int64_t rb, int64_t ab, mlora_tile_config &c) {
  const Entry *e = find(tb, rb, hidden, ab);
  bool other_width = false;
  if (!e) {
    // a width the table was not measured for: the entry of the nearest measured width (ratio-wise)
    double best = 0;
    for (int i = 0; i < kEntries; ++i) {
      if (kTable[i].tokens != tb || kTable[i].rank != rb || kTable[i].adapters != ab) continue;
      const double ratio = hidden > kTable[i].hidden ? (double)hidden / kTable[i].hidden
                                                     : (double)kTable[i].hidden / (hidden > 0 ? hidden : 1);
      if (!e || ratio < best) {
        e = &kTable[i];
        best = ratio;
      }
    }
    other_width = e != nullptr;
  }
  if (!e) return false;
  c = mlora_tile_config{e->bm_shrink, e->ksplit, e->bm_expand, e->flags};
  if (other_width) {   // the split-K factor cut to what the width can be split into
    const int64_t kcap = hidden / 128 > 1 ? hidden / 128 : 1;
    if (c.ksplit > kcap) c.ksplit = (int32_t)kcap;
    if (c.ksplit <= 1) c.flags &= ~MLORA_REDUCE_IN_EXPAND;
    if (hidden < 256) c.flags &= ~MLORA_ONE_LAUNCH;
  }
  if (max_rank > 64) {
    if (c.bm_shrink == 64) c.bm_shrink = 32;   // ranks above 64 have no 64-token shrink tile
    if (c.bm_shrink == 256) c.bm_shrink = 128;  // and no 256-token one
    c.flags &= ~MLORA_ONE_LAUNCH;
  }
  if (c.flags & MLORA_ONE_LAUNCH) c.flags |= MLORA_REDUCE_IN_EXPAND;
  return true;
}

// split-K factor for a plan that was cut with shrink tiles of `bm` tokens: the table's, if its entry for this
// shape uses that tile height, else the rule's
int tile_ksplit_for(int64_t T, int64_t max_rank, int64_t hidden, int64_t A, int bm) {
  const mlora_tile_config c = tile_lookup(T, max_rank, hidden, A);
  return c.bm_shrink == bm ? c.ksplit : rule_ksplit(T, A, bm, hidden);
}

// the largest split-K factor any width's entry of this shape asks for (workspace sizing)
int tile_max_ksplit(int64_t T, int64_t max_rank, int64_t A) {
  // every adapter bucket counts: a bucket without entries of its own is served from a neighbouring one
  const int64_t tb = bucket(T, kTokenBuckets), rb = bucket(max_rank, kRankBuckets);
  int ks = tile_fallback(T, max_rank, (int64_t)1 << 16, A).ksplit;
  for (int i = 0; i < kEntries; ++i)
    if (kTable[i].tokens == tb && kTable[i].rank == rb && kTable[i].ksplit > ks) ks = kTable[i].ksplit;
  return ks;
}

}  // namespace mlora

extern "C" {

int mlora_tile_lookup(int64_t n_tokens, int64_t max_rank, int64_t hidden, int64_t n_adapters, mlora_tile_config *out) {
  if (!out) return mlora::fail(MLORA_ERR_INVALID, "tile_lookup: out is null");
  if (n_tokens < 0 || max_rank < 0 || hidden < 0 || n_adapters < 0)
    return mlora::fail(MLORA_ERR_INVALID, "tile_lookup: negative size");
  *out = mlora::tile_lookup(n_tokens, max_rank, hidden, n_adapters);
  return MLORA_OK;
}

int mlora_tile_fallback(int64_t n_tokens, int64_t max_rank, int64_t hidden, int64_t n_adapters, mlora_tile_config *out) {
  if (!out) return mlora::fail(MLORA_ERR_INVALID, "tile_fallback: out is null");
  if (n_tokens < 0 || max_rank < 0 || hidden < 0 || n_adapters < 0)
    return mlora::fail(MLORA_ERR_INVALID, "tile_fallback: negative size");
  *out = mlora::tile_fallback(n_tokens, max_rank, hidden, n_adapters);
  return MLORA_OK;
}

}  // extern "C"
