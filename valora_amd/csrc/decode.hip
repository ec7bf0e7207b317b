// One-launch LoRA op for decode-like batches (few tokens per adapter) on gfx950:
//
//   y[t, o] = T( y[t, o] + scale_a * sum_j T(v[t, j]) * B_a[j, o] ),   v[t, j] = sum_k x[t, k] * A_a[j, k]
//
// At these sizes (tens of MB) two dependent launches cost more than the bytes: the expand's B fragments and
// y rows cannot be requested before the shrink's grid has drained.  Here both halves are work items of ONE
// grid.  Shrink items (tile, target, K chunk) compute their chunk's fp32 partial exactly like shrink_kernel
// and leave it in the scratch buffer.  Expand items (tile, target, 512 output columns) request their B
// fragments and y rows FIRST and only then wait for their tile's partials, so the wait overlaps loads they
// need anyway.
//
// The hand-off stays inside one XCD.  The 8 XCDs of the device have an L2 each, and anything that has to be
// visible across them goes to memory and back (measured here: 2.5 us per poll and 7 us to read a tile's
// partials with device-scope loads; 0.5 us and 0.8 us inside an L2).  Workgroups are dealt to the XCDs round
// robin by id, so the ids are laid out such that all items of tile t have id = t (mod 8): producer and
// consumers of a tile share an L2, and the partials are plain stores and plain loads that meet there.
// Nothing relies on the round-robin rule for correctness: a shrink item stamps its slot of the tile with
// (the launch's tag, the XCD it runs on), an expand item only accepts stamps that carry its own tag and its
// own XCD, and
//   * an expand item polls a BOUNDED number of times; when the bound runs out -- its producers ran on another
//     XCD, or were not scheduled, whatever the reason -- it computes the tile's partials itself, chunk by
//     chunk with the shrink item's own code, so it gets the same bits and NO workgroup ever waits without
//     limit: every wave of the grid reaches its end whatever the order, placement or residency of the
//     workgroups;
//   * the stamps are polled on the scalar path (scalar load that skips the scalar cache): a wave gets its
//     vector-memory results strictly in order, so a vector poll would sit behind the B and y loads;
//   * what tells a fresh stamp from one an earlier launch left behind is the launch's tag, which every item
//     derives from the tile's `done` word as it finds it when it starts: tag = word / DECODE_LAUNCH_WEIGHT.  Every
//     launch moves the word on by exactly that weight, whatever its numbers of shrink and expand items: each
//     shrink item adds 1 when it has finished, and the tile's LAST expand item (highest id) adds the rest at its
//     very end (device scope, nobody waits for the answer).  Launches on a plan do not overlap, so in launch
//     number n no item can read less than n * weight: a tag is never too low, and a stamp an earlier launch left
//     behind is never taken for a fresh one.  An item would read (n + 1) * weight, and match nothing, only if it
//     read the word after the tile's last expand item had ENDED.  The hardware starts workgroups in id order and
//     the read is an item's first instruction, so that takes an item whose first load is outlived by the whole
//     life of an item started after it; it would wait out its bound and compute the partials itself: slow, and
//     still correct.  Items that start late (a grid larger than the device holds, a device shared with another
//     stream) therefore take part in the hand-off like all others.  Nothing is ever reset, so there is no moment
//     at which a late writer could leave a stale "ready", and replays of a HIP graph (frozen arguments) need
//     nothing from the host.  (Every expand item adding its own share would make the bound on the word exact,
//     and costs 0.4 us on a 9.7 us op: the device-scope acknowledgements of 512 workgroups at the end of the
//     launch.)
//   * all shrink items have lower ids than all expand items, so by the time an expand item runs, every producer
//     it waits for has at least been started.
//   * a tile's partials occupy whole 128-byte lines of their own, so no line is fetched before the tile is
//     ready (a line shared with a neighbour tile could sit stale in a compute unit's L1).
// Chunks are summed in index order, the same order as the two-launch path: results are bit-identical to it.
// Launches that share a plan must not overlap in time (they share the scratch buffer and the words above).
//
// Reference semantics: valora/csrc/bgmv/bgmv_impl.cuh:14-148 (shrink) and :152-207 (expand).
#include "kernel_common.h"
#include "shrink_core.h"

namespace mlora {

namespace {

// 256-column chunks per expand item: two (fewer, fatter items: the whole grid should be resident at once, a waiting
// item holds its slot) up to rank 32; at rank 64 the B fragments of two chunks no longer fit the register budget of
// three waves per SIMD (16 registers spilled), so those items take one chunk.
constexpr int dec_ch(int nb) { return nb >= 4 ? 1 : 2; }
constexpr int dec_nb(int max_rank) { return max_rank <= 16 ? 1 : max_rank <= 32 ? 2 : 4; }
constexpr int DEC_WN = 64;         // outputs per wave and chunk
constexpr int DEC_STAGE_LD = DEC_WN + 4;

// device scope: visible to every compute unit, whichever XCD it sits on; the result is not asked for
__device__ __forceinline__ void add_device(uint32_t *p, uint32_t v) {
  (void)__hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// The 16 stamps of a tile as they are in this XCD's L2 right now, read on the scalar path: a scalar load with
// glc skips the scalar cache, and its answer does not queue behind the wave's outstanding vector loads (the B
// fragments and y rows requested just before), which come back strictly in order.
typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
// 1: all n stamps carry `want`; 2: one of them carries this launch's tag with another XCD's id, i.e. that producer
// ran where its partial cannot be read from here, and waiting longer is pointless; 0: not yet.
__device__ __forceinline__ int stamps_state(const uint32_t *stamps, int n, uint32_t want) {
  u32x16 v;
  asm volatile("s_load_dwordx16 %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(stamps) : "memory");
  // d = stamp ^ want is 0 for a match and 1..15 for this launch's tag with another XCD id (branch-free scalar code)
  uint32_t any_diff = 0u, least = 0xffffffffu;
#pragma unroll
  for (int i = 0; i < DECODE_MAX_PRODUCERS; ++i) {
    const uint32_t d = i < n ? (v[i] ^ want) : 0u;
    any_diff |= d;
    const uint32_t u = d - 1u;   // 0 -> 0xffffffff
    least = u < least ? u : least;
  }
  return any_diff == 0u ? 1 : least < 15u ? 2 : 0;
}
// workgroup barrier that orders LDS traffic only: outstanding global loads stay in flight across it
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// the launch's tag from the tile's `done` word as an item found it (see the head of this file), and the stamp a
// shrink item of that launch leaves when it runs on XCD `xcd` (never 0, the value the plan kernel leaves)
__device__ __forceinline__ uint32_t stamp_of(uint32_t done0, uint32_t xcd) {
  return (((done0 >> DECODE_TAG_SHIFT) + 1u) << 4) | xcd;
}

// item id -> (role, tile, item of the tile).  A group is 8 consecutive tiles.  Ids run: the shrink items of all
// groups, then the expand items of all groups, each as (group, item, tile within the group) with the tile as the
// fast index, so the tile index mod 8 equals the id mod 8 (one XCD per tile) and every producer is started before
// any consumer.  The grid is sized with an upper bound of the tile count; the tiles that do not exist are the
// last ones of either section, and their workgroups leave at once (measured against a layout that puts them at
// the end of the grid: equal on a batch that fits the device, 2 us faster on one that does not quite).
struct ItemId {
  bool shrink;
  int tile, item;
};
__device__ __forceinline__ ItemId item_of(int n_producers, int n_consumers, int shrink_ids, int id) {
  ItemId it;
  it.shrink = id < shrink_ids;
  const int l2 = it.shrink ? id : id - shrink_ids;
  const int per = it.shrink ? n_producers : n_consumers;
  const int q8 = l2 >> 3, g = q8 / per;
  it.item = q8 - g * per;
  it.tile = g * 8 + (l2 & 7);
  return it;
}

// One workgroup = one work item.  3 waves per SIMD = 3 workgroups per compute unit: an expand item keeps the B
// fragments and y rows of 512 columns in flight, a shrink item 8 K-steps of both operands.
// The leading scalar parameters repeat what the first dependent loads need (the tile records, the `done` words, the
// id layout): the library is built with kernel-argument preloading, which hands the first 8 dwords of the
// argument list to the wave in registers at launch, so the tile record can be requested without waiting for a load
// of the argument block first (0.35 us of a 10.3 us op).
template <typename T, int NB>
__global__ __launch_bounds__(256, 3) void decode_kernel(const int32_t *tiles_base, uint32_t *done_base, int h_n_producers,
                                                        int h_n_consumers, int h_n_tiles, int h_shrink_ids,
                                                        DecodeArgs a) {
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  constexpr int DEC_CH = dec_ch(NB), DEC_BN = 256 * DEC_CH;   // chunks and outputs per expand item
  constexpr int KB = (NB + 1) / 2;                  // 32-wide rank blocks of the expand
  constexpr int STAGE_FLOATS = 4 * 16 * DEC_STAGE_LD;
  constexpr int RED_FLOATS = 2 * NB * 256;          // cross-wave reduction of shrink_tile_to_lds
  constexpr int VACC_FLOATS = 16 * NB * 16;         // a tile's summed chunks (give-up path)
  static_assert(DECODE_MAX_PRODUCERS == 16, "stamps_match reads 16 stamps");
  static_assert(RED_FLOATS + VACC_FLOATS <= STAGE_FLOATS, "the shrink buffers alias the expand's staging tile");
  __shared__ __align__(16) float s_buf[STAGE_FLOATS];
  __shared__ int32_t s_perm[16];
  __shared__ int32_t s_ready;
  float(*red)[NB * 256] = reinterpret_cast<float(*)[NB * 256]>(s_buf);
  const int id = (int)blockIdx.x;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  const ItemId it = item_of(h_n_producers, h_n_consumers, h_shrink_ids, id);
  const bool shrink_item = it.shrink;
  const int item = it.item, tile_idx = it.tile;
  if (tile_idx >= h_n_tiles) return;
  const int32_t *__restrict__ tile = tiles_base + (int64_t)tile_idx * TILE_WORDS;

  // ONE scalar round trip per shrink item before its vector loads: the tile record, the tile's `done` word and every
  // field of the argument block the item is going to use are requested together and waited for once.  Left to
  // itself the compiler fetches each group of argument fields right before its first use, behind the previous
  // wait -- seven dependent scalar round trips in front of the first operand load, each an L2 access while all
  // workgroups of the grid start at the same moment.  The empty asm takes the values as read-write operands: they
  // have to be in registers at that point, and cannot be fetched again later instead of being kept.
  int ad = tile[0], r = tile[1], pos0 = tile[2], cnt = tile[3], astart = tile[4];
  uint32_t done0 = done_base[tile_idx];
  int rp = a.s.rp, n_producers = a.n_producers;
  const int32_t *plan_words = a.s.plan;
  int64_t off_perm = a.s.off_perm;
  float *partial_base = a.s.partial;
  uint32_t *stamps_base = a.stamps;

  // ------------------------------------------------------------------ shrink item
  if (shrink_item) {
    const uint16_t *x = a.s.x;
    PoolDev pool = a.s.pool;
    int h_in = a.s.h_in, ksplit = a.s.ksplit, kchunk = a.s.kchunk;
    int sl0 = a.s.slots[0], sl1 = a.s.slots[1], sl2 = a.s.slots[2], sl3 = a.s.slots[3];
    uint32_t *done = done_base;
    asm volatile("" : "+s"(ad), "+s"(r), "+s"(pos0), "+s"(cnt), "+s"(astart), "+s"(done0), "+s"(rp), "+s"(n_producers),
                      "+s"(plan_words), "+s"(off_perm), "+s"(partial_base), "+s"(stamps_base), "+s"(x), "+s"(pool.w),
                      "+s"(pool.w_rows), "+s"(pool.a_loc), "+s"(pool.a_loc_len), "+s"(h_in), "+s"(ksplit), "+s"(kchunk),
                      "+s"(sl0), "+s"(sl1), "+s"(sl2), "+s"(sl3), "+s"(done));
    if (cnt <= 0) return;   // records past the last tile are zero
    x = as_global(x);
    pool.w = as_global(pool.w);
    pool.a_loc = as_global(pool.a_loc);
    done = as_global(done);
    partial_base = as_global(partial_base);
    stamps_base = as_global(stamps_base);
    const int32_t *__restrict__ perm = as_global(plan_words) + off_perm;
    const uint32_t want_stamp = stamp_of(done0, xcd_id());
    uint32_t *const stamps = stamps_base + (int64_t)tile_idx * DECODE_MAX_PRODUCERS;
    // a tile's partials: [target][K chunk][16 rows][rp] floats, whole lines of the tile's own
    float *const tile_partial = partial_base + (int64_t)tile_idx * n_producers * 16 * rp;
    const int z = item / ksplit, s = item - z * ksplit;
    const int kbeg = s * kchunk;
    const int kend = min(h_in, kbeg + kchunk);
    const int slot = z == 0 ? sl0 : z == 1 ? sl1 : z == 2 ? sl2 : sl3;
    shrink_tile_to_lds<T, 1, NB>(x, h_in, pool, slot, perm, r, pos0, cnt, astart, kbeg, kend, red);
    if (wave == 0) {
      // wave 0 alone writes the partial and then the stamp: no barrier, and nothing else of its own in flight
      f32x4 *part = reinterpret_cast<f32x4 *>(tile_partial + (int64_t)item * 16 * rp);
      const int quarter = rp >> 2;
      for (int e = lane; e < 16 * quarter; e += 64) {
        const int row = e / quarter, c4 = e - row * quarter;
        const float *src = red[1] + row * (NB * 16) + 4 * c4;
        part[e] = f32x4{src[0], src[1], src[2], src[3]};
      }
      // the partial must sit in the L2 before the stamp that announces it
      wait_vmcnt<0>();
      if (lane == 0) __hip_atomic_store(stamps + item, want_stamp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    } else if (tid == 64) {
      add_device(done + tile_idx, 1u);   // this item's share of the launch's weight on the tile's `done` word
    }
    return;
  }

  // ------------------------------------------------------------------ expand item
  const int n_ochunks = a.e.n_ochunks, kmax = a.e.kmax, h_out = a.e.h_out, e_ksplit = a.e.ksplit, spin_limit = a.spin_limit;
  const uint16_t *const scales = a.e.scales;
  const int64_t *const a_loc = a.e.pool.a_loc;
  const int64_t a_loc_len = a.e.pool.a_loc_len;
  // (no joint round trip here: the expand items' loads are not what the op waits for -- requesting their argument
  // fields early as well measured 0.04 us slower, the target's operands on top of that another 0.08 us)
  if (cnt <= 0) return;   // records past the last tile are zero
  const int32_t *__restrict__ perm = plan_words + off_perm;
  // (never_ready: a stamp with the top bit set, which no shrink item leaves -- the wait runs to its bound)
  const uint32_t want_stamp = stamp_of(done0, xcd_id()) | (a.never_ready ? 0x80000000u : 0u);
  uint32_t *const stamps = stamps_base + (int64_t)tile_idx * DECODE_MAX_PRODUCERS;
  float *const tile_partial = partial_base + (int64_t)tile_idx * n_producers * 16 * rp;
  const int z = item / n_ochunks, oc = item - z * n_ochunks;
  const int rk = min(r, kmax);   // rank columns the narrow operand really has (bgmv_impl.cuh:167,186)
  const int slot = a.e.slots[z];
  uint16_t *const y = a.e.ys[z];
  const uint16_t *const wB = a.e.ws[z];
  const int64_t wB_rows = a.e.w_rows_t[z];

  const int lrow = lane & 15, kg = lane >> 4;
  int o_wave[DEC_CH];
#pragma unroll
  for (int c = 0; c < DEC_CH; ++c) o_wave[c] = oc * DEC_BN + c * 256 + wave * DEC_WN;

  // Everything that depends only on the tile record is requested first, in one round trip.  The set-up is
  // kept to few instructions and free of branches: with every workgroup of the grid resident, the vector
  // ALUs are what the first loads wait for.  Loads that have nothing to fetch read element 0 of their
  // array instead of being skipped, and their result is dropped.
  int my_perm = 0;
  if (tid < cnt) my_perm = perm[pos0 + tid];
  const float scale = Tr::to_float(scales[ad]);
  const float inv_h_out = 1.0f / (float)h_out;
  const uint32_t base32 = (uint32_t)(astart + r * slot), n_loc = (uint32_t)a_loc_len;
  const uint32_t step16 = 16u * (uint32_t)r;
  const bool can_step = step16 < (uint32_t)h_out;     // workgroup-uniform
  int64_t brow[DEC_CH][4][KB];
  uint32_t boff[DEC_CH][4][KB];
  bool bok[DEC_CH][4][KB];
#pragma unroll
  for (int c = 0; c < DEC_CH; ++c)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const uint32_t j0 = (uint32_t)(kb * 32 + kg * 8);
      BCursor cur = b_cursor((uint32_t)(o_wave[c] + lrow), (uint32_t)r, j0, (uint32_t)h_out, inv_h_out);
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        const int o = o_wave[c] + nb * 16 + lrow;
        if (nb > 0) {
          if (can_step) b_advance(cur, step16, (uint32_t)h_out);
          else cur = b_cursor((uint32_t)o, (uint32_t)r, j0, (uint32_t)h_out, inv_h_out);
        }
        const uint32_t idx = base32 + cur.bin;
        const bool ok = o < h_out && (int)j0 < rk && idx < n_loc;
        brow[c][nb][kb] = a_loc[ok ? idx : 0u];
        boff[c][nb][kb] = cur.off;
        bok[c][nb][kb] = ok;
      }
    }
  if (tid < 16) s_perm[tid] = my_perm;
  __syncthreads();

  // B fragments and y rows: the loads the hand-off wait is hidden behind
  u32x4 bfrag[DEC_CH][4][KB];
#pragma unroll
  for (int c = 0; c < DEC_CH; ++c)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int64_t row = brow[c][nb][kb];
        const bool ok = bok[c][nb][kb] && (uint64_t)row < (uint64_t)wB_rows;
        const u32x4 got = load16(wB + (ok ? row * h_out + boff[c][nb][kb] : 0));
        bfrag[c][nb][kb] = ok ? got : u32x4{0, 0, 0, 0};
      }
  const int rr0 = lane >> 3, c8 = (lane & 7) * 8;
  u32x4 yv[DEC_CH][2];
  uint16_t *yp[DEC_CH][2];
  bool yok[DEC_CH][2];
#pragma unroll
  for (int c = 0; c < DEC_CH; ++c)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int row = rr0 + 8 * h;
      yok[c][h] = (o_wave[c] + c8) < h_out && row < cnt;
      yp[c][h] = y + (yok[c][h] ? (int64_t)s_perm[row] * h_out + o_wave[c] + c8 : 0);
      yv[c][h] = load16(yp[c][h]);
    }
  // ---- bounded wait for the tile's stamps (one wave polls on the scalar path; the workgroup follows its
  //      verdict without draining its loads).  The producers were started before this item and run for a few
  //      microseconds; the bound (ticks of the 100 MHz clock, and a cap on the polls) only limits how long a
  //      workgroup can hold its slot when they are held up, and a producer seen on another XCD ends the wait at once.
  if (wave == 0) {
    int ok = 0;
    if (spin_limit > 0) {
      const uint64_t t0 = wall_clock64();
      for (int it = 0; it < ONE_LAUNCH_MAX_POLLS; ++it) {
        const int st = stamps_state(stamps, n_producers, want_stamp);
        if (st == 1) ok = 1;
        if (st != 0 || wall_clock64() - t0 > (uint64_t)spin_limit) break;
        __builtin_amdgcn_s_sleep(2);
      }
    }
    if (lane == 0) s_ready = ok;
  }
  lds_barrier();
  const bool ready = s_ready != 0;

  // ---- v fragment: rows = tokens (lrow), 8 consecutive rank elements per lane; chunks summed in index order
  u32x4 vfrag[KB];
  const bool pok = lrow < cnt;
  if (ready) {
    const float *part = tile_partial + (int64_t)z * e_ksplit * 16 * rp;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int j0 = kb * 32 + kg * 8;
      u32x4 v = {0, 0, 0, 0};
      if (pok && j0 < rk) {
        float f[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const float *src0 = part + lrow * rp + j0;
        for (int s0 = 0; s0 < e_ksplit; s0 += 4) {
          f32x4 lo[4], hi[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const bool ok = s0 + u < e_ksplit;
            const f32x4 *src = reinterpret_cast<const f32x4 *>(src0 + (int64_t)(s0 + u) * 16 * rp);
            lo[u] = ok ? src[0] : f32x4{0.f, 0.f, 0.f, 0.f};
            hi[u] = ok ? src[1] : f32x4{0.f, 0.f, 0.f, 0.f};
          }
#pragma unroll
          for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) { f[i] += lo[u][i]; f[4 + i] += hi[u][i]; }
        }
        v = pack8<T>(f);
      }
      vfrag[kb] = v;
    }
  } else {
    // give-up path: the tile's chunks computed here, one after the other with the shrink item's own code
    float *vacc = s_buf + RED_FLOATS;
    for (int e = tid; e < VACC_FLOATS; e += 256) vacc[e] = 0.f;
    const int slot_a = a.s.slots[z];
    for (int s = 0; s < a.s.ksplit; ++s) {
      const int kbeg = s * a.s.kchunk;
      const int kend = min(a.s.h_in, kbeg + a.s.kchunk);
      shrink_tile_to_lds<T, 1, NB>(a.s.x, a.s.h_in, a.s.pool, slot_a, perm, r, pos0, cnt, astart, kbeg, kend, red);
      for (int e = tid; e < VACC_FLOATS; e += 256) vacc[e] += red[1][e];
      __syncthreads();
    }
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int j0 = kb * 32 + kg * 8;
      u32x4 v = {0, 0, 0, 0};
      if (pok && j0 < rk && j0 < NB * 16) {
        float f[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = vacc[lrow * (NB * 16) + j0 + i];
        v = pack8<T>(f);
      }
      vfrag[kb] = v;
    }
    __syncthreads();   // vacc is about to be reused as the staging tile
  }

  // ---- delta blocks through the matrix cores, turned through a wave-private LDS tile for the y update
  float(*stage)[DEC_STAGE_LD] = reinterpret_cast<float(*)[DEC_STAGE_LD]>(s_buf + wave * 16 * DEC_STAGE_LD);
#pragma unroll
  for (int c = 0; c < DEC_CH; ++c) {
    if (o_wave[c] < h_out) {   // wave-uniform
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
          if (kb * 32 < rk) acc = Tr::mfma(as<vec8>(vfrag[kb]), as<vec8>(bfrag[c][nb][kb]), acc);
#pragma unroll
        for (int i = 0; i < 4; ++i) stage[kg * 4 + i][nb * 16 + lrow] = acc[i];
      }
      // the tile is private to this wave and a wave's LDS operations execute in order: only the compiler
      // has to be kept from moving the reads below over the writes above
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if (yok[c][h]) {
          const float *srow = &stage[rr0 + 8 * h][c8];
          float f[8];
          unpack8<T>(yv[c][h], f);
#pragma unroll
          for (int i = 0; i < 8; ++i) f[i] += scale * srow[i];
          store16(yp[c][h], pack8<T>(f));
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }
  // the tile's last expand item tops the tile's `done` word up to the launch's weight
  if (tid == 0 && item == h_n_consumers - 1) add_device(done_base + tile_idx, DECODE_LAUNCH_WEIGHT - (uint32_t)n_producers);
}

template <typename T>
int launch_decode_t(hipStream_t st, const DecodeArgs &a, int nb, dim3 grid, int shrink_ids) {
  switch (nb) {
    case 1: hipLaunchKernelGGL((decode_kernel<T, 1>), grid, dim3(256), 0, st, a.s.plan + a.e.off_tiles, a.done, a.n_producers, a.n_consumers, a.n_tiles, shrink_ids, a); break;
    case 2: hipLaunchKernelGGL((decode_kernel<T, 2>), grid, dim3(256), 0, st, a.s.plan + a.e.off_tiles, a.done, a.n_producers, a.n_consumers, a.n_tiles, shrink_ids, a); break;
    case 4: hipLaunchKernelGGL((decode_kernel<T, 4>), grid, dim3(256), 0, st, a.s.plan + a.e.off_tiles, a.done, a.n_producers, a.n_consumers, a.n_tiles, shrink_ids, a); break;
    default: return fail(MLORA_ERR_NO_KERNEL, "one-launch op: ranks above 64 use the two-launch path");
  }
  return check_launch("decode_kernel");
}

}  // namespace

int decode_bn(int max_rank) { return 256 * dec_ch(dec_nb(max_rank)); }

// floats of scratch the one-launch op needs for its partials: [tile][target][K chunk][16][rp]
size_t decode_partial_floats(int64_t n_tiles, int n_targets, int ksplit, int64_t rp) {
  return (size_t)n_tiles * (size_t)n_targets * (size_t)ksplit * 16u * (size_t)rp;
}

int launch_decode(hipStream_t st, const DecodeArgs &a, int max_rank, mlora_dtype dt) {
  int nb = (max_rank + 15) / 16;
  nb = nb <= 1 ? 1 : nb <= 2 ? 2 : nb <= 4 ? 4 : 8;
  if (a.n_tiles <= 0) return MLORA_OK;
  if (a.n_producers > DECODE_MAX_PRODUCERS)
    return fail(MLORA_ERR_NO_KERNEL, "one-launch op: ksplit * targets = %d exceeds %d", a.n_producers, DECODE_MAX_PRODUCERS);
  const int64_t groups = (a.n_tiles + 7) / 8;
  const int64_t shrink_ids = groups * 8 * a.n_producers;
  const int64_t total = shrink_ids + groups * 8 * a.n_consumers;
  if (total > 0x7fffffff) return fail(MLORA_ERR_NO_KERNEL, "one-launch op: grid too large");
  dim3 grid((unsigned)total);
  return dt == MLORA_F16 ? launch_decode_t<_Float16>(st, a, nb, grid, (int)shrink_ids)
                         : launch_decode_t<__bf16>(st, a, nb, grid, (int)shrink_ids);
}

}  // namespace mlora
