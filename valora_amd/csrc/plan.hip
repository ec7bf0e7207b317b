// Ragged segment / adapter-index builders for gfx950.
//
//  * plan_kernel              stable counting sort of tokens by adapter + adapter-grouped tile
//                             lists (what the shrink / expand kernels iterate over)
//  * count_consecutive_kernel parallel run-length encoding, bit-exact with the reference's
//                             single-thread count_consecutive_requests
//                             (atmm/valora/csrc/bgmv/bgmv_impl.cuh:39-72)
//  * ids_fill / ids_cover_*   per-token ids from segment or per-request operands
//
// All are single-workgroup or trivially parallel integer kernels: the inputs are a few KB and
// the work is launch-latency bound, so one 1024-thread workgroup with LDS histograms is used
// instead of a multi-pass device-wide sort.
#include "mlora_internal.h"

namespace mlora {

namespace {

constexpr int PLAN_THREADS = 1024;   // large batches; decode-sized ones run with PLAN_THREADS_SMALL
constexpr int PLAN_THREADS_SMALL = 256;
constexpr int PLAN_WAVES = PLAN_THREADS / 64;
constexpr int HIST_WORDS = 8192;  // LDS words for the per-wave histograms

__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    int n = __shfl_up(v, d, 64);
    if (lane >= d) v += n;
  }
  return v;
}

// exclusive prefix of v over the workgroup's threads (n_waves waves); *total gets the block sum.
__device__ __forceinline__ int block_exclusive_scan(int v, int *total, int *wsum /* LDS[17] */, int n_waves = PLAN_WAVES) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int inc = wave_inclusive_scan(v, lane);
  __syncthreads();  // wsum may still be read from a previous scan
  if (lane == 63) wsum[wave] = inc;
  __syncthreads();
  if (wave == 0) {
    int w = lane < n_waves ? wsum[lane] : 0;
    int winc = wave_inclusive_scan(w, lane);
    if (lane < n_waves) wsum[lane] = winc - w;
    if (lane == n_waves - 1) wsum[PLAN_WAVES] = winc;
  }
  __syncthreads();
  *total = wsum[PLAN_WAVES];
  return wsum[wave] + inc - v;
}

// The same for four counters at once (one pass of barriers instead of four).
struct Quad {
  int c, ts, te, g;
};
__device__ __forceinline__ Quad quad_add(Quad a, Quad b) { return Quad{a.c + b.c, a.ts + b.ts, a.te + b.te, a.g + b.g}; }
__device__ __forceinline__ Quad quad_wave_inclusive_scan(Quad v, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    Quad n{__shfl_up(v.c, d, 64), __shfl_up(v.ts, d, 64), __shfl_up(v.te, d, 64), __shfl_up(v.g, d, 64)};
    if (lane >= d) v = quad_add(v, n);
  }
  return v;
}
__device__ __forceinline__ Quad block_exclusive_scan4(Quad v, Quad *total, Quad *wsum /* LDS[17] */, int n_waves) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const Quad inc = quad_wave_inclusive_scan(v, lane);
  if (lane == 63) wsum[wave] = inc;
  __syncthreads();
  if (wave == 0) {
    const Quad w = lane < n_waves ? wsum[lane] : Quad{0, 0, 0, 0};
    const Quad winc = quad_wave_inclusive_scan(w, lane);
    if (lane < n_waves) wsum[lane] = Quad{winc.c - w.c, winc.ts - w.ts, winc.te - w.te, winc.g - w.g};
    if (lane == n_waves - 1) wsum[PLAN_WAVES] = winc;
  }
  __syncthreads();
  *total = wsum[PLAN_WAVES];
  const Quad base = wsum[wave];
  return Quad{base.c + inc.c - v.c, base.ts + inc.ts - v.ts, base.te + inc.te - v.te, base.g + inc.g - v.g};
}

constexpr int PLAN_SMALL_A = 2048;   // adapters whose per-adapter tables fit in LDS next to the histograms

// SMALL: the per-adapter tables (counts, group starts, tile offsets, ranks, a_start) live in LDS instead of
// the plan's scratch area, so the dependent look-ups of the later phases (the binary search of the tile
// lists above all) cost LDS latency instead of a global round trip each.
// THREADS: 1024, or 256 for decode-sized batches (a few hundred tokens), where the barriers and scans of sixteen
// waves cost more than the work they organise.
template <bool SMALL, int THREADS>
__global__ __launch_bounds__(THREADS) void plan_kernel(
    int32_t *__restrict__ plan, const int64_t *__restrict__ ids, const int64_t *__restrict__ a_start,
    const int64_t *__restrict__ a_len, int T, int A, int n_slots, int bm_s, int bm_e, int W,
    int64_t off_perm, int64_t off_padapter, int64_t off_prank, int64_t off_tiles_s,
    int64_t off_tiles_e, int64_t off_counters, int64_t off_scratch, int max_tiles, int n_flag_words) {
  constexpr int N_WAVES = THREADS / 64;
  __shared__ int32_t whist[HIST_WORDS];
  __shared__ Quad wsum[PLAN_WAVES + 1];
  __shared__ int s_wmaxr[PLAN_WAVES];

  __shared__ int32_t s_tab[SMALL ? 4 * PLAN_SMALL_A : 1];
  __shared__ int32_t s_rank[SMALL ? PLAN_SMALL_A : 1];
  __shared__ int64_t s_astart[SMALL ? PLAN_SMALL_A : 1];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int32_t *perm = plan + off_perm;
  int32_t *padapter = plan + off_padapter;
  int32_t *prank = plan + off_prank;
  int32_t *cnt = SMALL ? s_tab : plan + off_scratch;
  int32_t *gstart = cnt + (SMALL ? PLAN_SMALL_A : A);
  int32_t *toff_s = gstart + (SMALL ? PLAN_SMALL_A : A);
  int32_t *toff_e = toff_s + (SMALL ? PLAN_SMALL_A : A);
  // rank of adapter a (0 = not usable: ranks are multiples of 8 up to MAX_RANK) and its a_start
  auto rank_of = [&](int a) -> int {
    if (SMALL) return s_rank[a];
    const int64_t r = a_len[a] / n_slots;
    return (r > 0 && (r & 7) == 0 && r <= MAX_RANK) ? (int)r : 0;
  };
  auto start_of = [&](int a) -> int64_t { return SMALL ? s_astart[a] : a_start[a]; };

  // token range of each of the W histogram waves (contiguous, multiple of 64)
  const int cw = (int)align_up((T + W - 1) / W, 64);
  const int t_beg = wave * cw;
  const int t_end = (wave < W) ? min(T, t_beg + cw) : 0;

  // Every global load the set-up needs is requested before the first store: a wave gets its memory results in
  // issue order, so a load queued behind the zero-fill below would wait for those stores as well.
  const int64_t id0 = (t_beg + lane < t_end) ? ids[t_beg + lane] : -1;
  int64_t len0 = 0, start0 = 0;
  if (SMALL && tid < A) { len0 = a_len[tid]; start0 = a_start[tid]; }

  for (int i = tid; i < W * A; i += THREADS) whist[i] = 0;
  if (SMALL) {
    for (int a = tid; a < A; a += THREADS) {
      const int64_t r = (a == tid ? len0 : a_len[a]) / n_slots;
      s_rank[a] = (r > 0 && (r & 7) == 0 && r <= MAX_RANK) ? (int)r : 0;
      s_astart[a] = a == tid ? start0 : a_start[a];
    }
  }
  __syncthreads();
  for (int i = tid; i < n_flag_words; i += THREADS) plan[off_counters + i] = 0;

  // 1. per-wave histogram of valid tokens (the first 64 tokens of a wave stay in registers for step 3)
  int first_a = -1, first_r = 0;
  for (int t = t_beg + lane; t < t_end; t += 64) {
    const int64_t a64 = (t < t_beg + 64) ? id0 : ids[t];
    int a = -1, r = 0;
    if (a64 >= 0 && a64 < A) {
      r = rank_of((int)a64);
      if (r > 0) {
        a = (int)a64;
        atomicAdd(&whist[wave * A + a], 1);
      }
    }
    if (t < t_beg + 64) { first_a = a; first_r = r; }
  }
  __syncthreads();

  // 2. per-adapter totals, group starts, tile offsets (each thread owns a run of adapters)
  const int per = (A + THREADS - 1) / THREADS;
  const int a_beg = min(A, tid * per), a_endx = min(A, a_beg + per);
  int my_c = 0, my_ts = 0, my_te = 0, my_g = 0, my_maxr = 0;
  for (int a = a_beg; a < a_endx; ++a) {
    int c = 0;
    for (int w = 0; w < W; ++w) c += whist[w * A + a];
    cnt[a] = c;
    if (c > 0) {
      my_c += c;
      my_ts += (c + bm_s - 1) / bm_s;
      my_te += (c + bm_e - 1) / bm_e;
      my_g += 1;
      my_maxr = max(my_maxr, rank_of(a));
    }
  }
  Quad tot;
  const Quad pre = block_exclusive_scan4(Quad{my_c, my_ts, my_te, my_g}, &tot, wsum, N_WAVES);
  const int n_active = tot.c, n_ts = tot.ts, n_te = tot.te, n_g = tot.g;
  int pre_c = pre.c, pre_ts = pre.ts, pre_te = pre.te;
  {
    // widest rank among the adapters that have tokens.  Ranks are multiples of 8 up to MAX_RANK: a few votes per wave
    // find the wave's maximum (an LDS atomic per lane is serialised lane by lane by the compiler: 1.8 us here)
    int wave_maxr = 0;
    for (int rr = MAX_RANK; rr >= 8; rr -= 8)
      if (__ballot(my_maxr >= rr)) { wave_maxr = rr; break; }
    if (lane == 0) s_wmaxr[wave] = wave_maxr;
  }
  for (int a = a_beg; a < a_endx; ++a) {
    const int c = cnt[a];
    gstart[a] = pre_c;
    toff_s[a] = pre_ts;
    toff_e[a] = pre_te;
    int off = pre_c;
    for (int w = 0; w < W; ++w) {  // histogram -> running write offset of (wave, adapter)
      const int h = whist[w * A + a];
      whist[w * A + a] = off;
      off += h;
    }
    pre_c += c;
    pre_ts += (c + bm_s - 1) / bm_s;
    pre_te += (c + bm_e - 1) / bm_e;
  }
  __syncthreads();

  // 3. stable scatter: each wave walks its range in order, 64 tokens a step; lanes holding the
  //    same adapter get consecutive positions in lane order.
  const int a_bits = A > 1 ? 32 - __clz(A - 1) : 0;   // bits that tell two adapter indices apart
  for (int t0 = t_beg; t0 < t_end; t0 += 64) {
    const int t = t0 + lane;
    int a = -1, r = 0;
    if (t0 == t_beg) {
      a = first_a;
      r = first_r;
    } else if (t < t_end) {
      const int64_t a64 = ids[t];
      if (a64 >= 0 && a64 < A) {
        r = rank_of((int)a64);
        if (r > 0) a = (int)a64;
      }
    }
    // Lanes holding the same adapter get consecutive positions in lane order.  Which lanes hold my adapter comes from
    // one vote per bit of the adapter index (6 votes for 64 adapters), whatever the mix: one adapter for all 64 tokens
    // of a prefill request or 64 different ones in a decode batch.
    const unsigned long long valid = __ballot(a >= 0);
    if (valid) {   // wave-uniform
      unsigned long long same = valid;
      for (int b = 0; b < a_bits; ++b) {
        const bool bit = (a >> b) & 1;
        const unsigned long long m = __ballot(bit);
        same &= bit ? m : ~m;
      }
      if (a >= 0) {
        const int slot_idx = wave * A + a;
        const int pos = whist[slot_idx] + __popcll(same & ((1ull << lane) - 1ull));
        perm[pos] = t;
        padapter[pos] = a;
        prank[pos] = r;
        __builtin_amdgcn_wave_barrier();                           // every lane of the group has read the offset ...
        if (((same >> lane) >> 1) == 0) whist[slot_idx] = pos + 1;   // ... before its last lane moves it on
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
  __syncthreads();

  // 4. tile lists: tile i belongs to the last adapter whose tile offset is <= i
  const bool one_list = bm_s == bm_e;   // then both lists are the same records (the one-launch op: 16 / 16)
  for (int pass = 0; pass < (one_list ? 1 : 2); ++pass) {
    const int n_tiles = pass ? n_te : n_ts;
    const int bm = pass ? bm_e : bm_s;
    const int32_t *toff = pass ? toff_e : toff_s;
    int32_t *tiles = plan + (pass ? off_tiles_e : off_tiles_s);
    for (int i = tid; i < n_tiles; i += THREADS) {
      int lo = 0, hi = A;  // first adapter with toff > i
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (toff[mid] <= i) lo = mid + 1; else hi = mid;
      }
      const int a = lo - 1;
      const int k = i - toff[a];
      const int c = cnt[a];
      const int64_t st = start_of(a);
      // The index has fewer than 2^31 entries (checked on the host), so a start outside 31 bits lies outside the
      // index whatever it is: it becomes a position no look-up accepts, and the adapter's rows are skipped like
      // any other row outside the pool.
      const bool st_bad = st < 0 || st > 0x7fffffff;
      const int32_t rec[5] = {a, rank_of(a), gstart[a] + k * bm, min(bm, c - k * bm),
                              st_bad ? INT32_MIN / 2 : (int32_t)st};
      for (int list = 0; list < (one_list ? 2 : 1); ++list) {
        int32_t *tl = (list ? plan + off_tiles_e : tiles) + (int64_t)i * TILE_WORDS;
#pragma unroll
        for (int q = 0; q < TILE_WORDS; ++q) tl[q] = q < 5 ? rec[q] : 0;
      }
    }
    // the kernels' grids are sized with the upper bound of the tile count: records past the last
    // tile say "no tokens", so a workgroup needs no second look-up to know that it has nothing to do
    const int upper = (T + bm - 1) / bm + min(A, T);
    for (int i = n_tiles + tid; i < upper; i += THREADS) {
      for (int list = 0; list < (one_list ? 2 : 1); ++list) {
        int32_t *tl = (list ? plan + off_tiles_e : tiles) + (int64_t)i * TILE_WORDS;
#pragma unroll
        for (int k = 0; k < TILE_WORDS; ++k) tl[k] = 0;
      }
    }
  }
  __syncthreads();
  if (tid == 0) {
    plan[H_MAGIC] = PLAN_MAGIC;
    plan[H_T] = T;
    plan[H_NADAPTERS] = A;
    plan[H_NTILES_S] = n_ts;
    plan[H_NTILES_E] = n_te;
    plan[H_NGROUPS] = n_g;
    int maxrank = 0;
    for (int wv = 0; wv < N_WAVES; ++wv) maxrank = max(maxrank, s_wmaxr[wv]);
    plan[H_MAXRANK] = maxrank;
    plan[H_RESERVED] = 0;
    plan[H_BM_S] = bm_s;
    plan[H_BM_E] = bm_e;
    plan[H_NACTIVE] = n_active;
  }
}

// Parallel RLE.  Pass 1 marks run heads and scans them; pass 2 derives the run lengths.
__global__ __launch_bounds__(PLAN_THREADS) void count_consecutive_kernel(
    const int64_t *__restrict__ lora_rank, int64_t n_adapters, const int64_t *__restrict__ indicies,
    int T, int64_t *__restrict__ output_counts, int64_t *__restrict__ rank_counts,
    int64_t *__restrict__ lora_ids, int64_t *__restrict__ start_ids, int64_t *__restrict__ num_runs) {
  __shared__ int wsum[PLAN_WAVES + 1];
  const int tid = threadIdx.x;
  int carry = 0;
  for (int t0 = 0; t0 < T; t0 += PLAN_THREADS) {
    const int t = t0 + tid;
    int head = 0;
    int64_t id = 0;
    if (t < T) {
      id = indicies[t];
      head = (t == 0) || (indicies[t - 1] != id);
    }
    int total;
    const int pre = block_exclusive_scan(head, &total, wsum);
    if (head) {
      const int k = carry + pre;
      start_ids[k] = t;
      lora_ids[k] = id;
      rank_counts[k] = (id >= 0 && id < n_adapters) ? lora_rank[id] / 4 : 0;
    }
    carry += total;
  }
  __syncthreads();  // start_ids written by this workgroup are visible to it
  const int P = carry;
  for (int k = tid; k < P; k += PLAN_THREADS) {
    const int64_t s = start_ids[k];
    const int64_t e = (k + 1 < P) ? start_ids[k + 1] : (int64_t)T;
    output_counts[k] = e - s;
  }
  if (tid == 0) num_runs[0] = P;
}

__global__ void ids_fill_kernel(int64_t *ids_out, int64_t T, int64_t v) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < T) ids_out[t] = v;
}

__global__ void ids_cover_segments_kernel(int64_t *ids_out, const int64_t *ids_in,
                                          const int64_t *start_ids, const int64_t *output_counts,
                                          int64_t T) {
  const int64_t i = blockIdx.x;
  const int64_t s = start_ids[i], n = output_counts[i];
  if (s < 0 || n <= 0) return;
  const int64_t e = (s + n < T) ? s + n : T;
  for (int64_t t = s + threadIdx.x; t < e; t += blockDim.x) ids_out[t] = ids_in[t];
}

__global__ void ids_cover_requests_kernel(int64_t *ids_out, const int32_t *b_start_loc,
                                          const int32_t *b_seq_len, const int64_t *b_indicies,
                                          int64_t T, int64_t max_rows) {
  const int64_t i = blockIdx.x;
  const int64_t s = b_start_loc[i];
  int64_t n = b_seq_len[i];
  if (n > max_rows) n = max_rows;
  if (s < 0 || n <= 0) return;
  const int64_t e = (s + n < T) ? s + n : T;
  const int64_t a = b_indicies[i];
  for (int64_t t = s + threadIdx.x; t < e; t += blockDim.x) ids_out[t] = a;
}

}  // namespace

int launch_plan(hipStream_t st, int32_t *plan, const PlanLayout &L, const int64_t *ids,
                const int64_t *a_start, const int64_t *a_len, int n_slots, int bm_s, int bm_e) {
  const int A = (int)L.A;
  int W = A > 0 ? (int)(HIST_WORDS / A) : PLAN_WAVES;
  if (W > PLAN_WAVES) W = PLAN_WAVES;
  if (W < 1) return fail(MLORA_ERR_NO_KERNEL, "plan: more than %lld adapters", (long long)MAX_ADAPTERS);
  // the histogram is spread over as many waves as there are, W <= waves of the workgroup
  const bool few = L.T <= 1024 && A <= 512;
  if (few && W > PLAN_THREADS_SMALL / 64) W = PLAN_THREADS_SMALL / 64;
#define MLORA_LAUNCH_PLAN(SMALL, THREADS)                                                                          \
  hipLaunchKernelGGL((plan_kernel<SMALL, THREADS>), dim3(1), dim3(THREADS), 0, st, plan, ids, a_start, a_len,      \
                     (int)L.T, A, n_slots, bm_s, bm_e, W, L.off_perm, L.off_padapter, L.off_prank, L.off_tiles_s,  \
                     L.off_tiles_e, L.off_counters, L.off_scratch, (int)L.max_tiles,                              \
                     (int)(L.off_scratch - L.off_counters))
  if (few) MLORA_LAUNCH_PLAN(true, PLAN_THREADS_SMALL);
  else if (A <= PLAN_SMALL_A) MLORA_LAUNCH_PLAN(true, PLAN_THREADS);
  else MLORA_LAUNCH_PLAN(false, PLAN_THREADS);
#undef MLORA_LAUNCH_PLAN
  return check_launch("plan_kernel");
}

int launch_count_consecutive(hipStream_t st, const int64_t *lora_rank, int64_t n_adapters,
                             const int64_t *indicies, int64_t T, int64_t *output_counts,
                             int64_t *rank_counts, int64_t *lora_ids, int64_t *start_ids,
                             int64_t *num_runs) {
  hipLaunchKernelGGL(count_consecutive_kernel, dim3(1), dim3(PLAN_THREADS), 0, st, lora_rank,
                     n_adapters, indicies, (int)T, output_counts, rank_counts, lora_ids, start_ids,
                     num_runs);
  return check_launch("count_consecutive_kernel");
}

int launch_ids_from_segments(hipStream_t st, int64_t *ids_out, const int64_t *ids_in,
                             const int64_t *start_ids, const int64_t *output_counts, int64_t P,
                             int64_t T) {
  if (T <= 0) return MLORA_OK;
  hipLaunchKernelGGL(ids_fill_kernel, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, st, ids_out, T,
                     (int64_t)-1);
  if (int rc = check_launch("ids_fill_kernel")) return rc;
  if (P <= 0) return MLORA_OK;
  hipLaunchKernelGGL(ids_cover_segments_kernel, dim3((unsigned)P), dim3(256), 0, st, ids_out, ids_in,
                     start_ids, output_counts, T);
  return check_launch("ids_cover_segments_kernel");
}

int launch_ids_from_requests(hipStream_t st, int64_t *ids_out, const int32_t *b_start_loc,
                             const int32_t *b_seq_len, const int64_t *b_indicies, int64_t n_req,
                             int64_t T, int64_t max_rows) {
  if (T <= 0) return MLORA_OK;
  hipLaunchKernelGGL(ids_fill_kernel, dim3((unsigned)((T + 255) / 256)), dim3(256), 0, st, ids_out, T,
                     (int64_t)-1);
  if (int rc = check_launch("ids_fill_kernel")) return rc;
  if (n_req <= 0) return MLORA_OK;
  hipLaunchKernelGGL(ids_cover_requests_kernel, dim3((unsigned)n_req), dim3(256), 0, st, ids_out,
                     b_start_loc, b_seq_len, b_indicies, T, max_rows);
  return check_launch("ids_cover_requests_kernel");
}

}  // namespace mlora
