// LoRA shrink for gfx950:  v[row, j] = T( sum_k x[t, k] * A_a[j, k] )
//
// One workgroup (4 waves) owns one adapter-grouped tile of up to 16*MB tokens and one K-chunk.
// Both operands are K-contiguous in memory (token rows of x, rank rows of the pool), which is
// exactly the per-lane layout v_mfma_f32_16x16x32 wants: lane (row = lane%16, kgroup = lane/16)
// holds 8 consecutive K elements, so every operand is a single 16-byte global load straight
// into the MFMA source registers -- no LDS staging, no transposes.  The four waves interleave
// 32-element K-steps, so the workgroup reads 256 contiguous bytes of every row per round, and
// several K-steps are loaded before any is consumed (the kernel is latency bound: what counts
// is the number of 16-byte loads in flight per lane).
//
// Split-K without atomics: every workgroup writes its fp32 partial tile and is done; the chunks
// are summed in index order (bit-reproducible) by shrink_reduce_kernel or by the expand.
//
// Reference semantics: valora/csrc/bgmv/bgmv_impl.cuh:14-148 (per-token gather mat-vec with the
// rank rows gathered through loc_indicies, fp32 accumulation, one T store per output).
#include "kernel_common.h"
#include "shrink_core.h"

namespace mlora {

namespace {


// the arguments of target z of a multi-target launch
__device__ __forceinline__ ShrinkArgs select_target(const ShrinkArgs &a, int z) {
  ShrinkArgs p = a;
  p.slot = a.slots[z];
  p.out = a.out + (int64_t)z * a.out_tstride;
  p.partial = a.partial + (int64_t)z * a.partial_tstride;
  return p;
}

template <typename T>
__device__ __forceinline__ void store_v(const ShrinkArgs &p, int pos, int t, int r, int col, float v) {
  using Tr = Traits<T>;
  if (p.out_by_token) {
    // the caller's matrix, one row per token (dispatch_bgmv and friends)
    uint16_t *dst = p.out + (int64_t)t * p.out_stride + col;
    if (col < r && col < p.ncols) {
      if (p.mode == MLORA_SHRINK_ACCUMULATE) v += Tr::to_float(*dst);
      *dst = Tr::from_float(v);
    } else if (p.mode == MLORA_SHRINK_ZERO_PAD && col < p.width) {
      *dst = 0;
    }
  } else {
    // internal v buffer, one row of rp columns per sorted position; columns >= r hold zero
    if (col < p.rp) p.out[(int64_t)pos * p.out_stride + col] = Tr::from_float(col < r ? v : 0.f);
  }
}

// Epilogue shared by both shrink kernels.  `tile` is the workgroup's fp32 result in LDS, row-major
// with row stride ld: rows = tokens of the tile, columns = rank.
//   ksplit == 1 : rounded to T and stored.
//   ksplit  > 1 : stored as this K-chunk's fp32 partial (ordinary stores, then the workgroup is
//                 done); a later launch on the stream -- shrink_reduce_kernel, or the expand
//                 itself for small batches -- sums the chunks in index order and rounds once.
// (shrink_kernel can also sum the chunks itself, see there.)
template <typename T>
__device__ __forceinline__ void shrink_epilogue(const ShrinkArgs &p, const float *tile, int ld, int s, int pos0,
                                                int cnt, int r, const int32_t *perm) {
  const int tid = threadIdx.x;
  if (p.ksplit == 1) {
    const int n_el = cnt * p.rp;
    for (int e = tid; e < n_el; e += 256) {
      const int row = e / p.rp, col = e - row * p.rp;
      store_v<T>(p, pos0 + row, p.out_by_token ? perm[pos0 + row] : 0, r, col, tile[row * ld + col]);
    }
    return;
  }
  const int quarter = p.rp >> 2;       // rp is a multiple of 16
  const int n_vec = cnt * quarter;
  f32x4 *part = reinterpret_cast<f32x4 *>(p.partial + ((int64_t)s * p.T + pos0) * p.rp);
  for (int e = tid; e < n_vec; e += 256) {
    const int row = e / quarter, c4 = e - row * quarter;
    const float *src = tile + row * ld + 4 * c4;
    part[e] = f32x4{src[0], src[1], src[2], src[3]};
  }
}

// v[row, :] = T(sum_s partial[s][row][:]) for every row that has an adapter; one thread per four
// columns, every chunk requested before any is consumed.
template <typename T>
__global__ __launch_bounds__(256) void shrink_reduce_kernel(ShrinkArgs args_in) {
  const ShrinkArgs p = select_target(args_in, blockIdx.y);
  const int n_active = p.plan[H_NACTIVE];
  const int quarter = p.rp >> 2;
  const int64_t total = (int64_t)n_active * quarter;
  const int32_t *__restrict__ perm = p.plan + p.off_perm;
  const int32_t *__restrict__ prank = p.plan + p.off_prank;
  const int64_t sstride = (int64_t)p.T * quarter;
  const f32x4 *src = reinterpret_cast<const f32x4 *>(p.partial);
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
    const int pos = (int)(e / quarter), c4 = (int)(e - (int64_t)pos * quarter);
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < p.ksplit; s0 += 8) {
      f32x4 q[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) q[u] = (s0 + u < p.ksplit) ? src[(s0 + u) * sstride + e] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int u = 0; u < 8; ++u) v += q[u];
    }
    const int r = prank[pos];
    const int t = p.out_by_token ? perm[pos] : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) store_v<T>(p, pos, t, r, 4 * c4 + i, v[i]);
  }
}

// The leading scalar parameters repeat what the first dependent load (the tile record) needs: with kernel-argument
// preloading they arrive in registers at launch, so that load does not wait for a load of the argument block.
template <typename T, int MB, int NB>
__global__ __launch_bounds__(256) void shrink_kernel(const int32_t *tiles_base, int h_ksplit, int h_n_targets, int h_reduce_here,
                                                     int h_n_tiles, ShrinkArgs args_in) {
  int tile_idx, z_idx, s;
  if (h_reduce_here) {
    // The K chunks of a tile are summed by whichever of them finishes last, out of the L2 they share: the id
    // mod 8 selects the XCD, so all chunks (and targets) of a tile get ids that agree mod 8.
    const int per_tile = h_n_targets * h_ksplit;
    const int local = blockIdx.x >> 3, tl = local / per_tile, rem = local - tl * per_tile;
    tile_idx = tl * 8 + (blockIdx.x & 7);
    z_idx = rem / h_ksplit;
    s = rem - z_idx * h_ksplit;
    if (tile_idx >= h_n_tiles) return;
  } else {
    // workgroup id = (tile * targets + target) * ksplit + K chunk.  The id mod 8 selects the XCD, so
    // with the K chunk as the fast index the tiles of an adapter that share a K chunk of A, and the
    // targets that share a K chunk of x, meet in one L2.
    const int wg_tz = blockIdx.x / h_ksplit;
    tile_idx = wg_tz / h_n_targets;
    z_idx = wg_tz - tile_idx * h_n_targets;
    s = blockIdx.x - wg_tz * h_ksplit;
  }
  const int32_t *__restrict__ tile = tiles_base + (int64_t)tile_idx * TILE_WORDS;
  const ShrinkArgs p = select_target(args_in, z_idx);
  constexpr int NBLK = MB * NB;
  __shared__ float red[2][NBLK * 256];
  __shared__ int s_last;

  const int r = tile[1], pos0 = tile[2], cnt = tile[3], astart = tile[4];
  if (cnt <= 0) return;   // records past the last tile are zero
  const int32_t *__restrict__ perm = p.plan + p.off_perm;
  const int kbeg = s * p.kchunk;
  const int kend = min(p.h_in, kbeg + p.kchunk);
  shrink_tile_to_lds<T, MB, NB>(p.x, p.h_in, p.pool, p.slot, perm, r, pos0, cnt, astart, kbeg, kend, red);
  if (!p.reduce_here || p.ksplit == 1) {
    shrink_epilogue<T>(p, red[1], NB * 16, s, pos0, cnt, r, perm);
    return;
  }

  // ---- split-K summed here: every chunk leaves its partial in the L2, the last one to arrive adds them up.
  // Partials are plain stores into rows that own whole 128-byte lines (prp floats per row), so a line never
  // holds rows of two tiles and no compute unit has read it before the tile is complete.  A chunk announces
  // itself -- after its stores have been acknowledged by the L2 -- by adding to the tile's arrival word (one
  // atomic per workgroup, device scope): the count in the low byte, and one more count in the field of the XCD
  // it runs on.  Whoever brings the count to ksplit is the last: it knows all partials are written, and from
  // its XCD's field whether all of them were written through ITS L2.  If so it reads them back (L2 hits) and
  // sums them in index order; if not (the workgroups of the tile were not placed the way the id layout
  // expects) it computes every chunk itself, in the same order with the same code: same bits, no waiting
  // anywhere, and nothing depends on where or when a workgroup runs.  It then puts the word back to zero for
  // the next launch on this plan (launches that share a plan must not overlap).
  // (Worth it for small tiles only: one workgroup reads ksplit x tile x prp x 4 bytes at L2 latency.  For
  // 128-token tiles of rank 64 that is 256 KB and measured 8.5 us, against 3.7 us for the reduce launch.)
  const int tid = threadIdx.x;
  const int quarter = p.rp >> 2, pq = p.prp >> 2;
  {
    f32x4 *part = reinterpret_cast<f32x4 *>(p.partial + ((int64_t)s * p.T + pos0) * p.prp);
    for (int e = tid; e < cnt * quarter; e += 256) {
      const int row = e / quarter, c4 = e - row * quarter;
      const float *src = red[1] + row * (NB * 16) + 4 * c4;
      part[row * pq + c4] = f32x4{src[0], src[1], src[2], src[3]};
    }
  }
  wait_vmcnt<0>();
  __syncthreads();
  if (tid == 0) {
    const uint32_t xcd = xcd_id();
    unsigned long long *word = p.arrive + (int64_t)tile_idx * MLORA_MAX_TARGETS + z_idx;
    const unsigned long long add = 1ull + (xcd < 8 ? 1ull << (8 + 7 * xcd) : 0ull);
    const unsigned long long now = __hip_atomic_fetch_add(word, add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + add;
    int last = 0;
    if ((int)(now & 0xffull) == p.ksplit) {
      const bool all_here = xcd < 8 && (int)((now >> (8 + 7 * xcd)) & 0x7full) == p.ksplit;
      last = (all_here && p.reduce_here == 1) ? 1 : 2;
      __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    s_last = last;
  }
  __syncthreads();
  const int last = s_last;
  if (last == 0) return;
  if (last == 1) {
    // v[row, :] = T(0 + p_0 + p_1 + ...): the order shrink_reduce_kernel uses
    const f32x4 *src = reinterpret_cast<const f32x4 *>(p.partial + (int64_t)pos0 * p.prp);
    const int64_t sstride = (int64_t)p.T * pq;
    for (int e = tid; e < cnt * quarter; e += 256) {
      const int row = e / quarter, c4 = e - row * quarter;
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      for (int s0 = 0; s0 < p.ksplit; s0 += 8) {
        f32x4 q[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          q[u] = (s0 + u < p.ksplit) ? src[(s0 + u) * sstride + row * pq + c4] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 8; ++u) v += q[u];
      }
      const int t = p.out_by_token ? perm[pos0 + row] : 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) store_v<T>(p, pos0 + row, t, r, 4 * c4 + i, v[i]);
    }
    return;
  }
  // the chunks were not all written through this XCD's L2 (or the caller asked for this path): compute them
  // here, one after the other, and add them up in LDS
  __shared__ float vacc[16 * MB * NB * 16];
  for (int e = tid; e < 16 * MB * NB * 16; e += 256) vacc[e] = 0.f;
  for (int c = 0; c < p.ksplit; ++c) {
    const int kb = c * p.kchunk;
    __syncthreads();
    shrink_tile_to_lds<T, MB, NB>(p.x, p.h_in, p.pool, p.slot, perm, r, pos0, cnt, astart, kb, min(p.h_in, kb + p.kchunk),
                                  red);
    for (int e = tid; e < 16 * MB * NB * 16; e += 256) vacc[e] += red[1][e];
  }
  __syncthreads();
  for (int e = tid; e < cnt * p.rp; e += 256) {
    const int row = e / p.rp, col = e - row * p.rp;
    store_v<T>(p, pos0 + row, p.out_by_token ? perm[pos0 + row] : 0, r, col, vacc[row * (NB * 16) + col]);
  }
}

// Prefill-sized tiles (128 tokens): GEMM structure with a three-stage LDS ring.
//
// The four waves split the tile's tokens (32 each), so no cross-wave reduction is needed.  Both
// operands of a 64-wide K step go from global memory straight into LDS with 16-byte
// global_load_lds (no registers are held while the data is in flight): every wave streams its
// own x rows into a private part of the stage, the adapter's A rows are loaded once per
// workgroup and shared by all waves.  A load instruction covers 8 rows x 128 contiguous bytes
// (whole cache lines: asking for the two halves of a line with two instructions measured up to
// 30 % slower) and writes them to LDS in lane order, so a stage holds rows of 128 bytes; the
// lane that fills 16-byte chunk c of row R fetches global chunk c ^ (R & 7), which spreads the
// later ds_read_b128 of an MFMA operand (16 rows, one chunk column) over the banks.  Two stages
// are always in flight while the third is consumed; one s_barrier per K step.
template <typename T, int NB, int MBW>
__global__ __launch_bounds__(256) void shrink_gemm_kernel(const int32_t *tiles_base, int h_ksplit, int h_n_targets, int, int,
                                                          ShrinkArgs args_in) {
  // workgroup id = (tile * targets + target) * ksplit + K chunk.  The id mod 8 selects the XCD, so
  // with the K chunk as the fast index the tiles of an adapter that share a K chunk of A, and the
  // targets that share a K chunk of x, meet in one L2.
  const int wg_tz = blockIdx.x / h_ksplit;
  const int tile_idx = wg_tz / h_n_targets;
  const ShrinkArgs p = select_target(args_in, wg_tz - tile_idx * h_n_targets);
  const int s = blockIdx.x - wg_tz * h_ksplit;
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  constexpr int KC = 64, KS = KC / 32, STAGES = 3;      // MBW: 16-token blocks per wave (tile = 64 * MBW tokens)
  static_assert(KC * 2 == 128, "a K step is one 128-byte line per row");
  constexpr int XBLK = MBW * 2;                         // 8-row groups (1 KB) of x per wave per stage
  constexpr int ABLK = NB * 2;                          // 8-row groups of A per stage (shared)
  constexpr int APW = ABLK >= 4 ? ABLK / 4 : 1;         // A groups each wave loads per stage
  constexpr int A_SLOTS = APW * 4;                      // >= ABLK; surplus slots hold duplicates
  constexpr int STAGE_BYTES = (4 * XBLK + A_SLOTS) * 1024;
  constexpr int TILE_BYTES = 64 * MBW * NB * 16 * 4;
  constexpr int LOADS_PER_STAGE = XBLK + APW;           // per wave, identical for all waves
  constexpr int RING_BYTES = STAGES * STAGE_BYTES + 1024;   // + one scratch block for dummy loads
  __shared__ __align__(16) unsigned char s_raw[RING_BYTES > TILE_BYTES ? RING_BYTES : TILE_BYTES];

  const int32_t *__restrict__ tile = tiles_base + (int64_t)tile_idx * TILE_WORDS;
  const int r = tile[1], pos0 = tile[2], cnt = tile[3], astart = tile[4];
  if (cnt <= 0) return;   // records past the last tile are zero

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, kg = lane >> 4;           // MFMA operand roles
  const int grow = lane >> 3;                           // loader roles: row within an 8-row group,
  const int gchunk = (lane & 7) ^ grow;                 // global 16-byte chunk this lane fetches
  const int32_t *__restrict__ perm = p.plan + p.off_perm;
  const int64_t base = (int64_t)astart + (int64_t)r * p.slot;
  const int wrow0 = wave * 16 * MBW;
  const bool wave_active = wrow0 < cnt;                 // wave-uniform

  // this lane's global row pointers (already at its chunk)
  const uint16_t *xp[XBLK];
  bool xok[XBLK];
#pragma unroll
  for (int g = 0; g < XBLK; ++g) {
    const int row = wrow0 + g * 8 + grow;
    xok[g] = row < cnt;
    const int t = xok[g] ? perm[pos0 + row] : 0;
    xp[g] = p.x + (int64_t)t * p.h_in + gchunk * 8;
  }
  // A groups this wave loads: slot = wave*APW + i -> rows slot*8 .. slot*8+7 of the rank
  const uint16_t *ap[APW];
  bool aok[APW];
#pragma unroll
  for (int i = 0; i < APW; ++i) {
    const int slot = (wave * APW + i) % ABLK;           // surplus slots duplicate real groups
    const int j = slot * 8 + grow;
    const int64_t idx = base + j;
    bool ok = j < r && idx >= 0 && idx < p.pool.a_loc_len;
    const int64_t prow = ok ? p.pool.a_loc[idx] : 0;
    ok = ok && prow >= 0 && prow < p.pool.w_rows;
    aok[i] = ok;
    ap[i] = p.pool.w + (ok ? prow : 0) * p.h_in + gchunk * 8;
  }

  const int kbeg = s * p.kchunk;
  const int kend = min(p.h_in, kbeg + p.kchunk);
  const int n_steps = (kend - kbeg + KC - 1) / KC;

  // byte offsets inside a stage: x rows of this wave, then the shared A rows
  const uint32_t ring = lds_offset(s_raw);
  const uint32_t x_off = (uint32_t)(wave * XBLK) * 1024u;
  const uint32_t a_off = (uint32_t)(4 * XBLK) * 1024u;
  const u32x4 zero4 = {0, 0, 0, 0};

  // Issue every load of one K step: EXACTLY LOADS_PER_STAGE load instructions per wave, because the
  // consumer waits with a compile-time vmcnt.  A load whose lanes are all masked off would be skipped
  // by the hardware branch around it, so in that case a dummy load into a scratch block is issued
  // instead.  Lanes beyond the end of K write zeros into their own slot (no other lane touches it).
  unsigned char *dummy = s_raw + STAGES * STAGE_BYTES;
  auto load_or_dummy = [&](bool c, const uint16_t *src, unsigned char *dst) {
    if (__builtin_amdgcn_ballot_w64(c) != 0ull) {
      if (c) __builtin_amdgcn_global_load_lds(GLOBAL_PTR(src), LDS_PTR(dst), 16, 0, 0);
    } else {
      __builtin_amdgcn_global_load_lds(GLOBAL_PTR(p.plan), LDS_PTR(dummy), 16, 0, 0);
    }
  };
  auto issue = [&](int step) {
    const int stage = step % STAGES;
    const int k = kbeg + step * KC + gchunk * 8;        // first K element of this lane's chunk
    const bool kok = k < kend;
    unsigned char *sbase = s_raw + stage * STAGE_BYTES;
#pragma unroll
    for (int g = 0; g < XBLK; ++g) {
      unsigned char *dst = sbase + x_off + g * 1024;
      load_or_dummy(xok[g] && kok, xp[g] + kbeg + step * KC, dst);
      if (!kok) lds_write16(lds_offset(dst) + lane * 16, zero4);
    }
#pragma unroll
    for (int i = 0; i < APW; ++i) {
      unsigned char *dst = sbase + a_off + (wave * APW + i) * 1024;
      load_or_dummy(aok[i] && kok, ap[i] + kbeg + step * KC, dst);
      if (!kok) lds_write16(lds_offset(dst) + lane * 16, zero4);
    }
  };
  // where the MFMA operand (row R of a region, K block ks) of this lane sits inside a stage
  auto frag_off = [&](int R, int ks) -> uint32_t {
    return (uint32_t)R * 128u + (uint32_t)(((ks * 4 + kg) ^ (R & 7)) * 16);
  };

  f32x4 acc[MBW][NB];
#pragma unroll
  for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  issue(0);
  if (n_steps > 1) issue(1);
  for (int step = 0; step < n_steps; ++step) {
    // wait for this step's loads (the next step's may stay in flight), then meet the other waves:
    // after the barrier the stage is complete for everybody and the stage consumed in the previous
    // iteration is free to be refilled
    if (step + 1 < n_steps) wait_vmcnt<LOADS_PER_STAGE>(); else wait_vmcnt<0>();
    wait_lgkmcnt0();
    __builtin_amdgcn_s_barrier();
    if (step + 2 < n_steps) issue(step + 2);
    const int stage = step % STAGES;
    if (wave_active) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        u32x4 xf[MBW], bf[NB];
#pragma unroll
        for (int mb = 0; mb < MBW; ++mb)
          xf[mb] = lds_read16(ring + stage * STAGE_BYTES + x_off + frag_off(mb * 16 + lrow, ks));
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          bf[nb] = lds_read16(ring + stage * STAGE_BYTES + a_off + frag_off(nb * 16 + lrow, ks));
        wait_lgkmcnt0();
#pragma unroll
        for (int mb = 0; mb < MBW; ++mb) pin(xf[mb]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) pin(bf[nb]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          if (nb * 16 < r) {
#pragma unroll
            for (int mb = 0; mb < MBW; ++mb)
              acc[mb][nb] = Tr::mfma(as<vec8>(xf[mb]), as<vec8>(bf[nb]), acc[mb][nb]);
          }
        }
      }
    }
  }
  wait_lgkmcnt0();
  __syncthreads();   // everybody is done reading the ring: reuse it for the result tile

  float *otile = reinterpret_cast<float *>(s_raw);
#pragma unroll
  for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = wrow0 + mb * 16 + kg * 4 + i;
        const int col = nb * 16 + lrow;
        otile[row * (NB * 16) + col] = acc[mb][nb][i];
      }
  __syncthreads();
  shrink_epilogue<T>(p, otile, NB * 16, s, pos0, cnt, r, perm);
}

template <typename T, int MBW>
int launch_gemm_nb(hipStream_t st, const ShrinkArgs &a, int nb, dim3 grid) {
  switch (nb) {
    case 1: hipLaunchKernelGGL((shrink_gemm_kernel<T, 1, MBW>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.ksplit, a.n_targets, a.reduce_here, a.n_tiles, a); break;
    case 2: hipLaunchKernelGGL((shrink_gemm_kernel<T, 2, MBW>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.ksplit, a.n_targets, a.reduce_here, a.n_tiles, a); break;
    case 4: hipLaunchKernelGGL((shrink_gemm_kernel<T, 4, MBW>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.ksplit, a.n_targets, a.reduce_here, a.n_tiles, a); break;
    case 8:
      if constexpr (MBW <= 2) {
        hipLaunchKernelGGL((shrink_gemm_kernel<T, 8, MBW>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.ksplit, a.n_targets, a.reduce_here, a.n_tiles, a);
        break;
      }
      return fail(MLORA_ERR_NO_KERNEL, "shrink: rank > 64 has no 256-token tile");
    default: return fail(MLORA_ERR_NO_KERNEL, "shrink: no kernel for rank blocks=%d", nb);
  }
  return check_launch("shrink_gemm_kernel");
}

template <typename T, int MB>
int launch_shrink_nb(hipStream_t st, const ShrinkArgs &a, int nb, dim3 grid) {
  switch (nb) {
    case 1: hipLaunchKernelGGL((shrink_kernel<T, MB, 1>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.ksplit, a.n_targets, a.reduce_here, a.n_tiles, a); break;
    case 2: hipLaunchKernelGGL((shrink_kernel<T, MB, 2>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.ksplit, a.n_targets, a.reduce_here, a.n_tiles, a); break;
    case 4: hipLaunchKernelGGL((shrink_kernel<T, MB, 4>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.ksplit, a.n_targets, a.reduce_here, a.n_tiles, a); break;
    case 8: hipLaunchKernelGGL((shrink_kernel<T, (MB > 2 ? 2 : MB), 8>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.ksplit, a.n_targets, a.reduce_here, a.n_tiles, a); break;
    default: return fail(MLORA_ERR_NO_KERNEL, "shrink: no kernel for rank blocks=%d", nb);
  }
  return check_launch("shrink_kernel");
}

template <typename T>
int launch_shrink_t(hipStream_t st, const ShrinkArgs &a, int bm, int nb, dim3 grid) {
  switch (bm) {
    case 16: return launch_shrink_nb<T, 1>(st, a, nb, grid);
    case 32: return launch_shrink_nb<T, 2>(st, a, nb, grid);
    case 64: return launch_shrink_nb<T, 4>(st, a, nb, grid);
    case 128: return launch_gemm_nb<T, 2>(st, a, nb, grid);
    case 256: return launch_gemm_nb<T, 4>(st, a, nb, grid);
    default: return fail(MLORA_ERR_NO_KERNEL, "shrink: tile height %d not in {16,32,64,128,256}", bm);
  }
}

}  // namespace

int launch_shrink_reduce(hipStream_t st, const ShrinkArgs &a, mlora_dtype dt) {
  if (a.T <= 0) return MLORA_OK;
  int64_t blocks = ((int64_t)a.T * (a.rp >> 2) + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  if (blocks < 1) blocks = 1;
  if (dt == MLORA_F16)
    hipLaunchKernelGGL(shrink_reduce_kernel<_Float16>, dim3((unsigned)blocks, (unsigned)a.n_targets), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL(shrink_reduce_kernel<__bf16>, dim3((unsigned)blocks, (unsigned)a.n_targets), dim3(256), 0, st, a);
  return check_launch("shrink_reduce_kernel");
}

int launch_shrink(hipStream_t st, const ShrinkArgs &a, int bm, int max_rank, int64_t grid_tiles,
                  mlora_dtype dt) {
  int nb = (max_rank + 15) / 16;
  nb = nb <= 1 ? 1 : nb <= 2 ? 2 : nb <= 4 ? 4 : 8;
  if (nb == 8 && (bm == 64 || bm == 256)) return fail(MLORA_ERR_NO_KERNEL, "shrink: rank > 64 needs tile height 16, 32 or 128");
  if (grid_tiles <= 0) return MLORA_OK;
  if (a.reduce_here) grid_tiles = (grid_tiles + 7) / 8 * 8;   // ids are dealt to the 8 XCDs tile by tile
  if (grid_tiles * a.ksplit * a.n_targets > 0x7fffffff) return fail(MLORA_ERR_NO_KERNEL, "shrink: grid too large");
  dim3 grid((unsigned)(grid_tiles * a.ksplit * a.n_targets));
  return dt == MLORA_F16 ? launch_shrink_t<_Float16>(st, a, bm, nb, grid)
                         : launch_shrink_t<__bf16>(st, a, bm, nb, grid);
}

}  // namespace mlora
