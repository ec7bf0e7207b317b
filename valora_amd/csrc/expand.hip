// LoRA expand for gfx950:  y[t, o] = T( y[t, o] + scale_a * sum_{j<r} T(v[t, j]) * B_a[j, o] )
//
// The pool stores a slot's B block as [H_out, r] row-major spread over r pool rows, so output
// column o owns r consecutive elements at flat offset o*r: the B operand of the MFMA (column =
// output, 8 consecutive rank elements per lane) is again one 16-byte global load per lane, and
// 16 neighbouring outputs are one contiguous 32*r-byte run.  A workgroup owns one adapter-grouped
// tile of tokens and 256 output columns (64 per wave); each wave loads its B fragments once into
// registers and reuses them for every 16-token block of the tile.  The fp32 MFMA result is
// turned through a small LDS tile so that the read-modify-write of y is done with 16-byte
// accesses of 128 contiguous bytes per token row; the add is done in fp32 and rounded once.
//
// v is a T matrix: either the shrink's internal buffer (rows in sorted-position order; rounded
// to T once, as the reference does by holding `delta` in a T tensor between its two launches)
// or a matrix supplied by the caller (rows in token order).
//
// Reference semantics: valora/csrc/bgmv/bgmv_impl.cuh:152-207.
#include "kernel_common.h"

namespace mlora {

namespace {

constexpr int EXP_BN = 256;       // outputs per workgroup
constexpr int EXP_WN = 64;        // outputs per wave
constexpr int STAGE_LD = EXP_WN + 4;
constexpr int EXP_MBU = 2;         // 16-token blocks whose loads are in flight together
constexpr int EXP_MAX_BM = 256;   // tallest expand tile (tokens), one thread per token at set-up


// the arguments of target z of a multi-target launch
__device__ __forceinline__ ExpandArgs select_target(const ExpandArgs &a, int z) {
  ExpandArgs p = a;
  p.slot = a.slots[z];
  p.y = a.ys[z];
  p.pool.w = a.ws[z];
  p.pool.w_rows = a.w_rows_t[z];
  p.v = a.v + (int64_t)z * a.v_tstride;
  if (a.partial) p.partial = a.partial + (int64_t)z * a.partial_tstride;
  return p;
}

// Waves per SIMD the register allocator has to leave room for.  The rank-64 variant that reads a finished
// v sits 2 registers above the 96 that allow 5 waves; held to 5 it measured 1-6 % faster on the prefill and
// mixed shapes (more workgroups resident per round), at 6 it spills.  The others are left to the compiler.
constexpr int expand_min_waves(int kb, bool partial) { return (kb == 2 && !partial) ? 5 : 1; }

template <typename T, int KB, bool PARTIAL>
__global__ __launch_bounds__(256, expand_min_waves(KB, PARTIAL)) void expand_kernel(const int32_t *tiles_base, int h_n_ochunks,
                                                                                    ExpandArgs args_in) {
  // (tiles_base, h_n_ochunks: what the first dependent load needs, in front so that kernel-argument preloading
  // delivers them in registers)
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  __shared__ float stage[4][16][STAGE_LD];
  __shared__ int32_t s_perm[EXP_MAX_BM];

  const int tile_idx = blockIdx.x / h_n_ochunks;
  const int oc = blockIdx.x - tile_idx * h_n_ochunks;
  const int32_t *__restrict__ tile = tiles_base + (int64_t)tile_idx * TILE_WORDS;
  const int a = tile[0], r = tile[1], pos0 = tile[2], cnt = tile[3], astart = tile[4];
  if (cnt <= 0) return;   // records past the last tile are zero
  const ExpandArgs p = select_target(args_in, blockIdx.y);
  const int rk = min(r, p.kmax);  // rank columns the narrow operand really has (bgmv_impl.cuh:167,186)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, kg = lane >> 4;
  const int64_t base = (int64_t)astart + (int64_t)r * p.slot;
  const int o_wave = oc * EXP_BN + wave * EXP_WN;

  // Everything that depends only on the tile header is requested first, in one round trip:
  // the tile's token indices, the pool rows of the B fragments and the scale.
  int my_perm = 0;
  if (tid < cnt) my_perm = p.plan[p.off_perm + pos0 + tid];
  const float scale = Tr::to_float(p.scales[a]);
  const float inv_h_out = 1.0f / (float)p.h_out;
  int64_t brow[4][KB];
  uint32_t boff[4][KB];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int o = o_wave + nb * 16 + lrow;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int j0 = kb * 32 + kg * 8;
      brow[nb][kb] = -1;
      boff[nb][kb] = 0;
      if (o < p.h_out && j0 < rk) {
        const uint32_t flat = (uint32_t)o * (uint32_t)r + (uint32_t)j0;   // < 2^16 * 2^7
        uint32_t bin;
        divmod24(flat, (uint32_t)p.h_out, inv_h_out, bin, boff[nb][kb]);
        const int64_t idx = base + bin;
        if (idx >= 0 && idx < p.pool.a_loc_len) brow[nb][kb] = p.pool.a_loc[idx];
      }
    }
  }
  s_perm[tid] = my_perm;
  // The only workgroup-wide barrier: it also drains the loads above (which everything below needs
  // anyway).  No barrier may follow the bulk loads below -- a barrier waits for all outstanding
  // global loads and would serialise the B, y and v traffic into separate round trips.
  __syncthreads();

  // B fragments: bfrag[nb][kb] = B^T[o = o_wave + nb*16 + lrow][j0 .. j0+8), j0 = kb*32 + kg*8
  u32x4 bfrag[4][KB];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int64_t row = brow[nb][kb];
      bfrag[nb][kb] = (row >= 0 && row < p.pool.w_rows) ? load16(p.pool.w + row * p.h_out + boff[nb][kb])
                                                        : u32x4{0, 0, 0, 0};
    }

  // row-major roles for the y read-modify-write: 8 lanes x 16 B cover one token row of the wave's
  // 64 outputs; a wave covers 8 rows per access, two accesses per 16-token block.
  const int rr0 = lane >> 3, c8 = (lane & 7) * 8;
  const bool ocol_ok = (o_wave + c8) < p.h_out;

  // Two 16-token blocks per iteration: their y rows and v fragments are all requested before either
  // block is consumed, so an iteration costs one memory round trip for 32 tokens.
  const int n_mb = (cnt + 15) >> 4;
  for (int mb0 = 0; mb0 < n_mb; mb0 += EXP_MBU) {
    u32x4 yv[EXP_MBU][2];
    uint16_t *yp[EXP_MBU][2];
    bool yok[EXP_MBU][2];
    u32x4 vfrag[EXP_MBU][KB];
#pragma unroll
    for (int b = 0; b < EXP_MBU; ++b) {
      const int mb = mb0 + b;
      // ---- y rows first (the longest-latency loads of the iteration)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int row = mb * 16 + rr0 + 8 * h;
        yok[b][h] = ocol_ok && row < cnt;
        const int t = yok[b][h] ? s_perm[row] : 0;
        yp[b][h] = p.y + (int64_t)t * p.h_out + o_wave + c8;
        yv[b][h] = yok[b][h] ? load16(yp[b][h]) : u32x4{0, 0, 0, 0};
      }
      // ---- v fragments: rows = tokens (lrow), 8 consecutive rank elements per lane
      const int prow = mb * 16 + lrow;
      const bool pok = prow < cnt;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int j0 = kb * 32 + kg * 8;
        u32x4 v = {0, 0, 0, 0};
        if (pok && j0 < rk) {
          if constexpr (PARTIAL) {
            // split-K partials of the shrink: all chunks are requested before any is consumed,
            // summed in chunk order and rounded to T once
            float f[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            const float *src0 = p.partial + ((int64_t)pos0 + prow) * p.rp + j0;
            const int64_t sstride = (int64_t)p.T * p.rp;
            for (int s0 = 0; s0 < p.ksplit; s0 += 4) {
              f32x4 lo[4], hi[4];
#pragma unroll
              for (int u = 0; u < 4; ++u) {
                const bool ok = s0 + u < p.ksplit;
                const f32x4 *src = reinterpret_cast<const f32x4 *>(src0 + (int64_t)(s0 + u) * sstride);
                lo[u] = ok ? src[0] : f32x4{0.f, 0.f, 0.f, 0.f};
                hi[u] = ok ? src[1] : f32x4{0.f, 0.f, 0.f, 0.f};
              }
#pragma unroll
              for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i) { f[i] += lo[u][i]; f[4 + i] += hi[u][i]; }
            }
            v = pack8<T>(f);
          } else {
            const int64_t vrow = p.v_by_pos ? (int64_t)(pos0 + prow) : (int64_t)s_perm[prow];
            v = load16(p.v + vrow * p.v_stride + j0);
          }
        }
        vfrag[b][kb] = v;
      }
    }
#pragma unroll
    for (int b = 0; b < EXP_MBU; ++b) {
      if (mb0 + b < n_mb) {   // workgroup-uniform
        // ---- delta block through the matrix cores, staged to LDS in token-major order
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
          f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
            if (kb * 32 < rk) acc = Tr::mfma(as<vec8>(vfrag[b][kb]), as<vec8>(bfrag[nb][kb]), acc);
#pragma unroll
          for (int i = 0; i < 4; ++i) stage[wave][kg * 4 + i][nb * 16 + lrow] = acc[i];
        }
        // stage[wave] is private to this wave and a wave's LDS operations execute in order, so only
        // the compiler has to be kept from reordering the reads below over the writes above.
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          if (yok[b][h]) {
            const float *srow = &stage[wave][rr0 + 8 * h][c8];
            float f[8];
            unpack8<T>(yv[b][h], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] += scale * srow[i];
            store16(yp[b][h], pack8<T>(f));
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
    }
  }
}

// Decode-like tiles (at most 16 tokens, tile height 16): a (tile, 256-column chunk) pair is a few KB of B and y, too
// little for a workgroup of its own -- a q+k+v call of 256 decode tokens is 3000 workgroups that live 4.7 us each,
// most of it the look-up chain in front of the loads, and run in three rounds.  Here a workgroup walks over `h_cl`
// consecutive column chunks of one tile: tile record, token ids, the slot's pool rows (kept in LDS, so a chunk's B
// addresses need no further look-up) and the v fragment are fetched once, then every chunk is one round trip (B
// fragments and y rows requested together), and the grid is a quarter of the size.  Same arithmetic in the same
// order as expand_kernel: same bits.
template <typename T, int KB, bool PARTIAL>
__global__ __launch_bounds__(256) void expand_cols_kernel(const int32_t *tiles_base, int h_groups, int h_cl,
                                                          ExpandArgs args_in) {
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  __shared__ float stage[4][16][STAGE_LD];
  __shared__ int32_t s_perm[16];
  __shared__ int32_t s_row[MAX_RANK];

  const int tile_idx = blockIdx.x / h_groups;
  const int grp = blockIdx.x - tile_idx * h_groups;
  const int32_t *__restrict__ tile = tiles_base + (int64_t)tile_idx * TILE_WORDS;
  const int a = tile[0], r = tile[1], pos0 = tile[2], cnt = tile[3], astart = tile[4];
  if (cnt <= 0) return;   // records past the last tile are zero
  const ExpandArgs p = select_target(args_in, blockIdx.y);
  const int rk = min(r, p.kmax);  // rank columns the narrow operand really has (bgmv_impl.cuh:167,186)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, kg = lane >> 4;
  const int64_t base = (int64_t)astart + (int64_t)r * p.slot;

  // one round trip: the tile's token indices, the pool rows of the slot and the scale
  int my_perm = 0, my_row = -1;
  if (tid < cnt) my_perm = p.plan[p.off_perm + pos0 + tid];
  if (tid < r) {
    const int64_t idx = base + tid;
    if (idx >= 0 && idx < p.pool.a_loc_len) {
      const int64_t row = p.pool.a_loc[idx];
      if (row >= 0 && row < p.pool.w_rows) my_row = (int)row;   // pool rows fit 31 bits (checked on the host)
    }
  }
  const float scale = Tr::to_float(p.scales[a]);
  if (tid < 16) s_perm[tid] = my_perm;
  if (tid < MAX_RANK) s_row[tid] = my_row;
  __syncthreads();

  // v fragment of the tile's one 16-token block: rows = tokens (lrow), 8 consecutive rank elements per lane
  u32x4 vfrag[KB];
  {
    const bool pok = lrow < cnt;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int j0 = kb * 32 + kg * 8;
      u32x4 v = {0, 0, 0, 0};
      if (pok && j0 < rk) {
        if constexpr (PARTIAL) {
          float f[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          const float *src0 = p.partial + ((int64_t)pos0 + lrow) * p.rp + j0;
          const int64_t sstride = (int64_t)p.T * p.rp;
          for (int s0 = 0; s0 < p.ksplit; s0 += 4) {
            f32x4 lo[4], hi[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const bool ok = s0 + u < p.ksplit;
              const f32x4 *src = reinterpret_cast<const f32x4 *>(src0 + (int64_t)(s0 + u) * sstride);
              lo[u] = ok ? src[0] : f32x4{0.f, 0.f, 0.f, 0.f};
              hi[u] = ok ? src[1] : f32x4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
              for (int i = 0; i < 4; ++i) { f[i] += lo[u][i]; f[4 + i] += hi[u][i]; }
          }
          v = pack8<T>(f);
        } else {
          const int64_t vrow = p.v_by_pos ? (int64_t)(pos0 + lrow) : (int64_t)s_perm[lrow];
          v = load16(p.v + vrow * p.v_stride + j0);
        }
      }
      vfrag[kb] = v;
    }
  }

  const int rr0 = lane >> 3, c8 = (lane & 7) * 8;
  const float inv_h_out = 1.0f / (float)p.h_out;
  // one chunk after the other: a chunk's B fragments and y rows are requested together, one round trip per chunk
  // (both chunks' loads in flight at once measured slower, 20.5 against 19.2 us for q+k+v: the registers they take
  // cost more resident workgroups than the round trip saves)
  const int oc_end = min(p.n_ochunks, (grp + 1) * h_cl);
  for (int oc = grp * h_cl; oc < oc_end; ++oc) {
    const int o_wave = oc * EXP_BN + wave * EXP_WN;
    if (o_wave >= p.h_out) break;   // wave-uniform
    // ---- B fragments and y rows of this chunk, all requested before any is consumed
    u32x4 bfrag[4][KB];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      const int o = o_wave + nb * 16 + lrow;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int j0 = kb * 32 + kg * 8;
        u32x4 b = {0, 0, 0, 0};
        if (o < p.h_out && j0 < rk) {
          uint32_t bin, off;
          divmod24((uint32_t)o * (uint32_t)r + (uint32_t)j0, (uint32_t)p.h_out, inv_h_out, bin, off);   // < 2^16 * 2^7
          const int row = bin < (uint32_t)MAX_RANK ? s_row[bin] : -1;
          if (row >= 0) b = load16(p.pool.w + (int64_t)row * p.h_out + off);
        }
        bfrag[nb][kb] = b;
      }
    }
    u32x4 yv[2];
    uint16_t *yp[2];
    bool yok[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int row = rr0 + 8 * h;
      yok[h] = (o_wave + c8) < p.h_out && row < cnt;
      const int t = yok[h] ? s_perm[row] : 0;
      yp[h] = p.y + (int64_t)t * p.h_out + o_wave + c8;
      yv[h] = yok[h] ? load16(yp[h]) : u32x4{0, 0, 0, 0};
    }
    // ---- delta block through the matrix cores, staged to LDS in token-major order
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
        if (kb * 32 < rk) acc = Tr::mfma(as<vec8>(vfrag[kb]), as<vec8>(bfrag[nb][kb]), acc);
#pragma unroll
      for (int i = 0; i < 4; ++i) stage[wave][kg * 4 + i][nb * 16 + lrow] = acc[i];
    }
    // stage[wave] is private to this wave and a wave's LDS operations execute in order, so only the compiler has to
    // be kept from reordering the reads below over the writes above (and the next chunk's writes over these reads)
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (yok[h]) {
        const float *srow = &stage[wave][rr0 + 8 * h][c8];
        float f[8];
        unpack8<T>(yv[h], f);
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] += scale * srow[i];
        store16(yp[h], pack8<T>(f));
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
}

template <typename T>
int launch_expand_cols_t(hipStream_t st, const ExpandArgs &a, int kb, dim3 grid, int groups, int cl) {
#define MLORA_EXPAND_COLS(KB)                                                                                       \
  if (a.partial) hipLaunchKernelGGL((expand_cols_kernel<T, KB, true>), grid, dim3(256), 0, st, a.plan + a.off_tiles, \
                                    groups, cl, a);                                                                 \
  else hipLaunchKernelGGL((expand_cols_kernel<T, KB, false>), grid, dim3(256), 0, st, a.plan + a.off_tiles, groups, cl, a)
  switch (kb) {
    case 1: MLORA_EXPAND_COLS(1); break;
    case 2: MLORA_EXPAND_COLS(2); break;
    case 4: MLORA_EXPAND_COLS(4); break;
    default: return fail(MLORA_ERR_NO_KERNEL, "expand: no kernel for %d rank blocks", kb);
  }
#undef MLORA_EXPAND_COLS
  return check_launch("expand_cols_kernel");
}

template <typename T>
int launch_expand_t(hipStream_t st, const ExpandArgs &a, int kb, dim3 grid) {
  switch (kb) {
    case 1:
      if (a.partial) hipLaunchKernelGGL((expand_kernel<T, 1, true>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.n_ochunks, a);
      else hipLaunchKernelGGL((expand_kernel<T, 1, false>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.n_ochunks, a);
      break;
    case 2:
      if (a.partial) hipLaunchKernelGGL((expand_kernel<T, 2, true>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.n_ochunks, a);
      else hipLaunchKernelGGL((expand_kernel<T, 2, false>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.n_ochunks, a);
      break;
    case 4:
      if (a.partial) hipLaunchKernelGGL((expand_kernel<T, 4, true>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.n_ochunks, a);
      else hipLaunchKernelGGL((expand_kernel<T, 4, false>), grid, dim3(256), 0, st, a.plan + a.off_tiles, a.n_ochunks, a);
      break;
    default: return fail(MLORA_ERR_NO_KERNEL, "expand: no kernel for %d rank blocks", kb);
  }
  return check_launch("expand_kernel");
}

}  // namespace

int launch_expand(hipStream_t st, const ExpandArgs &a, int max_rank, int64_t grid_tiles, int bm_expand, mlora_dtype dt) {
  int kb = (max_rank + 31) / 32;
  kb = kb <= 1 ? 1 : kb <= 2 ? 2 : 4;
  if (grid_tiles <= 0) return MLORA_OK;
  // 16-token tiles whose (tile, chunk, target) grid is well above the 1280 workgroups the device holds at once: two
  // column chunks per workgroup (measured on 256 decode tokens / 64 adapters: q+k+v 22.6 -> 19.2 us, gate+up
  // 4096 -> 11008 29.4 -> 23.5 us, gate 19.0 -> 15.9 us; four chunks 21.2 / 23.1 / 17.2; a 1280-workgroup grid
  // such as a single 11008 -> 4096 target gets slower, 14.6 -> 16.0 us, and stays as it is)
  const int cl = 2;
  const bool many = grid_tiles * a.n_ochunks * a.n_targets >= 1920;
  if (bm_expand == 16 && a.n_ochunks >= 2 && (many || a.column_loop)) {
    const int groups = (a.n_ochunks + cl - 1) / cl;
    const int64_t blocks = grid_tiles * groups;
    if (blocks > 0x7fffffff) return fail(MLORA_ERR_NO_KERNEL, "expand: grid too large");
    dim3 grid((unsigned)blocks, (unsigned)a.n_targets);
    return dt == MLORA_F16 ? launch_expand_cols_t<_Float16>(st, a, kb, grid, groups, cl)
                           : launch_expand_cols_t<__bf16>(st, a, kb, grid, groups, cl);
  }
  const int64_t blocks = grid_tiles * a.n_ochunks;
  if (blocks > 0x7fffffff) return fail(MLORA_ERR_NO_KERNEL, "expand: grid too large");
  dim3 grid((unsigned)blocks, (unsigned)a.n_targets);
  return dt == MLORA_F16 ? launch_expand_t<_Float16>(st, a, kb, grid)
                         : launch_expand_t<__bf16>(st, a, kb, grid);
}

int expand_bn() { return EXP_BN; }

}  // namespace mlora
