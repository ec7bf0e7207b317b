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
// Split-K without atomics on data: every workgroup writes its fp32 partial tile, then bumps a
// per-tile counter in the plan; the workgroup that arrives last sums the `ksplit` partials in
// index order (so the result does not depend on which one was last), rounds once to T and
// stores v.  No workgroup ever waits for another, and the counter is reset for the next launch.
//
// Reference semantics: valora/csrc/bgmv/bgmv_impl.cuh:14-148 (per-token gather mat-vec with the
// rank rows gathered through loc_indicies, fp32 accumulation, one T store per output).
#include "kernel_common.h"

namespace mlora {

namespace {

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
//   ksplit  > 1 : stored as this K-chunk's partial; the last workgroup of the tile to get here sums
//                 the ksplit partials in index order (the result does not depend on which one was
//                 last) and stores v.
// The partials are written with device-scope stores and read back with device-scope loads, two
// floats at a time, so they never rely on an XCD's L2 being written back or invalidated: a full
// device-scope fence would flush and invalidate the whole L2 of the XCD once per workgroup
// (measured: 5-10x slower kernels).  __syncthreads() waits until the stores are acknowledged.
template <typename T>
__device__ __forceinline__ void shrink_epilogue(const ShrinkArgs &p, const float *tile, int ld, int tile_idx, int s,
                                                int pos0, int cnt, int r, const int32_t *perm, int *s_last) {
  const int tid = threadIdx.x;
  if (p.ksplit == 1) {
    const int n_el = cnt * p.rp;
    for (int e = tid; e < n_el; e += 256) {
      const int row = e / p.rp, col = e - row * p.rp;
      store_v<T>(p, pos0 + row, p.out_by_token ? perm[pos0 + row] : 0, r, col, tile[row * ld + col]);
    }
    return;
  }
  const int half = p.rp >> 1;          // rp is a multiple of 16
  const int n_pair = cnt * half;
  if (p.partial_only) {
    // the next launch on the stream sums the chunks: ordinary stores, no counters
    float2 *part = reinterpret_cast<float2 *>(p.partial + ((int64_t)s * p.T + pos0) * p.rp);
    for (int e = tid; e < n_pair; e += 256) {
      const int row = e / half, c2 = e - row * half;
      part[e] = make_float2(tile[row * ld + 2 * c2], tile[row * ld + 2 * c2 + 1]);
    }
    return;
  }
  {
    unsigned long long *part = reinterpret_cast<unsigned long long *>(p.partial + ((int64_t)s * p.T + pos0) * p.rp);
    for (int e = tid; e < n_pair; e += 256) {
      const int row = e / half, c2 = e - row * half;
      const float2 v = make_float2(tile[row * ld + 2 * c2], tile[row * ld + 2 * c2 + 1]);
      __hip_atomic_store(part + e, __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  __syncthreads();
  if (tid == 0) {
    const int prev = atomicAdd(p.counters + tile_idx, 1);
    *s_last = (prev == p.ksplit - 1);
  }
  __syncthreads();
  if (!*s_last) return;
  const unsigned long long *src = reinterpret_cast<const unsigned long long *>(p.partial + (int64_t)pos0 * p.rp);
  const int64_t sstride = (int64_t)p.T * half;
  for (int e = tid; e < n_pair; e += 256) {
    const int row = e / half, c2 = e - row * half;
    float2 v = make_float2(0.f, 0.f);
    // eight partials are requested before any is consumed (each is a round trip to memory);
    // the sum itself runs in index order
    for (int s0 = 0; s0 < p.ksplit; s0 += 8) {
      unsigned long long q[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        q[u] = (s0 + u < p.ksplit)
                   ? __hip_atomic_load(src + (s0 + u) * sstride + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                   : 0ull;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float2 f = __builtin_bit_cast(float2, q[u]);
        v.x += f.x;
        v.y += f.y;
      }
    }
    const int t = p.out_by_token ? perm[pos0 + row] : 0;
    store_v<T>(p, pos0 + row, t, r, 2 * c2, v.x);
    store_v<T>(p, pos0 + row, t, r, 2 * c2 + 1, v.y);
  }
  if (tid == 0) p.counters[tile_idx] = 0;  // ready for the next launch that uses this plan
}

template <typename T, int MB, int NB>
__global__ __launch_bounds__(256) void shrink_kernel(ShrinkArgs p) {
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  constexpr int NBLK = MB * NB;
  __shared__ float red[2][NBLK * 256];
  __shared__ int s_last;

  const int32_t *__restrict__ hdr = p.plan;
  const int tile_idx = blockIdx.x;
  if (tile_idx >= hdr[H_NTILES_S]) return;
  const int32_t *__restrict__ tile = p.plan + p.off_tiles + (int64_t)tile_idx * TILE_WORDS;
  const int r = tile[1], pos0 = tile[2], cnt = tile[3], astart = tile[4];
  const int s = blockIdx.y;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, kg = lane >> 4;
  const int32_t *__restrict__ perm = p.plan + p.off_perm;
  const int64_t base = (int64_t)astart + (int64_t)r * p.slot;

  const uint16_t *xp[MB];
  bool xok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int row = mb * 16 + lrow;
    xok[mb] = row < cnt;
    const int t = xok[mb] ? perm[pos0 + row] : 0;
    xp[mb] = p.x + (int64_t)t * p.h_in;
  }
  const uint16_t *wp[NB];
  bool wok[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int j = nb * 16 + lrow;
    const int64_t idx = base + j;
    bool ok = (j < r) && idx >= 0 && idx < p.pool.a_loc_len;
    int64_t row = ok ? p.pool.a_loc[idx] : 0;
    ok = ok && row >= 0 && row < p.pool.w_rows;
    wok[nb] = ok;
    wp[nb] = p.pool.w + (ok ? row : 0) * p.h_in;
  }

  f32x4 acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int kbeg = s * p.kchunk;
  const int kend = min(p.h_in, kbeg + p.kchunk);
  // The trip count must be wave-uniform: MFMA ignores EXEC, so a lane that left the loop early
  // would still feed its stale registers into the matrix core.  Lanes past the end load zeros.
  constexpr int U = (MB + NB <= 2) ? 8 : (MB + NB <= 4) ? 4 : (MB + NB <= 8) ? 2 : 1;
  for (int kb0 = kbeg + wave * 32; kb0 < kend; kb0 += 128 * U) {
    u32x4 xa[U][MB], wb[U][NB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = kb0 + u * 128 + kg * 8;
      const bool kok = k < kend;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) xa[u][mb] = (xok[mb] && kok) ? load16(xp[mb] + k) : u32x4{0, 0, 0, 0};
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) wb[u][nb] = (wok[nb] && kok) ? load16(wp[nb] + k) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        if (nb * 16 < r) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            acc[mb][nb] = Tr::mfma(as<vec8>(xa[u][mb]), as<vec8>(wb[u][nb]), acc[mb][nb]);
        }
      }
    }
  }

  // cross-wave reduction (tree): waves 2,3 -> LDS, waves 0,1 add; wave 1 -> LDS, wave 0 adds.
  if (wave >= 2) {
    float *dst = red[wave - 2];
#pragma unroll
    for (int b = 0; b < NBLK; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[(b * 4 + i) * 64 + lane] = acc[b / NB][b % NB][i];
  }
  __syncthreads();
  if (wave < 2) {
    const float *src = red[wave];
#pragma unroll
    for (int b = 0; b < NBLK; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[b / NB][b % NB][i] += src[(b * 4 + i) * 64 + lane];
  }
  __syncthreads();
  if (wave == 1) {
    float *dst = red[0];
#pragma unroll
    for (int b = 0; b < NBLK; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[(b * 4 + i) * 64 + lane] = acc[b / NB][b % NB][i];
  }
  __syncthreads();
  if (wave == 0) {
    // wave 0 adds the last slot and leaves the finished tile in red[1], row-major
    const float *src = red[0];
    float *otile = red[1];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int b = mb * NB + nb;
          const int row = mb * 16 + kg * 4 + i;  // C layout: column = lane%16, rows = 4*(lane/16)+i
          const int col = nb * 16 + lrow;
          otile[row * (NB * 16) + col] = acc[mb][nb][i] + src[(b * 4 + i) * 64 + lane];
        }
  }
  __syncthreads();
  shrink_epilogue<T>(p, red[1], NB * 16, tile_idx, s, pos0, cnt, r, perm, &s_last);
}

// Prefill-sized tiles: GEMM structure.  The four waves split the tile's tokens (16*MBW each), so
// no cross-wave reduction is needed; the adapter's A rows for the current 128-wide K step are
// staged once per workgroup in LDS (double buffered) and shared by all waves, which cuts the
// weight traffic into the compute unit by the tile height; x fragments still go straight from
// global memory into MFMA registers.  The next step's A tile and x fragments are requested
// before the current step is consumed.
template <typename T, int MBW, int NB>
__global__ __launch_bounds__(256) void shrink_gemm_kernel(ShrinkArgs p) {
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  constexpr int KC = (NB > 4) ? 64 : 128;     // K elements per step
  constexpr int KS = KC / 32;                 // MFMA k-steps per step
  constexpr int LDA = KC + 8;                 // LDS row stride (elements): 16 B of padding
  constexpr int AV = NB * 16 * (KC / 8) / 256;  // 16-byte vectors of the A tile per thread
  constexpr int VPR = KC / 8;                 // vectors per A row
  // LDS: two A buffers during the K loop, then the workgroup's fp32 result tile
  constexpr int A_BYTES = 2 * NB * 16 * LDA * 2;
  constexpr int TILE_BYTES = 64 * MBW * NB * 16 * 4;
  __shared__ __align__(16) unsigned char s_raw[A_BYTES > TILE_BYTES ? A_BYTES : TILE_BYTES];
  uint16_t(*s_a)[NB * 16][LDA] = reinterpret_cast<uint16_t(*)[NB * 16][LDA]>(s_raw);
  __shared__ int s_last;

  const int32_t *__restrict__ hdr = p.plan;
  const int tile_idx = blockIdx.x;
  if (tile_idx >= hdr[H_NTILES_S]) return;
  const int32_t *__restrict__ tile = p.plan + p.off_tiles + (int64_t)tile_idx * TILE_WORDS;
  const int r = tile[1], pos0 = tile[2], cnt = tile[3], astart = tile[4];
  const int s = blockIdx.y;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, kg = lane >> 4;
  const int32_t *__restrict__ perm = p.plan + p.off_perm;
  const int64_t base = (int64_t)astart + (int64_t)r * p.slot;
  const int wrow0 = wave * 16 * MBW;          // first tile row of this wave
  const bool wave_active = wrow0 < cnt;       // wave-uniform

  const uint16_t *xp[MBW];
  bool xok[MBW];
#pragma unroll
  for (int mb = 0; mb < MBW; ++mb) {
    const int row = wrow0 + mb * 16 + lrow;
    xok[mb] = row < cnt;
    const int t = xok[mb] ? perm[pos0 + row] : 0;
    xp[mb] = p.x + (int64_t)t * p.h_in;
  }
  // A staging role of this thread: vectors id = tid + i*256 -> (row = id / VPR, vector = id % VPR)
  const uint16_t *ap[AV];
  bool aok[AV];
  int arow[AV], acv[AV];
#pragma unroll
  for (int i = 0; i < AV; ++i) {
    const int id = tid + i * 256;
    arow[i] = id / VPR;
    acv[i] = id % VPR;
    const int64_t idx = base + arow[i];
    bool ok = arow[i] < r && idx >= 0 && idx < p.pool.a_loc_len;
    const int64_t prow = ok ? p.pool.a_loc[idx] : 0;
    ok = ok && prow >= 0 && prow < p.pool.w_rows;
    aok[i] = ok;
    ap[i] = p.pool.w + (ok ? prow : 0) * p.h_in + acv[i] * 8;
  }

  f32x4 acc[MBW][NB];
#pragma unroll
  for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int kbeg = s * p.kchunk;
  const int kend = min(p.h_in, kbeg + p.kchunk);

  u32x4 xa[MBW][KS], na[AV];
  auto load_x = [&](int k0, u32x4 (&dst)[MBW][KS]) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int k = k0 + ks * 32 + kg * 8;
#pragma unroll
      for (int mb = 0; mb < MBW; ++mb) dst[mb][ks] = (xok[mb] && k < kend) ? load16(xp[mb] + k) : u32x4{0, 0, 0, 0};
    }
  };
  auto load_a = [&](int k0) {
#pragma unroll
    for (int i = 0; i < AV; ++i) na[i] = (aok[i] && k0 + acv[i] * 8 < kend) ? load16(ap[i] + k0) : u32x4{0, 0, 0, 0};
  };
  auto store_a = [&](int buf) {
#pragma unroll
    for (int i = 0; i < AV; ++i) *reinterpret_cast<u32x4 *>(&s_a[buf][arow[i]][acv[i] * 8]) = na[i];
  };

  load_a(kbeg);
  load_x(kbeg, xa);
  store_a(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = kbeg; k0 < kend; k0 += KC) {
    const bool more = k0 + KC < kend;  // workgroup-uniform
    u32x4 nx[MBW][KS];
    if (more) {
      load_a(k0 + KC);
      load_x(k0 + KC, nx);
    }
    if (wave_active) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          if (nb * 16 < r) {
            const u32x4 bf = *reinterpret_cast<const u32x4 *>(&s_a[buf][nb * 16 + lrow][ks * 32 + kg * 8]);
#pragma unroll
            for (int mb = 0; mb < MBW; ++mb)
              acc[mb][nb] = Tr::mfma(as<vec8>(xa[mb][ks]), as<vec8>(bf), acc[mb][nb]);
          }
        }
      }
    }
    if (more) {
      store_a(buf ^ 1);
#pragma unroll
      for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) xa[mb][ks] = nx[mb][ks];
    }
    __syncthreads();
    buf ^= 1;
  }

  // every wave holds the complete K-chunk sums of its own tokens: lay the tile out row-major
  // in LDS (the A buffers are free after the loop's last barrier)
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
  shrink_epilogue<T>(p, otile, NB * 16, tile_idx, s, pos0, cnt, r, perm, &s_last);
}

template <typename T, int MBW>
int launch_gemm_nb(hipStream_t st, const ShrinkArgs &a, int nb, dim3 grid) {
  switch (nb) {
    case 1: hipLaunchKernelGGL((shrink_gemm_kernel<T, MBW, 1>), grid, dim3(256), 0, st, a); break;
    case 2: hipLaunchKernelGGL((shrink_gemm_kernel<T, MBW, 2>), grid, dim3(256), 0, st, a); break;
    case 4: hipLaunchKernelGGL((shrink_gemm_kernel<T, MBW, 4>), grid, dim3(256), 0, st, a); break;
    case 8: hipLaunchKernelGGL((shrink_gemm_kernel<T, MBW, 8>), grid, dim3(256), 0, st, a); break;
    default: return fail(MLORA_ERR_NO_KERNEL, "shrink: no kernel for rank blocks=%d", nb);
  }
  return check_launch("shrink_gemm_kernel");
}

template <typename T, int MB>
int launch_shrink_nb(hipStream_t st, const ShrinkArgs &a, int nb, dim3 grid) {
  switch (nb) {
    case 1: hipLaunchKernelGGL((shrink_kernel<T, MB, 1>), grid, dim3(256), 0, st, a); break;
    case 2: hipLaunchKernelGGL((shrink_kernel<T, MB, 2>), grid, dim3(256), 0, st, a); break;
    case 4: hipLaunchKernelGGL((shrink_kernel<T, MB, 4>), grid, dim3(256), 0, st, a); break;
    case 8: hipLaunchKernelGGL((shrink_kernel<T, (MB > 2 ? 2 : MB), 8>), grid, dim3(256), 0, st, a); break;
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
    default: return fail(MLORA_ERR_NO_KERNEL, "shrink: tile height %d not in {16,32,64,128}", bm);
  }
}

}  // namespace

int launch_shrink(hipStream_t st, const ShrinkArgs &a, int bm, int max_rank, int64_t grid_tiles,
                  mlora_dtype dt) {
  int nb = (max_rank + 15) / 16;
  nb = nb <= 1 ? 1 : nb <= 2 ? 2 : nb <= 4 ? 4 : 8;
  if (nb == 8 && bm == 64) return fail(MLORA_ERR_NO_KERNEL, "shrink: rank > 64 needs tile height 16, 32 or 128");
  if (grid_tiles <= 0) return MLORA_OK;
  dim3 grid((unsigned)grid_tiles, (unsigned)a.ksplit);
  return dt == MLORA_F16 ? launch_shrink_t<_Float16>(st, a, bm, nb, grid)
                         : launch_shrink_t<__bf16>(st, a, bm, nb, grid);
}

}  // namespace mlora
