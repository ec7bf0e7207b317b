// The direct-load shrink of one tile and one K range, shared by the two-launch shrink kernel and by
// the one-launch decode kernel (which must produce the same bits, chunk for chunk).
//
// One workgroup (4 waves) owns up to 16*MB tokens of one adapter.  Both operands are K-contiguous in
// memory (token rows of x, rank rows of the pool), which is exactly the per-lane layout
// v_mfma_f32_16x16x32 wants: lane (row = lane%16, kgroup = lane/16) holds 8 consecutive K elements,
// so every operand is a single 16-byte global load straight into the MFMA source registers -- no LDS
// staging, no transposes.  The four waves interleave 32-element K-steps, so the workgroup reads 256
// contiguous bytes of every row per round, and several K-steps are loaded before any is consumed
// (the kernel is latency bound: what counts is the number of 16-byte loads in flight per lane).
//
// Reference semantics: valora/csrc/bgmv/bgmv_impl.cuh:14-148 (per-token gather mat-vec with the
// rank rows gathered through loc_indicies, fp32 accumulation).
#pragma once

#include "kernel_common.h"

namespace mlora {

// Leaves the fp32 result of K range [kbeg, kend) in red[1], row-major with row stride NB*16
// (rows = tokens of the tile, columns = rank); every thread of the workgroup must call it, and all
// have passed a barrier when it returns.
template <typename T, int MB, int NB>
__device__ __forceinline__ void shrink_tile_to_lds(const uint16_t *__restrict__ x, int h_in, const PoolDev &pool,
                                                   int slot, const int32_t *__restrict__ perm, int r, int pos0,
                                                   int cnt, int astart, int kbeg, int kend,
                                                   float (*red)[MB * NB * 256]) {
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  constexpr int NBLK = MB * NB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, kg = lane >> 4;
  const int64_t base = (int64_t)astart + (int64_t)r * slot;

  const uint16_t *xp[MB];
  bool xok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int row = mb * 16 + lrow;
    xok[mb] = row < cnt;
    const int t = xok[mb] ? perm[pos0 + row] : 0;
    xp[mb] = x + (int64_t)t * h_in;
  }
  const uint16_t *wp[NB];
  bool wok[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int j = nb * 16 + lrow;
    const int64_t idx = base + j;
    bool ok = (j < r) && idx >= 0 && idx < pool.a_loc_len;
    int64_t row = ok ? pool.a_loc[idx] : 0;
    ok = ok && row >= 0 && row < pool.w_rows;
    wok[nb] = ok;
    wp[nb] = pool.w + (ok ? row : 0) * h_in;
  }

  f32x4 acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // The trip count must be wave-uniform: MFMA ignores EXEC, so a lane that left the loop early
  // would still feed its stale registers into the matrix core.  Lanes past the end load zeros.
  // (Whole 128-byte lines per wave and step -- 64 K elements, two loads per lane -- measured the same to
  // slightly slower than these half lines.)
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
}

}  // namespace mlora
