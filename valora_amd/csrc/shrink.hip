// LoRA shrink for gfx950:  partial[s][p][j] = sum_{k in K-chunk s} x[perm[p], k] * A_a[j, k]
//
// One workgroup (4 waves) owns one adapter-grouped tile of up to 16*MB tokens and one K-chunk.
// Both operands are K-contiguous in memory (token rows of x, rank rows of the pool), which is
// exactly the per-lane layout v_mfma_f32_16x16x32 wants: lane (row = lane%16, kgroup = lane/16)
// holds 8 consecutive K elements, so every operand is a single 16-byte global load straight
// into the MFMA source registers -- no LDS staging, no transposes.  The four waves interleave
// 32-element K-steps, so the workgroup reads 256 contiguous bytes of every row per round.
// fp32 accumulators are reduced across the waves through LDS and written as split-K partials;
// the consumer (expand or shrink_finish) sums the `ksplit` partials in a fixed order, which
// keeps the result deterministic without atomics or zero-initialisation.
//
// Reference semantics: valora/csrc/bgmv/bgmv_impl.cuh:14-148 (per-token gather mat-vec with the
// rank rows gathered through loc_indicies, fp32 accumulation).
#include "kernel_common.h"

namespace mlora {

namespace {

template <typename T, int MB, int NB>
__global__ __launch_bounds__(256) void shrink_kernel(ShrinkArgs p) {
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  constexpr int NBLK = MB * NB;
  __shared__ float red[2][NBLK * 256];

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
  // U K-steps are loaded before any is consumed: the kernel is bound by memory latency, so what
  // matters is how many 16-byte loads each lane has in flight (U * (MB + NB)).
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
    const float *src = red[0];
    float *__restrict__ out = p.partial + ((int64_t)s * p.T + pos0) * p.rp;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int b = mb * NB + nb;
          const float v = acc[mb][nb][i] + src[(b * 4 + i) * 64 + lane];
          const int row = mb * 16 + kg * 4 + i;  // C layout: column = lane%16, rows = 4*(lane/16)+i
          const int col = nb * 16 + lrow;
          if (row < cnt && col < p.rp) out[(int64_t)row * p.rp + col] = v;
        }
  }
}

// y[perm[p], j] (<- | +=) T(sum_s partial[s][p][j])
template <typename T>
__global__ __launch_bounds__(256) void shrink_finish_kernel(FinishArgs p) {
  using Tr = Traits<T>;
  const int n_active = p.plan[H_NACTIVE];
  const int cols = p.mode == MLORA_SHRINK_ZERO_PAD ? max(p.width, 0) : p.rp;
  const int64_t total = (int64_t)n_active * cols;
  for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total;
       e += (int64_t)gridDim.x * blockDim.x) {
    const int pos = (int)(e / cols), j = (int)(e % cols);
    const int t = p.plan[p.off_perm + pos];
    const int r = p.plan[p.off_prank + pos];
    uint16_t *dst = p.y + (int64_t)t * p.y_stride + j;
    if (j < r && j < p.ncols) {
      float v = 0.f;
      for (int s = 0; s < p.ksplit; ++s) v += p.partial[((int64_t)s * p.T + pos) * p.rp + j];
      if (p.mode == MLORA_SHRINK_ACCUMULATE) v += Tr::to_float(*dst);
      *dst = Tr::from_float(v);
    } else if (p.mode == MLORA_SHRINK_ZERO_PAD) {
      *dst = 0;
    }
  }
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
    default: return fail(MLORA_ERR_NO_KERNEL, "shrink: tile height %d not in {16,32,64}", bm);
  }
}

}  // namespace

int launch_shrink(hipStream_t st, const ShrinkArgs &a, int bm, int max_rank, int64_t grid_tiles,
                  mlora_dtype dt) {
  int nb = (max_rank + 15) / 16;
  nb = nb <= 1 ? 1 : nb <= 2 ? 2 : nb <= 4 ? 4 : 8;
  if (nb == 8 && bm > 32) return fail(MLORA_ERR_NO_KERNEL, "shrink: rank > 64 needs tile height <= 32");
  if (grid_tiles <= 0) return MLORA_OK;
  dim3 grid((unsigned)grid_tiles, (unsigned)a.ksplit);
  return dt == MLORA_F16 ? launch_shrink_t<_Float16>(st, a, bm, nb, grid)
                         : launch_shrink_t<__bf16>(st, a, bm, nb, grid);
}

int launch_finish(hipStream_t st, const FinishArgs &a, mlora_dtype dt) {
  if (a.T <= 0) return MLORA_OK;
  const int cols = a.mode == MLORA_SHRINK_ZERO_PAD ? (a.width > 0 ? a.width : 1) : a.rp;
  int64_t blocks = ((int64_t)a.T * cols + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (blocks < 1) blocks = 1;
  if (dt == MLORA_F16)
    hipLaunchKernelGGL(shrink_finish_kernel<_Float16>, dim3((unsigned)blocks), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL(shrink_finish_kernel<__bf16>, dim3((unsigned)blocks), dim3(256), 0, st, a);
  return check_launch("shrink_finish_kernel");
}

}  // namespace mlora
