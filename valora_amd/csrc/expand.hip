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
// v comes from the shrink's split-K partials (summed in a fixed order and rounded to T once, as
// the reference does by holding `delta` in a T tensor between its two launches) or from a T
// matrix supplied by the caller.
//
// Reference semantics: valora/csrc/bgmv/bgmv_impl.cuh:152-207.
#include "kernel_common.h"

namespace mlora {

namespace {

constexpr int EXP_BN = 256;       // outputs per workgroup
constexpr int EXP_WN = 64;        // outputs per wave
constexpr int STAGE_LD = EXP_WN + 4;

template <typename T, int KB>
__global__ __launch_bounds__(256) void expand_kernel(ExpandArgs p) {
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  __shared__ float stage[4][16][STAGE_LD];

  const int32_t *__restrict__ hdr = p.plan;
  const int tile_idx = blockIdx.x / p.n_ochunks;
  const int oc = blockIdx.x - tile_idx * p.n_ochunks;
  if (tile_idx >= hdr[H_NTILES_E]) return;
  const int32_t *__restrict__ tile = p.plan + p.off_tiles + (int64_t)tile_idx * TILE_WORDS;
  const int a = tile[0], r = tile[1], pos0 = tile[2], cnt = tile[3], astart = tile[4];
  const int rk = min(r, p.kmax);  // rank columns the narrow operand really has (bgmv_impl.cuh:167,186)

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, kg = lane >> 4;
  const int32_t *__restrict__ perm = p.plan + p.off_perm;
  const int64_t base = (int64_t)astart + (int64_t)r * p.slot;
  const float scale = Tr::to_float(p.scales[a]);
  const int o_wave = oc * EXP_BN + wave * EXP_WN;

  // B fragments: bfrag[nb][kb] = B^T[o = o_wave + nb*16 + lrow][j0 .. j0+8), j0 = kb*32 + kg*8
  u32x4 bfrag[4][KB];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int o = o_wave + nb * 16 + lrow;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int j0 = kb * 32 + kg * 8;
      u32x4 v = {0, 0, 0, 0};
      if (o < p.h_out && j0 < rk) {
        const uint32_t flat = (uint32_t)o * (uint32_t)r + (uint32_t)j0;   // < 2^16 * 2^7
        const uint32_t bin = flat / (uint32_t)p.h_out;
        const uint32_t off = flat - bin * (uint32_t)p.h_out;
        const int64_t idx = base + bin;
        if (idx >= 0 && idx < p.pool.a_loc_len) {
          const int64_t row = p.pool.a_loc[idx];
          if (row >= 0 && row < p.pool.w_rows) v = load16(p.pool.w + row * p.h_out + off);
        }
      }
      bfrag[nb][kb] = v;
    }
  }

  // row-major roles for the y read-modify-write: 8 lanes x 16 B cover one token row of the wave's
  // 64 outputs; a wave covers 8 rows per access, two accesses per 16-token block.
  const int rr0 = lane >> 3, c8 = (lane & 7) * 8;
  const bool ocol_ok = (o_wave + c8) < p.h_out;

  const int n_mb = (cnt + 15) >> 4;
  for (int mb = 0; mb < n_mb; ++mb) {
    // ---- v fragments: rows = tokens (lrow), 8 consecutive rank elements per lane
    const int prow = mb * 16 + lrow;
    const bool pok = prow < cnt;
    u32x4 vfrag[KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int j0 = kb * 32 + kg * 8;
      u32x4 v = {0, 0, 0, 0};
      if (pok && j0 < rk) {
        if (p.partial != nullptr) {
          float f[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          for (int s = 0; s < p.ksplit; ++s) {
            const f32x4 *src = reinterpret_cast<const f32x4 *>(
                p.partial + ((int64_t)s * p.T + pos0 + prow) * p.rp + j0);
            const f32x4 lo = src[0], hi = src[1];
#pragma unroll
            for (int i = 0; i < 4; ++i) { f[i] += lo[i]; f[4 + i] += hi[i]; }
          }
          v = pack8<T>(f);
        } else {
          const int t = perm[pos0 + prow];
          v = load16(p.xv + (int64_t)t * p.v_stride + j0);
        }
      }
      vfrag[kb] = v;
    }
    // ---- y rows (issued before the MFMAs so the loads overlap them)
    u32x4 yv[2];
    uint16_t *yp[2];
    bool yok[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int row = mb * 16 + rr0 + 8 * h;
      yok[h] = ocol_ok && row < cnt;
      const int t = yok[h] ? perm[pos0 + row] : 0;
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
    __syncthreads();
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
    __syncthreads();
  }
}

template <typename T>
int launch_expand_t(hipStream_t st, const ExpandArgs &a, int kb, dim3 grid) {
  switch (kb) {
    case 1: hipLaunchKernelGGL((expand_kernel<T, 1>), grid, dim3(256), 0, st, a); break;
    case 2: hipLaunchKernelGGL((expand_kernel<T, 2>), grid, dim3(256), 0, st, a); break;
    case 4: hipLaunchKernelGGL((expand_kernel<T, 4>), grid, dim3(256), 0, st, a); break;
    default: return fail(MLORA_ERR_NO_KERNEL, "expand: no kernel for %d rank blocks", kb);
  }
  return check_launch("expand_kernel");
}

}  // namespace

int launch_expand(hipStream_t st, const ExpandArgs &a, int max_rank, int64_t grid_tiles, mlora_dtype dt) {
  int kb = (max_rank + 31) / 32;
  kb = kb <= 1 ? 1 : kb <= 2 ? 2 : 4;
  if (grid_tiles <= 0) return MLORA_OK;
  const int64_t blocks = grid_tiles * a.n_ochunks;
  if (blocks > 0x7fffffff) return fail(MLORA_ERR_NO_KERNEL, "expand: grid too large");
  dim3 grid((unsigned)blocks);
  return dt == MLORA_F16 ? launch_expand_t<_Float16>(st, a, kb, grid)
                         : launch_expand_t<__bf16>(st, a, kb, grid);
}

int expand_bn() { return EXP_BN; }

}  // namespace mlora
