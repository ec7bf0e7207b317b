// Fused LoRA shrink + expand in ONE launch for decode-like batches (few tokens per adapter).
//
//   y[t, o] = T( y[t, o] + scale_a * sum_j T(v[t, j]) * B_a[j, o] ),   v[t, j] = sum_k x[t, k] * A_a[j, k]
//
// A workgroup of 16 waves owns one adapter-grouped tile of up to 16 tokens and one slice of the
// output columns.  It first computes the tile's complete v (the 16 waves split K and reduce
// through LDS), rounds it to T exactly where the reference stores its `delta` tensor, and then
// expands it over its own output slice.  The `replicas` workgroups that share a tile all
// recompute the same v: the A rows and x rows they re-read come out of L2 (replicas of a tile
// are placed on the same XCD), so HBM still sees every byte once, and in exchange there is no
// second launch, no split-K buffer and no dependency between workgroups.  Everything a
// workgroup needs from HBM -- x rows, A rows, the first B fragments and y rows -- is requested
// before anything is consumed: the op is bound by memory latency, not by arithmetic.
//
// Reference semantics: valora/csrc/bgmv/bgmv_impl.cuh:14-148 (shrink) and :152-207 (expand).
#include "kernel_common.h"

namespace mlora {

namespace {

constexpr int FW = 16;                 // waves per workgroup
constexpr int FT = FW * 64;            // threads per workgroup
constexpr int F_WN = 64;               // outputs per wave per pass
constexpr int F_BN = FW * F_WN;        // outputs per workgroup per pass (1024)
constexpr int F_STAGE_LD = F_WN + 4;

template <typename T, int NB>
__global__ __launch_bounds__(FT) void fused_kernel(FusedArgs p) {
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  constexpr int KB = (NB + 1) / 2;                 // 32-wide rank blocks of the expand
  constexpr int RP = NB * 16;                      // padded rank
  constexpr int U = NB == 1 ? 8 : NB == 2 ? 4 : 2; // K-steps loaded per batch
  // LDS: the cross-wave reduction buffer (8 slots) is reused as the expand's staging area
  constexpr int RED_FLOATS = 8 * NB * 256;
  constexpr int STAGE_FLOATS = FW * 16 * F_STAGE_LD;
  __shared__ float s_buf[RED_FLOATS > STAGE_FLOATS ? RED_FLOATS : STAGE_FLOATS];
  __shared__ uint16_t s_v[16][RP + 8];
  __shared__ int32_t s_perm[16];

  const int tile_idx = blockIdx.x % p.tiles_pad;
  const int rep = blockIdx.x / p.tiles_pad;
  if (tile_idx >= p.tiles) return;
  const int32_t *__restrict__ tile = p.plan + p.off_tiles + (int64_t)tile_idx * TILE_WORDS;
  const int a = tile[0], r = tile[1], pos0 = tile[2], cnt = tile[3], astart = tile[4];
  if (cnt <= 0) return;   // records past the last tile are zero
  const int rk = min(r, p.kmax);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, kg = lane >> 4;
  const int64_t base = (int64_t)astart + (int64_t)r * p.slot;
  const int o_begin = rep * p.o_per_wg;
  const int o_end = min(p.h_out, o_begin + p.o_per_wg);

  // ---- round trip 1: token indices, pool rows of A and of the first B fragments, scale
  const int my_t = (lrow < cnt) ? p.plan[p.off_perm + pos0 + lrow] : 0;
  const float scale = Tr::to_float(p.scales[a]);
  int64_t arow[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int j = nb * 16 + lrow;
    const int64_t idx = base + j;
    arow[nb] = (j < rk && idx >= 0 && idx < p.pa.a_loc_len) ? p.pa.a_loc[idx] : -1;
  }
  if (tid < 16) s_perm[tid] = (tid < cnt) ? p.plan[p.off_perm + pos0 + tid] : 0;

  auto b_address = [&](int o, int j0, const uint16_t *&ptr) -> bool {
    if (o >= o_end || j0 >= rk) return false;
    const uint32_t flat = (uint32_t)o * (uint32_t)r + (uint32_t)j0;
    const uint32_t bin = flat / (uint32_t)p.h_out;
    const uint32_t off = flat - bin * (uint32_t)p.h_out;
    const int64_t idx = base + bin;
    if (idx < 0 || idx >= p.pb.a_loc_len) return false;
    const int64_t row = p.pb.a_loc[idx];
    if (row < 0 || row >= p.pb.w_rows) return false;
    ptr = p.pb.w + row * p.h_out + off;
    return true;
  };
  const uint16_t *bptr[4][KB];
  bool bok[4][KB];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
      bok[nb][kb] = b_address(o_begin + wave * F_WN + nb * 16 + lrow, kb * 32 + kg * 8, bptr[nb][kb]);

  // ---- round trip 2: x rows, A rows, first B fragments, first y rows -- all in flight together
  const bool xok = lrow < cnt;
  const uint16_t *xp = p.x + (int64_t)my_t * p.h_in;
  const uint16_t *wp[NB];
  bool wok[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    wok[nb] = arow[nb] >= 0 && arow[nb] < p.pa.w_rows;
    wp[nb] = p.pa.w + (wok[nb] ? arow[nb] : 0) * p.h_in;
  }
  f32x4 acc[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 bfrag[4][KB];
  bool b_loaded = false;
  // wave-uniform trip count (MFMA ignores EXEC); lanes past the end of K feed zeros
  for (int kb0 = wave * 32; kb0 < p.h_in; kb0 += FW * 32 * U) {
    u32x4 xa[U], wb[U][NB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = kb0 + u * FW * 32 + kg * 8;
      const bool kok = k < p.h_in;
      xa[u] = (xok && kok) ? load16(xp + k) : u32x4{0, 0, 0, 0};
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) wb[u][nb] = (wok[nb] && kok) ? load16(wp[nb] + k) : u32x4{0, 0, 0, 0};
    }
    if (!b_loaded) {  // queue the first pass's B fragments behind the first batch of shrink loads
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) bfrag[nb][kb] = bok[nb][kb] ? load16(bptr[nb][kb]) : u32x4{0, 0, 0, 0};
      b_loaded = true;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        if (nb * 16 < rk) acc[nb] = Tr::mfma(as<vec8>(xa[u]), as<vec8>(wb[u][nb]), acc[nb]);
  }
  if (!b_loaded) {
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) bfrag[nb][kb] = bok[nb][kb] ? load16(bptr[nb][kb]) : u32x4{0, 0, 0, 0};
  }

  // ---- reduce the 16 waves' partial v tiles: waves 8..15 -> LDS, waves 0..7 add and store,
  //      then every (row, col) sums its 8 values in slot order and is rounded to T once.
  if (wave >= 8) {
    float *dst = s_buf + (wave - 8) * NB * 256;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[(nb * 4 + i) * 64 + lane] = acc[nb][i];
  }
  __syncthreads();
  if (wave < 8) {
    float *dst = s_buf + wave * NB * 256;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[(nb * 4 + i) * 64 + lane] += acc[nb][i];
  }
  __syncthreads();
  for (int e = tid; e < NB * 256; e += FT) {
    // e = (nb*4 + i)*64 + lane' ; C layout: column = lane'%16, row = 4*(lane'/16) + i
    const int ln = e & 63, bi = e >> 6, nb = bi >> 2, i = bi & 3;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < 8; ++w) v += s_buf[w * NB * 256 + e];
    const int row = (ln >> 4) * 4 + i, col = nb * 16 + (ln & 15);
    s_v[row][col] = Tr::from_float(col < rk ? v : 0.f);
  }
  __syncthreads();  // s_v complete; s_buf free for staging

  // v fragments of the expand: rows = tokens (lrow), 8 consecutive rank elements per lane
  u32x4 vfrag[KB];
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    const int j0 = kb * 32 + kg * 8;
    vfrag[kb] = (j0 < RP) ? *reinterpret_cast<const u32x4 *>(&s_v[lrow][j0]) : u32x4{0, 0, 0, 0};
  }

  float(*stage)[F_STAGE_LD] = reinterpret_cast<float(*)[F_STAGE_LD]>(s_buf + wave * 16 * F_STAGE_LD);
  const int rr0 = lane >> 3, c8 = (lane & 7) * 8;

  for (int o_pass = o_begin; o_pass < o_end; o_pass += F_BN) {
    const int o_wave = o_pass + wave * F_WN;
    if (o_pass != o_begin) {
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
          const uint16_t *ptr = nullptr;
          const bool ok = b_address(o_wave + nb * 16 + lrow, kb * 32 + kg * 8, ptr);
          bfrag[nb][kb] = ok ? load16(ptr) : u32x4{0, 0, 0, 0};
        }
    }
    u32x4 yv[2];
    uint16_t *yp[2];
    bool yok[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int row = rr0 + 8 * h;
      yok[h] = (o_wave + c8) < o_end && row < cnt;
      yp[h] = p.y + (int64_t)s_perm[row] * p.h_out + o_wave + c8;
      yv[h] = yok[h] ? load16(yp[h]) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      f32x4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kb = 0; kb < KB; ++kb)
        if (kb * 32 < rk) d = Tr::mfma(as<vec8>(vfrag[kb]), as<vec8>(bfrag[nb][kb]), d);
#pragma unroll
      for (int i = 0; i < 4; ++i) stage[kg * 4 + i][nb * 16 + lrow] = d[i];
    }
    // stage is private to the wave and a wave's LDS operations execute in order: only the
    // compiler has to be kept from moving the reads below over the writes above
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      if (yok[h]) {
        const float *srow = &stage[rr0 + 8 * h][c8];
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
int launch_fused_t(hipStream_t st, const FusedArgs &a, int nb, dim3 grid) {
  switch (nb) {
    case 1: hipLaunchKernelGGL((fused_kernel<T, 1>), grid, dim3(FT), 0, st, a); break;
    case 2: hipLaunchKernelGGL((fused_kernel<T, 2>), grid, dim3(FT), 0, st, a); break;
    case 4: hipLaunchKernelGGL((fused_kernel<T, 4>), grid, dim3(FT), 0, st, a); break;
    default: return fail(MLORA_ERR_NO_KERNEL, "fused: ranks above 64 use the two-launch path");
  }
  return check_launch("fused_kernel");
}

}  // namespace

int fused_bn() { return F_BN; }

int launch_fused(hipStream_t st, const FusedArgs &a, int max_rank, int replicas, mlora_dtype dt) {
  int nb = (max_rank + 15) / 16;
  nb = nb <= 1 ? 1 : nb <= 2 ? 2 : nb <= 4 ? 4 : 8;
  const int64_t blocks = (int64_t)a.tiles_pad * replicas;
  if (blocks <= 0) return MLORA_OK;
  if (blocks > 0x7fffffff) return fail(MLORA_ERR_NO_KERNEL, "fused: grid too large");
  dim3 grid((unsigned)blocks);
  return dt == MLORA_F16 ? launch_fused_t<_Float16>(st, a, nb, grid) : launch_fused_t<__bf16>(st, a, nb, grid);
}

}  // namespace mlora
