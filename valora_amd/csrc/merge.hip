// Merging one adapter into the base weights and taking it out again, for gfx950:
//
//     W_slot[i, o] = T( W_slot[i, o] +- T( sum_{j<r} A[i, j] * T(B[j, o] * scaling) ) )
//
// for the slots (q, k, v, o) of one layer.  This is the reference's merge_adapter / unmerge_adapter
// (valora/models/peft/lora_single_batch_infer.py:103-149): `b = B * scaling` is a T tensor there,
// `ab = bmm(a, b)` is a T tensor (fp32 accumulation inside the GEMM), and `add_` / `sub_` round once
// more; the three rounding points are kept.  The reference first copies the adapter out of the pool
// into dense [H, r] / [r, H] matrices (:81-98), runs the batched GEMM into a [4, H, H] temporary
// and then updates the four weights; here the pool rows are read in place and W is read and
// written exactly once, so the traffic is 2 * H_in * H_out * sizeof(T) per slot.
//
// Layouts: W is [H_in, H_out] row-major (the transposed weight the reference keeps, x @ W).
// B of a slot is [H_out, r] flat over r pool rows -- K-contiguous for the MFMA, loaded straight
// into registers as in the expand.  A of a slot is r pool rows of H_in elements, i.e. [r, H_in]:
// the MFMA wants 8 consecutive rank elements of ONE input row per lane, so the workgroup's
// [r x tile height] slice of A goes through LDS and is read back transposed with 2-byte reads (the row
// stride of tile height + 4 elements spreads the four rank groups of a wave over different banks).
#include "kernel_common.h"

namespace mlora {

namespace {

constexpr int MG_BN = 256;        // output columns per workgroup, 64 per wave
// input rows (of W) per workgroup: taller tiles re-read B less often, but the transposed LDS reads of the
// A slice grow with the rank -- 256 rows measured faster up to rank 32, 128 rows above
constexpr int merge_bm(int kb) { return kb == 1 ? 256 : 128; }
constexpr int MG_STAGE_LD = 64 + 4;

struct MergeArgs {
  uint16_t *w[MLORA_MAX_TARGETS];
  int slots[MLORA_MAX_TARGETS];
  int64_t ld;                 // elements between rows of W
  PoolDev pa, pb;
  const int64_t *a_start, *a_len;
  int adapter, n_slots_pool;
  int h_in, h_out;
  float scaling, sign;
  int n_ochunks;
};

template <typename T, int KB>
__global__ __launch_bounds__(256) void merge_kernel(MergeArgs p) {
  using Tr = Traits<T>;
  using vec8 = typename Tr::vec8;
  constexpr int MG_BM = merge_bm(KB);
  constexpr int MG_RS = MG_BM + 4;   // LDS row stride of the A slice, elements (see the file header)
  __shared__ __align__(16) uint16_t s_a[KB * 32][MG_RS];
  __shared__ float stage[4][16][MG_STAGE_LD];

  const int z = blockIdx.y;
  const int slot = p.slots[z];
  uint16_t *__restrict__ W = p.w[z];
  const int itile = blockIdx.x / p.n_ochunks;
  const int oc = blockIdx.x - itile * p.n_ochunks;
  const int i0 = itile * MG_BM;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lrow = lane & 15, kg = lane >> 4;
  const int o_wave = oc * MG_BN + wave * 64;

  const int64_t alen = p.a_len[p.adapter];
  const int r = (int)(alen / p.n_slots_pool);
  if (r <= 0 || (r & 7) || r > KB * 32) return;      // same adapters the LoRA op accepts
  const int64_t base = p.a_start[p.adapter] + (int64_t)r * slot;

  // ---- B fragments, scaled and rounded to T: bfrag[nb][kb] = T(B^T[o][j0..j0+8) * scaling)
  u32x4 bfrag[4][KB];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int o = o_wave + nb * 16 + lrow;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int j0 = kb * 32 + kg * 8;
      u32x4 b = {0, 0, 0, 0};
      if (o < p.h_out && j0 < r) {
        const uint32_t flat = (uint32_t)o * (uint32_t)r + (uint32_t)j0;
        const uint32_t bin = flat / (uint32_t)p.h_out;
        const uint32_t off = flat - bin * (uint32_t)p.h_out;
        const int64_t idx = base + bin;
        if (idx >= 0 && idx < p.pb.a_loc_len) {
          const int64_t row = p.pb.a_loc[idx];
          if (row >= 0 && row < p.pb.w_rows) b = load16(p.pb.w + row * p.h_out + off);
        }
      }
      float f[8];
      unpack8<T>(b, f);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // the reference's `B * scaling` is an fp32 product rounded to T afterwards: keep the two roundings
        // apart (a fused multiply-and-convert rounds once and differs whenever the fp32 product lands on a
        // tie of T, which decimal scalings such as 1.7 or 0.9 do for a few percent of the elements)
        f[e] *= p.scaling;
        asm volatile("" : "+v"(f[e]));
      }
      bfrag[nb][kb] = pack8<T>(f);
    }
  }

  // ---- the [r x MG_BM] slice of A into LDS (rank rows beyond r are zero)
  for (int idx = tid; idx < KB * 32 * (MG_BM / 8); idx += 256) {
    const int j = idx / (MG_BM / 8), c = idx - j * (MG_BM / 8);
    const int i = i0 + c * 8;
    u32x4 a = {0, 0, 0, 0};
    if (j < r && i < p.h_in) {
      const int64_t ai = base + j;
      if (ai >= 0 && ai < p.pa.a_loc_len) {
        const int64_t row = p.pa.a_loc[ai];
        if (row >= 0 && row < p.pa.w_rows) a = load16(p.pa.w + row * p.h_in + i);
      }
    }
    uint2 *dst = reinterpret_cast<uint2 *>(&s_a[j][c * 8]);   // rows are 8-byte, not 16-byte, aligned
    dst[0] = uint2{a[0], a[1]};
    dst[1] = uint2{a[2], a[3]};
  }
  __syncthreads();

  const int rr0 = lane >> 3, c8 = (lane & 7) * 8;
  const bool ocol_ok = (o_wave + c8) < p.h_out;

  for (int rb0 = 0; rb0 < MG_BM / 16; rb0 += 2) {
    u32x4 wv[2][2];
    uint16_t *wp[2][2];
    bool wok[2][2];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int i = i0 + (rb0 + b) * 16 + rr0 + 8 * h;
        wok[b][h] = ocol_ok && i < p.h_in;
        wp[b][h] = W + (int64_t)(wok[b][h] ? i : 0) * p.ld + o_wave + c8;
        wv[b][h] = wok[b][h] ? load16(wp[b][h]) : u32x4{0, 0, 0, 0};
      }
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      // A^T fragment: row = input row (lrow), 8 consecutive rank elements, read transposed from LDS
      u32x4 afrag[KB];
      const int il = (rb0 + b) * 16 + lrow;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int j0 = kb * 32 + kg * 8;
        uint32_t e[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) e[k] = s_a[j0 + k][il];
        afrag[kb] = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
      }
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
          if (kb * 32 < r) acc = Tr::mfma(as<vec8>(afrag[kb]), as<vec8>(bfrag[nb][kb]), acc);
#pragma unroll
        for (int t = 0; t < 4; ++t) stage[wave][kg * 4 + t][nb * 16 + lrow] = acc[t];
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if (wok[b][h]) {
          const float *srow = &stage[wave][rr0 + 8 * h][c8];
          float f[8];
          unpack8<T>(wv[b][h], f);
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            const float ab = Tr::to_float(Tr::from_float(srow[k]));   // the GEMM result is a T tensor
            f[k] += p.sign * ab;
          }
          store16(wp[b][h], pack8<T>(f));
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }
}

template <typename T>
int launch_merge_t(hipStream_t st, const MergeArgs &a, int kb, dim3 grid) {
  switch (kb) {
    case 1: hipLaunchKernelGGL((merge_kernel<T, 1>), grid, dim3(256), 0, st, a); break;
    case 2: hipLaunchKernelGGL((merge_kernel<T, 2>), grid, dim3(256), 0, st, a); break;
    case 4: hipLaunchKernelGGL((merge_kernel<T, 4>), grid, dim3(256), 0, st, a); break;
    default: return fail(MLORA_ERR_NO_KERNEL, "merge: no kernel for %d rank blocks", kb);
  }
  return check_launch("merge_kernel");
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

}  // namespace mlora

using namespace mlora;

extern "C" int mlora_merge_adapter(void *stream, void *const *w, const int32_t *slots, int32_t n_targets, int64_t ld,
                                   int64_t h_in, int64_t h_out, const mlora_pool *pool_a, const mlora_pool *pool_b,
                                   int64_t adapter, int64_t max_rank, float scaling, int32_t sign, mlora_dtype dtype) {
  if (dtype != MLORA_F16 && dtype != MLORA_BF16)
    return fail(MLORA_ERR_NO_KERNEL, "No suitable kernel. h_in=%lld h_out=%lld dtype=%d", (long long)h_in,
                (long long)h_out, (int)dtype);
  if (!pool_a || !pool_b || !w || !slots) return fail(MLORA_ERR_INVALID, "merge_adapter: null pointer");
  if (n_targets < 1 || n_targets > MLORA_MAX_TARGETS)
    return fail(MLORA_ERR_INVALID, "merge_adapter: n_targets=%d outside [1,%d]", n_targets, MLORA_MAX_TARGETS);
  if (h_in <= 0 || h_out <= 0 || h_in >= 65536 || h_out >= 65536 || (h_in % 8) || (h_out % 8) || ld < h_out || (ld % 8))
    return fail(MLORA_ERR_NO_KERNEL, "No suitable kernel. h_in=%lld h_out=%lld ld=%lld", (long long)h_in,
                (long long)h_out, (long long)ld);
  if (max_rank <= 0 || max_rank > MAX_RANK || (max_rank % 8))
    return fail(MLORA_ERR_NO_KERNEL, "merge_adapter: max_rank=%lld not a multiple of 8 in (0,%d]", (long long)max_rank,
                MAX_RANK);
  if (adapter < 0 || adapter >= pool_a->n_adapters || pool_a->n_adapters != pool_b->n_adapters)
    return fail(MLORA_ERR_INVALID, "merge_adapter: adapter %lld outside [0,%lld)", (long long)adapter,
                (long long)pool_a->n_adapters);
  if (sign != 1 && sign != -1) return fail(MLORA_ERR_INVALID, "merge_adapter: sign must be +1 or -1");
  if (!pool_a->w || !pool_b->w || !pool_a->a_start || !pool_a->a_len || !pool_a->a_loc || !aligned16(pool_a->w) ||
      !aligned16(pool_b->w))
    return fail(MLORA_ERR_INVALID, "merge_adapter: pool tensors are null or misaligned");
  MergeArgs a;
  for (int i = 0; i < MLORA_MAX_TARGETS; ++i) {
    const int k = i < n_targets ? i : 0;
    if (!w[k] || !aligned16(w[k])) return fail(MLORA_ERR_INVALID, "merge_adapter: weight %d is null or misaligned", k);
    if (slots[k] < 0 || slots[k] >= pool_a->n_slots)
      return fail(MLORA_ERR_INVALID, "merge_adapter: slot %d outside [0,%d)", slots[k], pool_a->n_slots);
    a.w[i] = static_cast<uint16_t *>(w[k]);
    a.slots[i] = slots[k];
  }
  a.ld = ld;
  a.pa = PoolDev{static_cast<const uint16_t *>(pool_a->w), pool_a->w_rows, pool_a->a_loc, pool_a->a_loc_len};
  a.pb = PoolDev{static_cast<const uint16_t *>(pool_b->w), pool_b->w_rows, pool_b->a_loc, pool_b->a_loc_len};
  a.a_start = pool_a->a_start;
  a.a_len = pool_a->a_len;
  a.adapter = (int)adapter;
  a.n_slots_pool = pool_a->n_slots;
  a.h_in = (int)h_in;
  a.h_out = (int)h_out;
  a.scaling = scaling;
  a.sign = (float)sign;
  a.n_ochunks = (int)((h_out + MG_BN - 1) / MG_BN);
  int kb = (int)((max_rank + 31) / 32);
  kb = kb <= 1 ? 1 : kb <= 2 ? 2 : 4;
  const int bm = merge_bm(kb);
  const int64_t blocks = ((h_in + bm - 1) / bm) * a.n_ochunks;
  dim3 grid((unsigned)blocks, (unsigned)n_targets);
  return dtype == MLORA_F16 ? launch_merge_t<_Float16>((hipStream_t)stream, a, kb, grid)
                            : launch_merge_t<__bf16>((hipStream_t)stream, a, kb, grid);
}
