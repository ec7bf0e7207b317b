/* CPU restatement of the reference BGMV kernels, written index-for-index from the CUDA text.
 * TEST INFRASTRUCTURE ONLY: nothing in the shipped package links or loads this file.
 *
 * It exists to pin oracle/lora_oracle.py: that module formulates the op through dense
 * reshapes ([r,H].T and [H,r].T), this file walks the flat offsets exactly like the kernels
 * (valora/csrc/bgmv/bgmv_impl.cuh), so a transposed operand or a wrong flat index in either
 * one makes the two disagree.
 *
 *   shrink : valora/csrc/bgmv/bgmv_impl.cuh:14-148
 *   expand : valora/csrc/bgmv/bgmv_impl.cuh:152-207
 *
 * dtype: 0 = IEEE fp16, 1 = bfloat16.  Accumulation is fp32 like the kernels'.
 */
#include <stdint.h>
#include <string.h>

static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; e++; } while ((man & 0x400u) == 0);
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t float_to_half(float f) { /* round to nearest even */
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | ((absx > 0x7f800000u) ? 0x200u : 0));
  if (absx >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* overflow after rounding */
  if (absx < 0x33000001u) return (uint16_t)sign;               /* rounds to zero */
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t m = (absx & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t hexp;
  if (e < -14) { shift = 13 + (-14 - e); hexp = 0; } else { shift = 13; hexp = (uint32_t)(e + 15); }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) q++;
  uint32_t out;
  if (hexp == 0) out = q;                       /* subnormal (q may carry into exp = 1) */
  else out = ((hexp - 1) << 10) + q;            /* q includes the hidden bit (0x400) */
  return (uint16_t)(sign | out);
}

static float bf16_to_float(uint16_t h) {
  uint32_t bits = (uint32_t)h << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static uint16_t float_to_bf16(float f) { /* round to nearest even */
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

static float ld(const uint16_t *p, int dtype) { return dtype ? bf16_to_float(*p) : half_to_float(*p); }
static uint16_t st(float f, int dtype) { return dtype ? float_to_bf16(f) : float_to_half(f); }

/* conversions exported so the tests can pin them against torch's */
float bgmv_ref_to_float(uint16_t h, int dtype) { return ld(&h, dtype); }
uint16_t bgmv_ref_from_float(float f, int dtype) { return st(f, dtype); }

/* Y[T, feat_out] (feat_out = scratch width R), X[T, feat_in], W rows of feat_in elements. */
int bgmv_ref_shrink(uint16_t *Y, const uint16_t *X, const uint16_t *W, const int64_t *start_indicies,
                    const int64_t *lora_ranks, const int64_t *loc_indicies, const int64_t *indicies,
                    int64_t qkvo, int64_t batch, int64_t feat_in, int64_t feat_out, int dtype) {
  for (int64_t b = 0; b < batch; ++b) {
    int64_t lora_idx = indicies[b];
    int64_t lora_rank = lora_ranks[lora_idx] / 4;               /* :35 */
    for (int64_t j = 0; j < feat_out; ++j) {                    /* grid.x = feat_out, :232 */
      if (j >= lora_rank) continue;                             /* :36 */
      int64_t mem_pos = start_indicies[lora_idx] + lora_rank * qkvo; /* :37 */
      int64_t idx = loc_indicies[mem_pos + j];                  /* :38 */
      float y = 0.f;
      for (int64_t k = 0; k < feat_in; ++k)                     /* W + idx*feat_in + k, :48 */
        y += ld(W + idx * feat_in + k, dtype) * ld(X + b * feat_in + k, dtype);
      Y[b * feat_out + j] = st(y, dtype);                       /* :147 */
    }
  }
  return 0;
}

/* Y[T, feat_out], X[T, feat_in] (feat_in = scratch width R), W rows of feat_out elements. */
int bgmv_ref_expand(uint16_t *Y, const uint16_t *X, const uint16_t *W, const int64_t *start_indicies,
                    const int64_t *lora_ranks, const int64_t *loc_indicies, const int64_t *indicies,
                    int64_t qkvo, const uint16_t *lora_scales, int64_t batch, int64_t feat_in,
                    int64_t feat_out, int dtype) {
  const int64_t vec = 8;                                        /* 16 B / sizeof(T), :166 */
  const int64_t tx_n = feat_in / vec;                           /* :167 */
  for (int64_t b = 0; b < batch; ++b) {
    int64_t lora_idx = indicies[b];
    int64_t lora_rank = lora_ranks[lora_idx] / 4;               /* :165 */
    int64_t start_idx = start_indicies[lora_idx];
    float scale = ld(lora_scales + lora_idx, dtype);            /* :180 */
    for (int64_t o = 0; o < feat_out; ++o) {                    /* o = tile*tz*ty + z*ty + y, :206 */
      float sum = 0.f;
      for (int64_t tx = 0; tx < tx_n; ++tx) {
        if (tx * vec >= lora_rank) continue;                    /* zero fill, :186-188 */
        int64_t flat = o * lora_rank + tx * vec;                /* :174-177 */
        int64_t bin = flat / feat_out;
        int64_t bin_offset = flat % feat_out;
        int64_t w_outer = loc_indicies[start_idx + lora_rank * qkvo + bin]; /* :178 */
        for (int64_t i = 0; i < vec; ++i)                       /* :196-198 */
          sum += ld(W + w_outer * feat_out + bin_offset + i, dtype) *
                 ld(X + b * feat_in + tx * vec + i, dtype) * scale;
      }
      float yv = ld(Y + b * feat_out + o, dtype) + sum;         /* Y += sum, :205-207 */
      Y[b * feat_out + o] = st(yv, dtype);
    }
  }
  return 0;
}
