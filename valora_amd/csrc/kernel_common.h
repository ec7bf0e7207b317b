// Device-side helpers shared by the gfx950 LoRA kernels: 16-byte vector access and the
// per-dtype MFMA / conversion traits.  (The reference's counterpart is the 1300-line
// vec_dtypes.cuh, valora/csrc/bgmv/vec_dtypes.cuh:16-30,754-800; only fp16 and bf16 exist here.)
#pragma once

#include "mlora_internal.h"

namespace mlora {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

template <typename To, typename From>
__device__ __forceinline__ To as(const From &v) {
  static_assert(sizeof(To) == sizeof(From), "size mismatch");
  return __builtin_bit_cast(To, v);
}

// One global_load_dwordx4 / global_store_dwordx4.  Addresses must be 16-byte aligned.
__device__ __forceinline__ u32x4 load16(const uint16_t *p) { return *reinterpret_cast<const u32x4 *>(p); }
__device__ __forceinline__ void store16(uint16_t *p, u32x4 v) { *reinterpret_cast<u32x4 *>(p) = v; }

// Direct global -> LDS load: each active lane copies 16 bytes from its own global address to
// lds_base + lane*16 (lds_base is wave-uniform); completion is tracked by vmcnt.
#define GLOBAL_PTR(p) (reinterpret_cast<const __attribute__((address_space(1))) void *>(reinterpret_cast<uintptr_t>(p)))
// A pointer that went through an inline asm operand has lost what the compiler knew about it; telling it again that
// the memory is global keeps its loads and stores on the global path (flat accesses count against two wait counters)
template <typename P>
__device__ __forceinline__ P *as_global(P *p) {
  typedef __attribute__((address_space(1))) P *GP;
  return (P *)(GP)(uintptr_t)p;
}
#define LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

// wait until at most N vector-memory loads of this wave are outstanding (loads retire in order)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void wait_lgkmcnt0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

// LDS accesses the compiler does not see as LDS accesses.  Around direct-to-LDS loads the
// compiler's own wait insertion is conservative (it drains ALL outstanding loads before any LDS
// access that might alias their destination), which would serialise a multi-stage ring; with
// these the kernel orders things itself: wait_vmcnt<N>() before reading a stage,
// wait_lgkmcnt0() + pin() before using what lds_read16 returned.
__device__ __forceinline__ uint32_t lds_offset(const void *p) {
  return (uint32_t)(uintptr_t)LDS_PTR(const_cast<void *>(p));
}
__device__ __forceinline__ u32x4 lds_read16(uint32_t off) {
  u32x4 v;
  asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(off) : "memory");
  return v;
}
__device__ __forceinline__ void lds_write16(uint32_t off, u32x4 v) {
  asm volatile("ds_write_b128 %0, %1" ::"v"(off), "v"(v) : "memory");
}
// makes v "produced here" for the compiler, so nothing that uses it moves above a preceding wait
__device__ __forceinline__ void pin(u32x4 &v) { asm volatile("" : "+v"(v)); }

// q = n / d and rem = n % d for n < 2^24 (exact in fp32) from a reciprocal computed once: the float estimate of
// the quotient is off by at most one.  An integer division by a run-time divisor costs some 35 vector
// instructions, and the kernels' address set-up does several per lane before the first load can be issued.
__device__ __forceinline__ void divmod24(uint32_t n, uint32_t d, float inv_d, uint32_t &q, uint32_t &rem) {
  q = (uint32_t)((float)n * inv_d);
  int32_t m = (int32_t)(n - q * d);
  if (m < 0) {
    q -= 1u;
    m += (int32_t)d;
  } else if (m >= (int32_t)d) {
    q += 1u;
    m -= (int32_t)d;
  }
  rem = (uint32_t)m;
}

// Walks the B operand of the expand.  A slot's B block is r pool rows that, concatenated, hold [h_out, r]
// row-major: the 8 rank elements [j0, j0 + 8) of output column o start at flat offset o*r + j0, i.e. in the
// slot's pool row number `bin` at element `off`.  Outputs 16 apart are 16*r elements apart, so after one
// division the cursor moves on with an add and a compare.
struct BCursor {
  uint32_t bin, off;
};
__device__ __forceinline__ BCursor b_cursor(uint32_t o, uint32_t r, uint32_t j0, uint32_t h_out, float inv_h_out) {
  BCursor c;
  divmod24(o * r + j0, h_out, inv_h_out, c.bin, c.off);   // o < 2^16, r <= 2^7
  return c;
}
// `step` elements further on; step < h_out
__device__ __forceinline__ void b_advance(BCursor &c, uint32_t step, uint32_t h_out) {
  c.off += step;
  if (c.off >= h_out) {
    c.off -= h_out;
    c.bin += 1u;
  }
}

template <typename T>
struct Traits;

template <>
struct Traits<_Float16> {
  using vec8 = f16x8;
  static __device__ __forceinline__ f32x4 mfma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_float(uint16_t h) { return (float)as<_Float16>(h); }
  static __device__ __forceinline__ uint16_t from_float(float f) { return as<uint16_t>((_Float16)f); }
};

template <>
struct Traits<__bf16> {
  using vec8 = bf16x8;
  static __device__ __forceinline__ f32x4 mfma(vec8 a, vec8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_float(uint16_t h) { return as<float>((uint32_t)h << 16); }
  // round to nearest even; NaN stays NaN
  static __device__ __forceinline__ uint16_t from_float(float f) {
    uint32_t x = as<uint32_t>(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
  }
};

// which of the device's XCDs this wave runs on (bits 3:0 of the XCC_ID hardware register)
__device__ __forceinline__ uint32_t xcd_id() { return (uint32_t)__builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20); }

// 8 packed T values <-> 8 floats
template <typename T>
__device__ __forceinline__ void unpack8(u32x4 v, float (&f)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = Traits<T>::to_float((uint16_t)(v[i] & 0xffffu));
    f[2 * i + 1] = Traits<T>::to_float((uint16_t)(v[i] >> 16));
  }
}

template <typename T>
__device__ __forceinline__ u32x4 pack8(const float (&f)[8]) {
  u32x4 v;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    v[i] = (uint32_t)Traits<T>::from_float(f[2 * i]) | ((uint32_t)Traits<T>::from_float(f[2 * i + 1]) << 16);
  return v;
}

}  // namespace mlora
