// Device-side arithmetic shared by the W4A16 kernels: nibble -> biased 16-bit element, the correction operand
// that removes bias and zero point inside the MFMA accumulator, and the element-type specific MFMA.
#pragma once

#include "ksq_internal.h"

namespace ksq {
namespace w4 {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct Ops;

template <>
struct Ops<_Float16> {
  // word of eight nibbles -> four registers of two biased fp16 each.  Element 2p sits in nibble p and element
  // 2p + 1 in nibble p + 4; nibbles 0/4 and 2/6 take the 1024 + u form, nibbles 1/5 and 3/7 the 64 + u form.
  static __device__ inline u32x4 unpack(uint32_t x, uint32_t m_lo, uint32_t m_hi, uint32_t c_lo, uint32_t c_hi) {
    const uint32_t y = x >> 8;
    u32x4 v;
    v[0] = (x & m_lo) | c_lo;
    v[1] = (x & m_hi) | c_hi;
    v[2] = (y & m_lo) | c_lo;
    v[3] = (y & m_hi) | c_hi;
    return v;
  }
  static constexpr uint32_t kMaskLo = 0x000F000Fu, kMaskHi = 0x00F000F0u;
  static constexpr uint32_t kMagicLo = 0x64006400u, kMagicHi = 0x54005400u;
  // the same word with every nibble in the 1024 + u form (two more shifts): one bias for all elements, so that
  // sum a * (bias + z) factors into (bias + z) * sum a
  static __device__ inline u32x4 unpack_uniform(uint32_t x, uint32_t m_lo, uint32_t c_lo) {
    u32x4 v;
    v[0] = (x & m_lo) | c_lo;
    v[1] = ((x >> 4) & m_lo) | c_lo;
    v[2] = ((x >> 8) & m_lo) | c_lo;
    v[3] = ((x >> 12) & m_lo) | c_lo;
    return v;
  }
  static constexpr float kBias = 1024.f;
  static constexpr uint32_t kOnes = 0x3C003C00u;
  // -(bias + z) per element for the correction MFMA; zc = z replicated into both halves
  static __device__ inline u32x4 correction(uint32_t zc) {
    const uint32_t lo = 0xE400E400u | zc, hi = 0xD400D400u | (zc << 4);
    return u32x4{lo, hi, lo, hi};
  }
  static __device__ inline f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0,
                                                  0, 0);
  }
  static __device__ inline float scale_to_float(uint32_t szw) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(szw & 0xFFFFu));
  }
  static __device__ inline uint16_t to_bits(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
};

template <>
struct Ops<__bf16> {
  // bf16 has 7 mantissa bits: only nibbles at bits 0-3 of a half can be or-ed in, as 128 + u
  static __device__ inline u32x4 unpack(uint32_t x, uint32_t m_lo, uint32_t, uint32_t c_lo, uint32_t) {
    u32x4 v;
    v[0] = (x & m_lo) | c_lo;
    v[1] = ((x >> 4) & m_lo) | c_lo;
    v[2] = ((x >> 8) & m_lo) | c_lo;
    v[3] = ((x >> 12) & m_lo) | c_lo;
    return v;
  }
  static constexpr uint32_t kMaskLo = 0x000F000Fu, kMaskHi = 0x000F000Fu;
  static constexpr uint32_t kMagicLo = 0x43004300u, kMagicHi = 0x43004300u;
  static __device__ inline u32x4 unpack_uniform(uint32_t x, uint32_t m_lo, uint32_t c_lo) {
    return unpack(x, m_lo, m_lo, c_lo, c_lo);
  }
  static constexpr float kBias = 128.f;
  static constexpr uint32_t kOnes = 0x3F803F80u;
  static __device__ inline u32x4 correction(uint32_t zc) {
    const uint32_t v = 0xC300C300u | zc;
    return u32x4{v, v, v, v};
  }
  static __device__ inline f32x4 mfma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                   0, 0, 0);
  }
  static __device__ inline float scale_to_float(uint32_t szw) { return __builtin_bit_cast(float, szw << 16); }
  static __device__ inline uint16_t to_bits(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }
};

// Weight-side dequantisation for the kernels with many row tiles: a word of eight nibbles becomes eight fp16
// values T((u - z) * s), u - z exact and the product rounded once.
typedef _Float16 half2v __attribute__((ext_vector_type(2)));

template <typename T>
struct Dequant;

template <>
struct Dequant<_Float16> {
  // per (group, column): packed (s, s), packed (1024 + z), packed (64 + z)
  struct Consts {
    uint32_t s2, c_lo, c_hi;
  };
  static __device__ inline Consts prepare(uint32_t szw) {
    const uint32_t z = (szw >> 16) & 15u, zc = z | (z << 16);
    Consts k;
    k.s2 = (szw & 0xFFFFu) | (szw << 16);
    k.c_lo = 0x64006400u | zc;
    k.c_hi = 0x54005400u | (zc << 4);
    return k;
  }
  static __device__ inline u32x4 run(uint32_t x, const Consts& k, uint32_t m_lo, uint32_t m_hi, uint32_t g_lo,
                                     uint32_t g_hi) {
    const uint32_t y = x >> 8;
    const half2v s = __builtin_bit_cast(half2v, k.s2);
    const half2v clo = __builtin_bit_cast(half2v, k.c_lo), chi = __builtin_bit_cast(half2v, k.c_hi);
    half2v r0 = (__builtin_bit_cast(half2v, (x & m_lo) | g_lo) - clo) * s;
    half2v r1 = (__builtin_bit_cast(half2v, (x & m_hi) | g_hi) - chi) * s;
    half2v r2 = (__builtin_bit_cast(half2v, (y & m_lo) | g_lo) - clo) * s;
    half2v r3 = (__builtin_bit_cast(half2v, (y & m_hi) | g_hi) - chi) * s;
    return u32x4{__builtin_bit_cast(uint32_t, r0), __builtin_bit_cast(uint32_t, r1), __builtin_bit_cast(uint32_t, r2),
                 __builtin_bit_cast(uint32_t, r3)};
  }
};

template <>
struct Dequant<__bf16> : Dequant<_Float16> {
  // Scales arrive as bf16 bits; the arithmetic is the fp16 one.  A bf16 scale can lie far outside the fp16 range, so
  // the scale is first divided by 2^E, E = the column's largest scale exponent (bits 24..31 of every scale/zero word
  // of the column, written by the repack): the column's largest scale becomes 1.x, smaller ones keep all their
  // bits down to 2^-14 of it.  column_factors() below gives the 2^E that the fp32 result of the column is owed.
  static __device__ inline Consts prepare(uint32_t szw) {
    const _Float16 sh = (_Float16)__builtin_ldexpf(__builtin_bit_cast(float, szw << 16), -((int)szw >> 24));
    const uint32_t sb = __builtin_bit_cast(uint16_t, sh);
    return Dequant<_Float16>::prepare((szw & 0x000F0000u) | sb);
  }
};

// 2^E of the eight columns col .. col + 7 (col a multiple of 8, col + 8 <= N) of a weight with bf16 scales; sz is the
// scale/zero buffer [N/16][G][16].
__device__ inline void column_factors(const void* sz, int G, int col, float (&f)[8]) {
  const uint32_t* w = static_cast<const uint32_t*>(sz) + ((size_t)(col >> 4) * G) * 16 + (col & 15);
  const u32x4 lo = *reinterpret_cast<const u32x4*>(w), hi = *reinterpret_cast<const u32x4*>(w + 4);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    f[q] = __builtin_bit_cast(float, (uint32_t)(((int)lo[q] >> 24) + 127) << 23);
    f[4 + q] = __builtin_bit_cast(float, (uint32_t)(((int)hi[q] >> 24) + 127) << 23);
  }
}

}  // namespace w4
}  // namespace ksq
