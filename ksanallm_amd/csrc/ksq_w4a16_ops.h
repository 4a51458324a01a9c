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

}  // namespace w4
}  // namespace ksq
