// FP8 e4m3 quantisation arithmetic shared by the quantisation kernels and the GEMM that quantises its own
// activations: scale = max(absmax / 448, 1 / (448 * 512)), q = e4m3(clamp(x / scale, +-448)) with a true division
// (Fp8E4m3Quantize of the reference: LU/cuda_fp8_utils.cu:27-44, 85-127, constants cuda_fp8_utils.h:42-43).
#pragma once

#include "ksq_internal.h"

namespace ksq {
namespace fp8ops {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float kE4m3Max = 448.0f;
constexpr float kMinScale = 1.0f / 448.0f / 512.0f;  // FP8_E4M3_MIN_SCALE of the reference

// eight 16-bit elements (one 16-byte access) as floats
template <typename T>
__device__ inline void unpack8(u32x4 v, float (&f)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (__is_same(T, _Float16)) {
      f[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[i] & 0xFFFFu));
      f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(v[i] >> 16));
    } else {
      f[2 * i] = __builtin_bit_cast(float, v[i] << 16);
      f[2 * i + 1] = __builtin_bit_cast(float, v[i] & 0xFFFF0000u);
    }
  }
}

__device__ inline float absmax8(const float (&f)[8], float mx) {
#pragma unroll
  for (int i = 0; i < 8; ++i) mx = fmaxf(mx, fabsf(f[i]));
  return mx;
}

__device__ inline u32x2 quantize8(const float (&f)[8], float scale) {
  float c[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) c[i] = fminf(fmaxf(f[i] / scale, -kE4m3Max), kE4m3Max);
  int lo = __builtin_amdgcn_cvt_pk_fp8_f32(c[0], c[1], 0, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(c[2], c[3], lo, true);
  int hi = __builtin_amdgcn_cvt_pk_fp8_f32(c[4], c[5], 0, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(c[6], c[7], hi, true);
  return u32x2{(uint32_t)lo, (uint32_t)hi};
}

}  // namespace fp8ops
}  // namespace ksq
