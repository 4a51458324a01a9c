// What every GEMM kernel of the library does with its fp32 result on the way out: nothing, a bias row, or
// SiLU(gate) * up on column pairs (see ksq_epilogue in include/ksq.h).  Two store shapes cover all kernels: the MFMA
// accumulator layout (a lane holds four rows of one column) and a row segment of eight consecutive columns.
#pragma once

#include "ksq_internal.h"

namespace ksq {

typedef float epi_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t epi_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t epi_u32x2 __attribute__((ext_vector_type(2)));

template <typename T>
__device__ inline uint16_t epi_bits(float v) {
  return __builtin_bit_cast(uint16_t, (T)v);
}
template <typename T>
__device__ inline float epi_float(uint16_t b) {
  return (float)__builtin_bit_cast(T, b);
}

__device__ inline float epi_silu(float x) { return x / (1.0f + __expf(-x)); }

// Accumulator layout: the lane holds v[e] = result at (row0 + e, col), and lane ^ 1 holds column col ^ 1 of the
// same rows.  Every lane of the wave must make the call (it contains a cross-lane exchange); `ok` says whether this
// lane's column exists, rows are clipped against M.  N is the width of the GEMM (of the weight).
template <typename T>
__device__ inline void epi_store_acc(const Epilogue& ep, uint16_t* out, epi_f32x4 v, int row0, int col, int M, int N,
                                     bool ok) {
  if (ep.kind == KSQ_EPILOGUE_SILU_MUL) {
    // value of the neighbouring lane (lane ^ 1): DPP quad permutation [1, 0, 3, 2].  The elements are copied into
    // scalars first: a bit cast applied to a vector element directly reads element 0 whatever the index.
    epi_f32x4 up;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float mine = v[e];
      up[e] = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, mine), 0xB1, 0xF, 0xF, true));
    }
    if (ok && !(col & 1)) {
      const size_t half = (size_t)(N >> 1);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (row0 + e < M) out[(size_t)(row0 + e) * half + (col >> 1)] = epi_bits<T>(epi_silu(v[e]) * up[e]);
    }
    return;
  }
  if (!ok) return;
  float b = 0.f;
  if (ep.kind == KSQ_EPILOGUE_BIAS) b = epi_float<T>(static_cast<const uint16_t*>(ep.bias)[col]);
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (row0 + e < M) out[(size_t)(row0 + e) * N + col] = epi_bits<T>(v[e] + b);
}

// Row segment: src[0..7] = results at (row, col .. col + 7), col a multiple of 8 and col + 8 <= N, row < M.
template <typename T>
__device__ inline void epi_store_row8(const Epilogue& ep, uint16_t* out, const float (&src)[8], int row, int col,
                                      int N) {
  if (ep.kind == KSQ_EPILOGUE_SILU_MUL) {
    epi_u32x2 packed;
#pragma unroll
    for (int q = 0; q < 2; ++q)
      packed[q] = (uint32_t)epi_bits<T>(epi_silu(src[4 * q]) * src[4 * q + 1]) |
                  ((uint32_t)epi_bits<T>(epi_silu(src[4 * q + 2]) * src[4 * q + 3]) << 16);
    *reinterpret_cast<epi_u32x2*>(out + (size_t)row * (size_t)(N >> 1) + (col >> 1)) = packed;
    return;
  }
  float b[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (ep.kind == KSQ_EPILOGUE_BIAS) {
    const epi_u32x4 bw = *reinterpret_cast<const epi_u32x4*>(static_cast<const uint16_t*>(ep.bias) + col);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      b[2 * q] = epi_float<T>((uint16_t)(bw[q] & 0xFFFFu));
      b[2 * q + 1] = epi_float<T>((uint16_t)(bw[q] >> 16));
    }
  }
  epi_u32x4 packed;
#pragma unroll
  for (int q = 0; q < 4; ++q)
    packed[q] = (uint32_t)epi_bits<T>(src[2 * q] + b[2 * q]) | ((uint32_t)epi_bits<T>(src[2 * q + 1] + b[2 * q + 1]) << 16);
  *reinterpret_cast<epi_u32x4*>(out + (size_t)row * N + col) = packed;
}

}  // namespace ksq
