// What every GEMM kernel of the library does with its fp32 result on the way out: nothing, a bias row, or
// SiLU(gate) * up on column pairs (see ksq_epilogue in include/ksq.h).  Two store shapes cover all kernels: the MFMA
// accumulator layout (a lane holds four rows of one column) and a row segment of eight consecutive columns.
#pragma once

#include "ksq_internal.h"

namespace ksq {

typedef float epi_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t epi_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t epi_u32x2 __attribute__((ext_vector_type(2)));

// The element a kernel stores: 16-bit patterns for fp16 / bf16 results, floats for fp32 ones (the FP8 GEMM only: the
// reference's Fp8MatMulLayer<float> takes an fp32 result from its GEMM, KS/kernels/nvidia/kernel_wrapper.cpp:1043).
template <typename T>
struct EpiElem {
  typedef uint16_t type;
};
template <>
struct EpiElem<float> {
  typedef float type;
};
template <typename T>
using epi_elem_t = typename EpiElem<T>::type;

template <typename T>
__device__ inline epi_elem_t<T> epi_bits(float v) {
  if constexpr (__is_same(T, float)) return v;
  else return __builtin_bit_cast(uint16_t, (T)v);
}
template <typename T>
__device__ inline float epi_float(epi_elem_t<T> b) {
  if constexpr (__is_same(T, float)) return b;
  else return (float)__builtin_bit_cast(T, b);
}

__device__ inline float epi_silu(float x) { return x / (1.0f + __expf(-x)); }

// Accumulator layout: the lane holds v[e] = result at (row0 + e, col), and lane ^ 1 holds column col ^ 1 of the
// same rows.  Every lane of the wave must make the call (it contains a cross-lane exchange); `ok` says whether this
// lane's column exists, rows are clipped against M.  N is the width of the GEMM (of the weight).
template <typename T>
__device__ inline void epi_store_acc(const Epilogue& ep, epi_elem_t<T>* out, epi_f32x4 v, int row0, int col, int M, int N,
                                     bool ok) {
  epi_elem_t<T> bits[4];
  bool mine = ok;
  size_t width = (size_t)N;
  int ocol = col;
  if (ep.kind == KSQ_EPILOGUE_SILU_MUL) {
    // value of the neighbouring lane (lane ^ 1): DPP quad permutation [1, 0, 3, 2].  The elements are copied into
    // scalars first: a bit cast applied to a vector element directly reads element 0 whatever the index.
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float gate = v[e];
      const float up = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, gate), 0xB1, 0xF, 0xF, true));
      bits[e] = epi_bits<T>(epi_silu(gate) * up);
    }
    mine = ok && !(col & 1);
    width = (size_t)(N >> 1);
    ocol = col >> 1;
  } else {
    float b = 0.f;
    if (ep.kind == KSQ_EPILOGUE_BIAS && ok) b = epi_float<T>(static_cast<const epi_elem_t<T>*>(ep.bias)[col]);
#pragma unroll
    for (int e = 0; e < 4; ++e) bits[e] = epi_bits<T>(v[e] + b);
  }
  if (mine) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (row0 + e < M) out[(size_t)(row0 + e) * width + ocol] = bits[e];
  }
  if (ep.row_absmax) {
    // The largest |stored value| of every row, for whoever quantises this output per token next: the 16 lanes that
    // hold a row's 16 columns of this tile agree on their maximum, one of them folds it into row_absmax[row] with an
    // atomic maximum on the bit pattern (non-negative floats order like unsigned integers), as the reference's
    // quantiser merges its blocks (LU/cuda_fp8_utils.cu:111-115).  Uniform over the wave: every lane gets here.
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float a = (mine && row0 + e < M) ? __builtin_fabsf(epi_float<T>(bits[e])) : 0.f;
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) a = __builtin_fmaxf(a, __shfl_xor(a, off));
      if ((col & 15) == 0 && row0 + e < M)
        atomicMax(reinterpret_cast<unsigned*>(ep.row_absmax) + (row0 + e), __builtin_bit_cast(unsigned, a));
    }
  }
}

// Row segment: src[0..7] = results at (row, col .. col + 7), col a multiple of 8 and col + 8 <= N, row < M.  Returns the
// largest |stored value| of the segment.
template <typename T>
__device__ inline float epi_store_row8(const Epilogue& ep, epi_elem_t<T>* out, const float (&src)[8], int row, int col,
                                       int N) {
  float mx = 0.f;
  if constexpr (__is_same(T, float)) {  // 32-bit results: sixteen or thirty-two bytes per segment
    if (ep.kind == KSQ_EPILOGUE_SILU_MUL) {
      epi_f32x4 r;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        r[q] = epi_silu(src[2 * q]) * src[2 * q + 1];
        mx = __builtin_fmaxf(mx, __builtin_fabsf(r[q]));
      }
      *reinterpret_cast<epi_f32x4*>(out + (size_t)row * (size_t)(N >> 1) + (col >> 1)) = r;
      return mx;
    }
    epi_f32x4 lo, hi;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      float b0 = 0.f, b1 = 0.f;
      if (ep.kind == KSQ_EPILOGUE_BIAS) {
        b0 = static_cast<const float*>(ep.bias)[col + q];
        b1 = static_cast<const float*>(ep.bias)[col + 4 + q];
      }
      lo[q] = src[q] + b0;
      hi[q] = src[4 + q] + b1;
      mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(lo[q]), __builtin_fabsf(hi[q])));
    }
    epi_f32x4* dst = reinterpret_cast<epi_f32x4*>(out + (size_t)row * N + col);
    dst[0] = lo;
    dst[1] = hi;
    return mx;
  } else {
  if (ep.kind == KSQ_EPILOGUE_SILU_MUL) {
    epi_u32x2 packed;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const uint16_t lo = epi_bits<T>(epi_silu(src[4 * q]) * src[4 * q + 1]);
      const uint16_t hi = epi_bits<T>(epi_silu(src[4 * q + 2]) * src[4 * q + 3]);
      packed[q] = (uint32_t)lo | ((uint32_t)hi << 16);
      mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(epi_float<T>(lo)), __builtin_fabsf(epi_float<T>(hi))));
    }
    *reinterpret_cast<epi_u32x2*>(out + (size_t)row * (size_t)(N >> 1) + (col >> 1)) = packed;
    return mx;
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
  for (int q = 0; q < 4; ++q) {
    const uint16_t lo = epi_bits<T>(src[2 * q] + b[2 * q]), hi = epi_bits<T>(src[2 * q + 1] + b[2 * q + 1]);
    packed[q] = (uint32_t)lo | ((uint32_t)hi << 16);
    mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(epi_float<T>(lo)), __builtin_fabsf(epi_float<T>(hi))));
  }
  *reinterpret_cast<epi_u32x4*>(out + (size_t)row * N + col) = packed;
  return mx;
  }
}

// The tile kernels' form: every lane of the wave makes the call, `live` says whether this lane has a segment to store;
// the eight lanes lane & ~7 .. hold the same row (when `row_ok`), so with ep.row_absmax set they agree on the row's
// maximum over their 64 columns before one of them merges it.
template <typename T>
__device__ inline void epi_store_row8_wave(const Epilogue& ep, epi_elem_t<T>* out, const float (&src)[8], int row, int col,
                                           int N, bool live, bool row_ok, int lane) {
  float mx = 0.f;
  if (live) mx = epi_store_row8<T>(ep, out, src, row, col, N);
  if (ep.row_absmax) {
#pragma unroll
    for (int off = 1; off < 8; off <<= 1) mx = __builtin_fmaxf(mx, __shfl_xor(mx, off));
    if ((lane & 7) == 0 && row_ok)
      atomicMax(reinterpret_cast<unsigned*>(ep.row_absmax) + row, __builtin_bit_cast(unsigned, mx));
  }
}

}  // namespace ksq
