// Load-time repack: checkpoint / canonical int4 layouts -> MFMA fragment order (see include/ksq.h).
// Pure byte shuffling, bound by HBM bandwidth; one thread builds one 32-bit output word (eight nibbles).
#include <vector>

#include "ksq_internal.h"

namespace ksq {
namespace {

struct RepackArgs {
  const void* qweight;
  const void* zeros;
  const void* scales;
  uint32_t* dst_weight;
  uint32_t* dst_sz;
  size_t K, N, g;  // K = rows of the source tensors
  size_t Kp;       // rows of the destination: K rounded up to whole 128-row tiles (the rows past K hold u = z = 8
                   // under a zero scale, and the GEMM gives them zero activations)
  int layout, zero_kind, scale_dtype;
  const int32_t* row_perm;  // destination row i holds source row row_perm[i]; null = identity
  int column_order;
  const int8_t* col_exp;    // host repack: column_exponent() of every source scale column, computed once; else null
};

// bf16 scales only: the largest binary exponent among the finite, non-zero scales of source scale column `ns` (0
// when there is none).  The kernels that run their matrix instructions in fp16 divide a column's scales by 2 to
// this power, which keeps them inside the fp16 range whatever their magnitude, and put the factor back on the fp32
// result of the column.
__host__ __device__ inline int column_exponent(const RepackArgs& a, size_t ns) {
  if (a.scale_dtype != KSQ_BF16) return 0;
  if (a.col_exp) return a.col_exp[ns];
  const size_t G = a.K / a.g;
  int best = -1000;
  for (size_t gi = 0; gi < G; ++gi) {
    const int e = (static_cast<const uint16_t*>(a.scales)[gi * a.N + ns] >> 7) & 0xFF;
    if (e != 0 && e != 255 && e - 127 > best) best = e - 127;
  }
  return best == -1000 ? 0 : best;
}

// source column of destination column n
__host__ __device__ inline size_t source_column(const RepackArgs& a, size_t n) {
  if (a.column_order == KSQ_COLS_HALVES_INTERLEAVED) return (n & 1) * (a.N >> 1) + (n >> 1);
  return n;
}

__host__ __device__ inline float bits16_to_float(uint16_t b, int dtype) {
  if (dtype == KSQ_BF16) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    __builtin_memcpy(&f, &u, 4);
    return f;
  }
  // fp16 -> fp32 by hand so that host and device agree bit for bit
  uint32_t s = (uint32_t)(b & 0x8000u) << 16, e = (b >> 10) & 0x1Fu, m = b & 0x3FFu, u;
  if (e == 0) {
    if (m == 0) {
      u = s;
    } else {
      int sh = 0;
      while (!(m & 0x400u)) {
        m <<= 1;
        ++sh;
      }
      u = s | ((uint32_t)(113 - sh) << 23) | ((m & 0x3FFu) << 13);
    }
  } else if (e == 31) {
    u = s | 0x7F800000u | (m << 13);
  } else {
    u = s | ((e + 112u) << 23) | (m << 13);
  }
  float f;
  __builtin_memcpy(&f, &u, 4);
  return f;
}

// unsigned nibble u[k, n] of the source tensor
__host__ __device__ inline uint32_t source_nibble(const RepackArgs& a, size_t k, size_t n) {
  switch (a.layout) {
    case KSQ_W4_GPTQ_INT32_KPACK: {
      uint32_t w = static_cast<const uint32_t*>(a.qweight)[(k >> 3) * a.N + n];
      return (w >> (4 * (k & 7))) & 0xFu;
    }
    case KSQ_W4_AWQ_INT32_NPACK: {
      // logical column 8c + i sits in slot [0,4,1,5,2,6,3,7][i]
      uint32_t w = static_cast<const uint32_t*>(a.qweight)[k * (a.N >> 3) + (n >> 3)];
      int i = (int)(n & 7);
      int slot = (i >> 1) + 4 * (i & 1);
      return (w >> (4 * slot)) & 0xFu;
    }
    case KSQ_W4_CUTLASS_SM80_INTERLEAVED: {
      // Inverse of the four steps of preprocess_weights_for_mixed_gemm for W4_A16 on sm80
      // (LK/asymmetric_gemm/cutlass_preprocessors.cpp:466-508), read backwards:
      //  row permutation inside groups of 32 rows (:129-141, :143-197): position r' of a group holds row map[r'];
      //  transpose to column major, eight consecutive rows per 32-bit register (:203-323);
      //  four columns interleaved in tiles of 64 rows = 8 registers (:426-464, with the layout
      //  ColumnMajorTileInterleave<64, 4> of LK/cutlass_extensions/gemm/kernel/mixed_gemm_B_layout.h);
      //  + 8 and the register relayout [e0 e2 e4 e6 e1 e3 e5 e7] (:352-401).
      const size_t r32 = k & 31;
      // inverse of {0,1,8,9,16,17,24,25, 2,3,10,11,18,19,26,27, 4,5,12,13,20,21,28,29, 6,7,14,15,22,23,30,31}:
      // row r32 = 8a + 2b + c (a, b < 4, c < 2) sits at position 8b + 2a + c
      const size_t pos = 8 * ((r32 >> 1) & 3) + 2 * (r32 >> 3) + (r32 & 1);
      const size_t rp = (k - r32) + pos;
      const size_t v = rp >> 3, e = rp & 7;                    // register along k and element inside it
      const size_t vw = 4 * (v & ~(size_t)7) + 8 * (n & 3) + (v & 7);
      const uint32_t w = static_cast<const uint32_t*>(a.qweight)[(n >> 2) * (a.K >> 3) * 4 + vw];
      const int slot = (e & 1) ? 4 + (int)(e >> 1) : (int)(e >> 1);
      return (w >> (4 * slot)) & 0xFu;  // already unsigned
    }
    case KSQ_W4_MARLIN: {
      // inverse of repack_tile (LK/gptq_marlin/gptq_marlin_repack.cu:128-206): thread th of warp w packs
      // k = 2 * (th % 4) + {0, 1, 8, 9} of columns 16 w + th / 4 and + 8 into word th * 4 + w of the 16 x 64 tile
      const size_t kk = k & 15, nn = n & 63;
      const size_t w = nn >> 4, blk = (nn >> 3) & 1, tc_col = nn & 7;
      const size_t th = tc_col * 4 + ((kk >> 1) & 3);
      const int v = (int)((kk & 1) + 2 * (kk >> 3) + 4 * blk);   // index into vals[8]
      const int slot = (v & 1) ? 4 + (v >> 1) : (v >> 1);        // pack_idx[slot] == v
      const size_t word = ((k >> 4) * (a.N >> 6) + (n >> 6)) * 128 + th * 4 + w;
      return (static_cast<const uint32_t*>(a.qweight)[word] >> (4 * slot)) & 0xFu;
    }
    case KSQ_W4_CUTLASS_SM90_COLMAJOR: {  // transpose only: int8 [N, K/2], signed
      uint8_t b = static_cast<const uint8_t*>(a.qweight)[n * (a.K >> 1) + (k >> 1)];
      uint32_t nib = (k & 1) ? (b >> 4) : (b & 0xFu);
      return nib ^ 8u;
    }
    default: {  // KSQ_W4_ROWMAJOR_INT4_SIGNED: two's-complement q, u = q + 8 = nibble ^ 8
      uint8_t b = static_cast<const uint8_t*>(a.qweight)[k * (a.N >> 1) + (n >> 1)];
      uint32_t nib = (n & 1) ? (b >> 4) : (b & 0xFu);
      return nib ^ 8u;
    }
  }
}

__host__ __device__ inline uint32_t build_weight_word(const RepackArgs& a, size_t word) {
  size_t k0, n;
  frag_word_origin(word, a.Kp, &k0, &n);
  n = source_column(a, n);
  uint32_t out = 0;
  if (k0 >= a.K) return 0x88888888u;  // padding rows (eight rows at a time: K is a multiple of 64)
  if (a.row_perm) {
    for (int e = 0; e < 8; ++e) {
      size_t kr = (size_t)(uint32_t)a.row_perm[k0 + e];
      if (kr >= a.K) kr = 0;  // a bad entry must not turn into a wild read
      out |= source_nibble(a, kr, n) << (4 * frag_nibble_of(e));
    }
    return out;
  }
  if (a.layout == KSQ_W4_GPTQ_INT32_KPACK) {
    // the eight elements are the eight nibbles of one source word, in k order
    uint32_t w = static_cast<const uint32_t*>(a.qweight)[(k0 >> 3) * a.N + n];
    for (int e = 0; e < 8; ++e) out |= ((w >> (4 * e)) & 0xFu) << (4 * frag_nibble_of(e));
    return out;
  }
  for (int e = 0; e < 8; ++e) out |= source_nibble(a, k0 + e, n) << (4 * frag_nibble_of(e));
  return out;
}

__host__ __device__ inline uint32_t build_sz_word(const RepackArgs& a, size_t idx) {
  // idx enumerates [N/16][G][16], G counted over the padded rows
  const size_t G = a.Kp / a.g;
  size_t c = idx & 15, rest = idx >> 4;
  size_t gi = rest % G, nt = rest / G;
  size_t n = source_column(a, nt * kTileN + c);
  const bool padding = gi >= a.K / a.g;
  if (padding) gi = 0;  // the padding group: zero scale, z = 8, the column's exponent field like every other word
  // Marlin keeps scales (and zero points) permuted inside blocks of 64 columns, or of 32 when there is a single
  // group (MarlinPermuteScales, KS/models/quant/quant_weight.cpp:350-375): entry p of a block is column
  // p / 8 + 8 * (p % 8), resp. 2 * (p / 8) + {0,1,8,9,16,17,24,25}[p % 8]
  size_t ns = n;
  if (a.layout == KSQ_W4_MARLIN) {
    if (G > 1) {
      const size_t q = n & 63;
      ns = (n & ~(size_t)63) + 8 * (q & 7) + (q >> 3);
    } else {
      const size_t q = n & 31, pair = q >> 1, odd = q & 1;  // q = 2 i + (8 h + odd): i = pair & 3, h = pair >> 2
      ns = (n & ~(size_t)31) + 8 * (pair & 3) + 2 * (pair >> 2) + odd;
    }
  }
  uint16_t sbits = static_cast<const uint16_t*>(a.scales)[gi * a.N + ns];
  uint32_t z = 8;
  if (padding) return (8u << 16) | ((uint32_t)(uint8_t)(int8_t)column_exponent(a, ns) << 24);
  switch (a.zero_kind) {
    case KSQ_ZERO_AWQ_INT32: {
      uint32_t w = static_cast<const uint32_t*>(a.zeros)[gi * (a.N >> 3) + (n >> 3)];
      int i = (int)(n & 7);
      int slot = (i >> 1) + 4 * (i & 1);
      z = (w >> (4 * slot)) & 0xFu;
      break;
    }
    case KSQ_ZERO_MARLIN_INT32: {
      // MarlinZeroPoints (quant_weight.cpp:397-426): the grouped scale permutation on blocks of 64, then
      // [0,2,4,6,1,3,5,7] on blocks of 8, then eight consecutive columns per word
      const size_t q = n & 63, p = 8 * (q & 7) + (q >> 3), r = p & 7;
      const size_t t = (r & 1) ? 4 + (r >> 1) : (r >> 1);
      const size_t col = (n & ~(size_t)63) + (p & ~(size_t)7) + t;
      uint32_t w = static_cast<const uint32_t*>(a.zeros)[gi * (a.N >> 3) + (col >> 3)];
      z = (w >> (4 * (col & 7))) & 0xFu;
      break;
    }
    case KSQ_ZERO_UINT8:
      z = static_cast<const uint8_t*>(a.zeros)[gi * a.N + n] & 0xFu;
      break;
    case KSQ_ZERO_ADDITIVE: {
      // zeros' = T(s * (8 - z)): the quotient is within 2^-8 of the integer 8 - z, so rounding recovers z
      float s = bits16_to_float(sbits, a.scale_dtype);
      float za = bits16_to_float(static_cast<const uint16_t*>(a.zeros)[gi * a.N + n], a.scale_dtype);
      float q = (s != 0.0f) ? za / s : 0.0f;
      float r = 8.0f - (q >= 0.0f ? (float)(int)(q + 0.5f) : -(float)(int)(-q + 0.5f));
      if (!(r >= 0.0f)) r = 0.0f;
      if (r > 15.0f) r = 15.0f;
      z = (uint32_t)r;
      break;
    }
    default:
      break;
  }
  return (uint32_t)sbits | (z << 16) | ((uint32_t)(uint8_t)(int8_t)column_exponent(a, ns) << 24);
}

__global__ __launch_bounds__(256) void repack_weight_kernel(RepackArgs a, size_t words) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < words) a.dst_weight[i] = build_weight_word(a, i);
}

__global__ __launch_bounds__(256) void repack_sz_kernel(RepackArgs a, size_t count) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < count) a.dst_sz[i] = build_sz_word(a, i);
}

int validate(int layout, const void* qweight, int zero_kind, const void* zeros, const void* scales, int scale_dtype,
             size_t k, size_t n, size_t g, int column_order, const void* dw, const void* dsz) {
  KSQ_REQUIRE(layout >= KSQ_W4_GPTQ_INT32_KPACK && layout <= KSQ_W4_MARLIN, KSQ_ERR_INVALID_ARGUMENT,
              "bad source layout %d", layout);
  KSQ_REQUIRE(zero_kind >= KSQ_ZERO_NONE && zero_kind <= KSQ_ZERO_MARLIN_INT32, KSQ_ERR_INVALID_ARGUMENT,
              "bad zero kind %d", zero_kind);
  KSQ_REQUIRE(layout != KSQ_W4_MARLIN || n % 64 == 0, KSQ_ERR_UNSUPPORTED,
              "the Marlin layout needs n %% 64 == 0 (got %zu)", n);
  KSQ_REQUIRE((zero_kind == KSQ_ZERO_MARLIN_INT32) == (layout == KSQ_W4_MARLIN && zero_kind != KSQ_ZERO_NONE),
              KSQ_ERR_INVALID_ARGUMENT, "Marlin zero points go with the Marlin weight layout and with no other");
  KSQ_REQUIRE(scale_dtype == KSQ_F16 || scale_dtype == KSQ_BF16, KSQ_ERR_INVALID_ARGUMENT, "bad scale dtype %d",
              scale_dtype);
  KSQ_REQUIRE(column_order == KSQ_COLS_NATURAL || column_order == KSQ_COLS_HALVES_INTERLEAVED,
              KSQ_ERR_INVALID_ARGUMENT, "bad column order %d", column_order);
  KSQ_REQUIRE(qweight && scales && dw && dsz, KSQ_ERR_INVALID_ARGUMENT, "null tensor pointer");
  KSQ_REQUIRE(zero_kind == KSQ_ZERO_NONE || zeros, KSQ_ERR_INVALID_ARGUMENT, "zero points requested but null");
  size_t wb, sb;
  int rc = ksq_w4a16_repack_sizes(k, n, g, &wb, &sb);
  if (rc != KSQ_OK) return rc;
  KSQ_REQUIRE(n % 8 == 0, KSQ_ERR_UNSUPPORTED, "n must be a multiple of 8");
  return KSQ_OK;
}

RepackArgs make_args(int layout, const void* qweight, int zero_kind, const void* zeros, const void* scales,
                     int scale_dtype, size_t k, size_t n, size_t g, const int32_t* row_perm, int column_order,
                     void* dst_weight, void* dst_sz) {
  RepackArgs a{};
  a.qweight = qweight;
  a.zeros = zeros;
  a.scales = scales;
  a.dst_weight = static_cast<uint32_t*>(dst_weight);
  a.dst_sz = static_cast<uint32_t*>(dst_sz);
  a.K = k;
  a.Kp = (k + kTileK - 1) / kTileK * kTileK;
  a.N = n;
  a.g = g;
  a.layout = layout;
  a.zero_kind = zero_kind;
  a.scale_dtype = scale_dtype;
  a.row_perm = row_perm;
  a.column_order = column_order;
  return a;
}

// out [m][k_out] = in [m][k_in] then zeros: one thread per eight destination elements
__global__ __launch_bounds__(256) void pad_rows_kernel(uint32_t* out, const uint32_t* in, size_t m, size_t k_in,
                                                       size_t k_out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t per_row = k_out / 8;
  if (i >= m * per_row) return;
  const size_t row = i / per_row, c = i - row * per_row;
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  if (c * 8 < k_in) {
    const uint32_t* src = in + (row * k_in + c * 8) / 2;
    for (int q = 0; q < 4; ++q) w[q] = src[q];
  }
  uint32_t* dst = out + (row * k_out + c * 8) / 2;
  for (int q = 0; q < 4; ++q) dst[q] = w[q];
}

// out[m, i] = in[m, perm[i]]: one thread per eight destination elements (16 bytes stored)
__global__ __launch_bounds__(256) void permute_columns_kernel(uint16_t* out, const uint16_t* in, const int32_t* perm,
                                                              size_t m, size_t k) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;  // group of eight columns
  const size_t per_row = k / 8;
  if (i >= m * per_row) return;
  const size_t row = i / per_row, c0 = (i - row * per_row) * 8;
  const uint16_t* src = in + row * k;
  uint32_t w[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    uint32_t p0 = (uint32_t)perm[c0 + 2 * q], p1 = (uint32_t)perm[c0 + 2 * q + 1];
    p0 = p0 < k ? p0 : 0;  // a bad entry must not turn into a wild read
    p1 = p1 < k ? p1 : 0;
    const uint32_t lo = src[p0], hi = src[p1];
    w[q] = lo | (hi << 16);
  }
  uint4 v{w[0], w[1], w[2], w[3]};
  *reinterpret_cast<uint4*>(out + row * k + c0) = v;
}

// out row 2i = in row i, out row 2i + 1 = in row rows/2 + i; one thread per 32-bit word
__global__ __launch_bounds__(256) void interleave_halves_kernel(uint32_t* out, const uint32_t* in, size_t rows,
                                                                size_t row_words) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * row_words) return;
  const size_t r = i / row_words, w = i - r * row_words;
  const size_t src = (r & 1) * (rows / 2) + (r >> 1);
  out[i] = in[src * row_words + w];
}

}  // namespace
}  // namespace ksq

using namespace ksq;

extern "C" int ksq_w4a16_repack_ex(int layout, const void* qweight, int zero_kind, const void* zeros,
                                   const void* scales, int scale_dtype, size_t k, size_t n, size_t g,
                                   const int32_t* row_perm, int column_order, void* dst_weight, void* dst_sz,
                                   void* stream) {
  int rc = validate(layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, g, column_order, dst_weight, dst_sz);
  if (rc != KSQ_OK) return rc;
  RepackArgs a = make_args(layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, g, row_perm, column_order,
                           dst_weight, dst_sz);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t words = a.Kp * n / 8, count = (a.Kp / g) * n;
  KSQ_REQUIRE((words + 255) / 256 < (1ull << 31), KSQ_ERR_UNSUPPORTED, "tensor too large for one launch");
  hipLaunchKernelGGL(repack_weight_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, a, words);
  hipLaunchKernelGGL(repack_sz_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, a, count);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

int ksq::pad_rows(void* out, const void* in, size_t m, size_t k_in, size_t k_out, hipStream_t s) {
  const size_t threads = m * (k_out / 8);
  KSQ_REQUIRE((threads + 255) / 256 < (1ull << 31), KSQ_ERR_UNSUPPORTED, "tensor too large for one launch");
  hipLaunchKernelGGL(pad_rows_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s,
                     static_cast<uint32_t*>(out), static_cast<const uint32_t*>(in), m, k_in, k_out);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

extern "C" int ksq_w4a16_repack(int layout, const void* qweight, int zero_kind, const void* zeros,
                                const void* scales, int scale_dtype, size_t k, size_t n, size_t g, void* dst_weight,
                                void* dst_sz, void* stream) {
  return ksq_w4a16_repack_ex(layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, g, nullptr,
                             KSQ_COLS_NATURAL, dst_weight, dst_sz, stream);
}

extern "C" int ksq_w4a16_repack_ex_host(int layout, const void* qweight, int zero_kind, const void* zeros,
                                        const void* scales, int scale_dtype, size_t k, size_t n, size_t g,
                                        const int32_t* row_perm, int column_order, void* dst_weight, void* dst_sz) {
  int rc = validate(layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, g, column_order, dst_weight, dst_sz);
  if (rc != KSQ_OK) return rc;
  if (row_perm)
    for (size_t i = 0; i < k; ++i)
      KSQ_REQUIRE(row_perm[i] >= 0 && (size_t)row_perm[i] < k, KSQ_ERR_INVALID_ARGUMENT,
                  "row_perm[%zu] = %d is outside [0, %zu)", i, row_perm[i], k);
  RepackArgs a = make_args(layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, g, row_perm, column_order,
                           dst_weight, dst_sz);
  const size_t words = a.Kp * n / 8, count = (a.Kp / g) * n;
  std::vector<int8_t> col_exp;
  if (scale_dtype == KSQ_BF16) {
    col_exp.resize(n);
    for (size_t ns = 0; ns < n; ++ns) col_exp[ns] = (int8_t)column_exponent(a, ns);
    a.col_exp = col_exp.data();
  }
  for (size_t i = 0; i < words; ++i) a.dst_weight[i] = build_weight_word(a, i);
  for (size_t i = 0; i < count; ++i) a.dst_sz[i] = build_sz_word(a, i);
  return KSQ_OK;
}

extern "C" int ksq_w4a16_repack_host(int layout, const void* qweight, int zero_kind, const void* zeros,
                                     const void* scales, int scale_dtype, size_t k, size_t n, size_t g,
                                     void* dst_weight, void* dst_sz) {
  return ksq_w4a16_repack_ex_host(layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, g, nullptr,
                                  KSQ_COLS_NATURAL, dst_weight, dst_sz);
}

extern "C" int ksq_gptq_act_order_perm(const int32_t* g_idx, size_t k, size_t g, int32_t* perm) {
  KSQ_REQUIRE(g_idx && perm, KSQ_ERR_INVALID_ARGUMENT, "null pointer");
  KSQ_REQUIRE(g > 0 && k > 0 && k % g == 0 && k < (1ull << 31), KSQ_ERR_INVALID_ARGUMENT,
              "k=%zu must be a positive multiple of the group size %zu", k, g);
  const size_t groups = k / g;
  // counting sort = stable argsort for keys in [0, groups)
  std::vector<size_t> fill(groups, 0);
  for (size_t i = 0; i < k; ++i) {
    KSQ_REQUIRE(g_idx[i] >= 0 && (size_t)g_idx[i] < groups, KSQ_ERR_INVALID_ARGUMENT,
                "g_idx[%zu] = %d is outside [0, %zu)", i, g_idx[i], groups);
    ++fill[(size_t)g_idx[i]];
  }
  for (size_t gi = 0; gi < groups; ++gi)
    KSQ_REQUIRE(fill[gi] == g, KSQ_ERR_UNSUPPORTED,
                "group %zu has %zu rows, not %zu: a partial group cannot run on kernels for grouped rows", gi,
                fill[gi], g);
  for (size_t gi = 0; gi < groups; ++gi) fill[gi] = gi * g;
  for (size_t i = 0; i < k; ++i) perm[fill[(size_t)g_idx[i]]++] = (int32_t)i;
  return KSQ_OK;
}

extern "C" int ksq_permute_columns(void* out, const void* in, const int32_t* perm, size_t m, size_t k,
                                   void* stream) {
  KSQ_REQUIRE(out && in && perm, KSQ_ERR_INVALID_ARGUMENT, "null pointer");
  KSQ_REQUIRE(out != in, KSQ_ERR_INVALID_ARGUMENT, "in-place permutation is not supported");
  KSQ_REQUIRE(k % 8 == 0, KSQ_ERR_UNSUPPORTED, "k=%zu must be a multiple of 8", k);
  KSQ_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15) == 0, KSQ_ERR_INVALID_ARGUMENT, "out must be 16-byte aligned");
  if (m == 0 || k == 0) return KSQ_OK;
  const size_t items = m * (k / 8);
  KSQ_REQUIRE((items + 255) / 256 < (1ull << 31), KSQ_ERR_UNSUPPORTED, "tensor too large for one launch");
  hipLaunchKernelGGL(permute_columns_kernel, dim3((unsigned)((items + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint16_t*>(out), static_cast<const uint16_t*>(in),
                     perm, m, k);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

extern "C" int ksq_interleave_halves(void* out, const void* in, size_t rows, size_t row_bytes, void* stream) {
  KSQ_REQUIRE(out && in && out != in, KSQ_ERR_INVALID_ARGUMENT, "null or aliased pointers");
  KSQ_REQUIRE(rows % 2 == 0 && row_bytes % 4 == 0, KSQ_ERR_UNSUPPORTED,
              "rows=%zu must be even and row_bytes=%zu a multiple of 4", rows, row_bytes);
  if (rows == 0 || row_bytes == 0) return KSQ_OK;
  const size_t words = rows * (row_bytes / 4);
  KSQ_REQUIRE((words + 255) / 256 < (1ull << 31), KSQ_ERR_UNSUPPORTED, "tensor too large for one launch");
  hipLaunchKernelGGL(interleave_halves_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint32_t*>(out), static_cast<const uint32_t*>(in),
                     rows, row_bytes / 4);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}
