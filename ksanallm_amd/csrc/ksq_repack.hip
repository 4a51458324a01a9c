// Load-time repack: checkpoint / canonical int4 layouts -> MFMA fragment order (see include/ksq.h).
// Pure byte shuffling, bound by HBM bandwidth; one thread builds one 32-bit output word (eight nibbles).
#include "ksq_internal.h"

namespace ksq {
namespace {

struct RepackArgs {
  const void* qweight;
  const void* zeros;
  const void* scales;
  uint32_t* dst_weight;
  uint32_t* dst_sz;
  size_t K, N, g;
  int layout, zero_kind, scale_dtype;
};

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
    default: {  // KSQ_W4_ROWMAJOR_INT4_SIGNED: two's-complement q, u = q + 8 = nibble ^ 8
      uint8_t b = static_cast<const uint8_t*>(a.qweight)[k * (a.N >> 1) + (n >> 1)];
      uint32_t nib = (n & 1) ? (b >> 4) : (b & 0xFu);
      return nib ^ 8u;
    }
  }
}

__host__ __device__ inline uint32_t build_weight_word(const RepackArgs& a, size_t word) {
  size_t k0, n;
  frag_word_origin(word, a.K, &k0, &n);
  uint32_t out = 0;
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
  // idx enumerates [N/16][G][16]
  const size_t G = a.K / a.g;
  size_t c = idx & 15, rest = idx >> 4;
  size_t gi = rest % G, nt = rest / G;
  size_t n = nt * kTileN + c;
  uint16_t sbits = static_cast<const uint16_t*>(a.scales)[gi * a.N + n];
  uint32_t z = 8;
  switch (a.zero_kind) {
    case KSQ_ZERO_AWQ_INT32: {
      uint32_t w = static_cast<const uint32_t*>(a.zeros)[gi * (a.N >> 3) + (n >> 3)];
      int i = (int)(n & 7);
      int slot = (i >> 1) + 4 * (i & 1);
      z = (w >> (4 * slot)) & 0xFu;
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
  return (uint32_t)sbits | (z << 16);
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
             size_t k, size_t n, size_t g, const void* dw, const void* dsz) {
  KSQ_REQUIRE(layout >= KSQ_W4_GPTQ_INT32_KPACK && layout <= KSQ_W4_ROWMAJOR_INT4_SIGNED, KSQ_ERR_INVALID_ARGUMENT,
              "bad source layout %d", layout);
  KSQ_REQUIRE(zero_kind >= KSQ_ZERO_NONE && zero_kind <= KSQ_ZERO_ADDITIVE, KSQ_ERR_INVALID_ARGUMENT,
              "bad zero kind %d", zero_kind);
  KSQ_REQUIRE(scale_dtype == KSQ_F16 || scale_dtype == KSQ_BF16, KSQ_ERR_INVALID_ARGUMENT, "bad scale dtype %d",
              scale_dtype);
  KSQ_REQUIRE(qweight && scales && dw && dsz, KSQ_ERR_INVALID_ARGUMENT, "null tensor pointer");
  KSQ_REQUIRE(zero_kind == KSQ_ZERO_NONE || zeros, KSQ_ERR_INVALID_ARGUMENT, "zero points requested but null");
  size_t wb, sb;
  int rc = ksq_w4a16_repack_sizes(k, n, g, &wb, &sb);
  if (rc != KSQ_OK) return rc;
  KSQ_REQUIRE(n % 8 == 0, KSQ_ERR_UNSUPPORTED, "n must be a multiple of 8");
  return KSQ_OK;
}

}  // namespace
}  // namespace ksq

using namespace ksq;

extern "C" int ksq_w4a16_repack(int layout, const void* qweight, int zero_kind, const void* zeros,
                                const void* scales, int scale_dtype, size_t k, size_t n, size_t g, void* dst_weight,
                                void* dst_sz, void* stream) {
  int rc = validate(layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, g, dst_weight, dst_sz);
  if (rc != KSQ_OK) return rc;
  RepackArgs a{qweight, zeros, scales, static_cast<uint32_t*>(dst_weight), static_cast<uint32_t*>(dst_sz),
               k,       n,     g,      layout,                             zero_kind,
               scale_dtype};
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t words = k * n / 8, count = (k / g) * n;
  KSQ_REQUIRE((words + 255) / 256 < (1ull << 31), KSQ_ERR_UNSUPPORTED, "tensor too large for one launch");
  hipLaunchKernelGGL(repack_weight_kernel, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, a, words);
  hipLaunchKernelGGL(repack_sz_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s, a, count);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

extern "C" int ksq_w4a16_repack_host(int layout, const void* qweight, int zero_kind, const void* zeros,
                                     const void* scales, int scale_dtype, size_t k, size_t n, size_t g,
                                     void* dst_weight, void* dst_sz) {
  int rc = validate(layout, qweight, zero_kind, zeros, scales, scale_dtype, k, n, g, dst_weight, dst_sz);
  if (rc != KSQ_OK) return rc;
  RepackArgs a{qweight, zeros, scales, static_cast<uint32_t*>(dst_weight), static_cast<uint32_t*>(dst_sz),
               k,       n,     g,      layout,                             zero_kind,
               scale_dtype};
  const size_t words = k * n / 8, count = (k / g) * n;
  for (size_t i = 0; i < words; ++i) a.dst_weight[i] = build_weight_word(a, i);
  for (size_t i = 0; i < count; ++i) a.dst_sz[i] = build_sz_word(a, i);
  return KSQ_OK;
}
