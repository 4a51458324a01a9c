// FP8 e4m3 GEMM, large M (MFMA-bound): out[m,n] = T((sum_k a[m,k] * w[n,k]) * w_scale[n] * a_scale[m]).
//
// Workgroup tile 128 rows x 256 columns, four waves side by side, every wave 8 x 4 MFMA tiles of 16 x 16 with fp32
// accumulators, K = 128 per instruction (v_mfma_f32_16x16x128_f8f6f4, both operands OCP e4m3, no block scaling).
// Activations go through LDS in fragment order (one 128-row x 128-k stage = 16 KiB, double-buffered, one barrier per
// stage); weights are read by each wave for its own 64 columns straight from the [N][K] tensor, one stage ahead.
// Inside one instruction lane (r, j) holds bytes [16j, 16j+16) and [64+16j, 64+16j+16) of row r's 128-byte k
// slice -- the same assignment on both operands, so the products pair up, and every 128-bit load of a 16-lane
// group covers 64 contiguous bytes of a row.
#include "ksq_internal.h"

namespace ksq {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

struct Fp8PrefillArgs {
  const uint8_t* aq;  // [M][K]
  const uint8_t* wq;  // [N][K]
  const float* a_scale;
  const float* w_scale;
  void* out;
  int M, N, K, KS /* 128-byte k stages, rounded up */, mblocks, nblocks;
  int a_scale_per_row, w_scale_per_col;
};

constexpr int kBM = 128, kBN = 256, kMT = 8, kNT = 4;

template <typename T>
__device__ inline uint16_t out_bits(float v);
template <>
__device__ inline uint16_t out_bits<_Float16>(float v) {
  return __builtin_bit_cast(uint16_t, (_Float16)v);
}
template <>
__device__ inline uint16_t out_bits<__bf16>(float v) {
  return __builtin_bit_cast(uint16_t, (__bf16)v);
}

__device__ inline i32x8 join(u32x4 lo, u32x4 hi) {
  i32x8 v;
  v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
  v[4] = hi[0]; v[5] = hi[1]; v[6] = hi[2]; v[7] = hi[3];
  return v;
}

template <typename T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void fp8_prefill_kernel(Fp8PrefillArgs p) {
  constexpr int kStage = kMT * 2 * 64;  // 16-byte elements per activation stage
  constexpr int kEpiStride = 68;
  __shared__ u32x4 lds[2 * kStage];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, j = lane >> 4;

  const int total = gridDim.x, per_xcd = total >> 3;
  const int lid = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int mb = lid / p.nblocks, nb = lid - mb * p.nblocks;
  if (mb >= p.mblocks) return;
  const int m0 = mb * kBM, n0 = nb * kBN + wave * (kNT * 16);

  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.aq), 0, (int)((size_t)p.M * p.K), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.wq), 0, (int)((size_t)p.N * p.K), 0x00020000);
  // activation staging role: fragments f = 4 * wave + i (row tile f >> 1, half f & 1), this lane's 16 bytes
  unsigned a_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int f = 4 * wave + i, mt = f >> 1, h = f & 1;
    const int row = m0 + 16 * mt + r;
    a_off[i] = row < p.M ? (unsigned)row * p.K + 64 * h + 16 * j : 0x80000000u;
  }
  unsigned w_off[kNT];
#pragma unroll
  for (int t = 0; t < kNT; ++t) {
    const int row = n0 + 16 * t + r;
    w_off[t] = row < p.N ? (unsigned)row * p.K + 16 * j : 0x80000000u;
  }
  // a 16-byte piece at k offset ko inside a row is valid iff ko + 16 <= K (K % 16 == 0); otherwise it reads zero

  f32x4 acc[kMT][kNT];
#pragma unroll
  for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
    for (int t = 0; t < kNT; ++t) acc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 a_reg[4];
  u32x4 b_cur[kNT][2], b_nxt[kNT][2];
  auto load_a = [&](int s) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned ko = (unsigned)s * 128u + 64u * ((4 * wave + i) & 1) + 16u * j;
      a_reg[i] = __builtin_bit_cast(
          u32x4, __builtin_amdgcn_raw_buffer_load_b128(
                     rs_a, (ko + 16u <= (unsigned)p.K && a_off[i] != 0x80000000u) ? a_off[i] + s * 128u : 0x80000000u, 0,
                     0));
    }
  };
  auto write_a = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) lds[buf * kStage + (4 * wave + i) * 64 + lane] = a_reg[i];
  };
  auto load_b = [&](int s) {
#pragma unroll
    for (int t = 0; t < kNT; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const unsigned ko = (unsigned)s * 128u + 64u * h + 16u * j;
        b_nxt[t][h] = __builtin_bit_cast(
            u32x4,
            __builtin_amdgcn_raw_buffer_load_b128(
                rs_w, (ko + 16u <= (unsigned)p.K && w_off[t] != 0x80000000u) ? w_off[t] + s * 128u + 64u * h : 0x80000000u,
                0, 0));
      }
  };
  auto compute = [&](int buf) {
#pragma unroll
    for (int mt = 0; mt < kMT; ++mt) {
      const i32x8 af = join(lds[buf * kStage + (mt * 2 + 0) * 64 + lane], lds[buf * kStage + (mt * 2 + 1) * 64 + lane]);
#pragma unroll
      for (int t = 0; t < kNT; ++t)
        acc[mt][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af, join(b_cur[t][0], b_cur[t][1]), acc[mt][t], 0,
                                                                      0, 0, 0, 0, 0);
    }
  };

  load_b(0);
  load_a(0);
  write_a(0);
  load_a(1);
  for (int s = 0; s < p.KS; ++s) {
#pragma unroll
    for (int t = 0; t < kNT; ++t) {
      b_cur[t][0] = b_nxt[t][0];
      b_cur[t][1] = b_nxt[t][1];
    }
    __syncthreads();        // stage s is visible; everyone has finished reading the other buffer
    write_a((s + 1) & 1);   // stage s + 1
    load_a(s + 2);
    load_b(s + 1);
    compute(s & 1);
  }

  // ---- epilogue: scales, then a transpose through LDS so that every lane stores 16 contiguous bytes
  __syncthreads();
  float* epi = reinterpret_cast<float*>(lds) + wave * (16 * kEpiStride);
  uint16_t* out = static_cast<uint16_t*>(p.out);
  float ws[kNT];
#pragma unroll
  for (int t = 0; t < kNT; ++t) {
    const int col = n0 + 16 * t + r;
    ws[t] = p.w_scale[p.w_scale_per_col ? (col < p.N ? col : p.N - 1) : 0];
  }
#pragma unroll
  for (int mt = 0; mt < kMT; ++mt) {
#pragma unroll
    for (int t = 0; t < kNT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) epi[(4 * j + i) * kEpiStride + 16 * t + r] = acc[mt][t][i] * ws[t];
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      const int rr = (lane >> 3) + 8 * pass, cc = (lane & 7) * 8;
      const float* src = epi + rr * kEpiStride + cc;
      const int row = m0 + 16 * mt + rr, col = n0 + cc;
      const float as = p.a_scale[p.a_scale_per_row ? (row < p.M ? row : p.M - 1) : 0];
      u32x4 packed;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        packed[q] = (uint32_t)out_bits<T>(src[2 * q] * as) | ((uint32_t)out_bits<T>(src[2 * q + 1] * as) << 16);
      if (row < p.M && col + 8 <= p.N) *reinterpret_cast<u32x4*>(out + (size_t)row * p.N + col) = packed;
    }
  }
}

}  // namespace

bool fp8_prefill_supported(size_t m, size_t n, size_t k) {
  return m >= 128 && n % 8 == 0 && k % 16 == 0 && m * k < 0x7FFFFF00ull && n * k < 0x7FFFFF00ull;
}

int fp8_launch_prefill(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                       const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                       hipStream_t s) {
  KSQ_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15) == 0, KSQ_ERR_INVALID_ARGUMENT, "output must be 16-byte aligned");
  Fp8PrefillArgs a{};
  a.aq = static_cast<const uint8_t*>(act_q);
  a.wq = static_cast<const uint8_t*>(w_q);
  a.a_scale = act_scale;
  a.w_scale = w_scale;
  a.out = out;
  a.M = (int)m;
  a.N = (int)n;
  a.K = (int)k;
  a.KS = (int)((k + 127) / 128);
  a.mblocks = (int)((m + kBM - 1) / kBM);
  a.nblocks = (int)((n + kBN - 1) / kBN);
  a.a_scale_per_row = act_scale_count > 1;
  a.w_scale_per_col = w_scale_count > 1;
  const size_t total = ((size_t)a.mblocks * a.nblocks + 7) / 8 * 8;
  KSQ_REQUIRE(total < (1ull << 31), KSQ_ERR_UNSUPPORTED, "grid too large");
  if (out_dtype == KSQ_F16) hipLaunchKernelGGL(fp8_prefill_kernel<_Float16>, dim3((unsigned)total), dim3(256), 0, s, a);
  else hipLaunchKernelGGL(fp8_prefill_kernel<__bf16>, dim3((unsigned)total), dim3(256), 0, s, a);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

}  // namespace ksq
