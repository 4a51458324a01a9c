// W4A16 streaming kernel (decode regime, M <= 64; also the fallback for shapes the prefill kernel does not take).
//
// HBM-bound: every wave streams 1 KiB weight tiles (one 128-bit load per lane = the B operands of four
// 16x16x32 MFMAs), unpacks nibbles to exact small integers in registers, multiplies on the matrix cores and
// applies the group scale to the fp32 group sum.  Weights are read exactly once; activations come from L2.
//
//   fp16: B = (u - z) exactly, built with two bit operations and one packed subtract per register.
//   bf16: gfx950 has no packed bf16 arithmetic, so B = 128 + u (pure bit operations) and the bias is removed
//         per group in fp32:  acc += s * (P - (128 + z) * R),  R = row sums of the activations over the group,
//         obtained from one extra MFMA against a vector of ones (exact products, fp32 sums).
#include <type_traits>

#include "ksq_internal.h"

namespace ksq {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct StreamArgs {
  const u32x4* weight;  // [ntiles][KT][64]
  const uint32_t* sz;   // [ntiles][G][16]
  const void* act;      // [M][K]
  void* out;            // [M][N]
  f32x4* partial;       // [ksplit][mblocks][ntiles][MT][64]
  unsigned* counters;   // [mblocks * ngroups]
  int M, N, K, KT, G, ntiles, ngroups, ksplit;
};

template <typename T>
struct Ops;

template <>
struct Ops<_Float16> {
  static constexpr bool kBias = false;
  // word -> eight fp16 values u - z (exact); zc = z replicated as 0x000z000z
  static __device__ inline half8 unpack(uint32_t x, uint32_t zc) {
    const uint32_t c_lo = 0x64006400u | zc;         // 1024 + z
    const uint32_t c_hi = 0x54005400u | (zc << 4);  // 64 + z
    uint32_t y = x >> 8;
    uint32_t v0 = (x & 0x000F000Fu) | 0x64006400u;  // 1024 + u   (elements 0,1)
    uint32_t v1 = (x & 0x00F000F0u) | 0x54005400u;  // 64 + u     (elements 2,3)
    uint32_t v2 = (y & 0x000F000Fu) | 0x64006400u;  // elements 4,5
    uint32_t v3 = (y & 0x00F000F0u) | 0x54005400u;  // elements 6,7
    half2v r0 = __builtin_bit_cast(half2v, v0) - __builtin_bit_cast(half2v, c_lo);
    half2v r1 = __builtin_bit_cast(half2v, v1) - __builtin_bit_cast(half2v, c_hi);
    half2v r2 = __builtin_bit_cast(half2v, v2) - __builtin_bit_cast(half2v, c_lo);
    half2v r3 = __builtin_bit_cast(half2v, v3) - __builtin_bit_cast(half2v, c_hi);
    half8 o;
    o[0] = r0[0]; o[1] = r0[1]; o[2] = r1[0]; o[3] = r1[1];
    o[4] = r2[0]; o[5] = r2[1]; o[6] = r3[0]; o[7] = r3[1];
    return o;
  }
  static __device__ inline f32x4 mfma(u32x4 a, half8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), b, c, 0, 0, 0);
  }
  static __device__ inline float scale_to_float(uint32_t szw) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(szw & 0xFFFFu));
  }
  static __device__ inline uint16_t to_bits(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
};

template <>
struct Ops<__bf16> {
  static constexpr bool kBias = true;
  typedef bf16x8 frag;
  // word -> eight bf16 values 128 + u (exact)
  static __device__ inline bf16x8 unpack(uint32_t x, uint32_t) {
    u32x4 v;
    v[0] = (x & 0x000F000Fu) | 0x43004300u;
    v[1] = ((x >> 4) & 0x000F000Fu) | 0x43004300u;
    v[2] = ((x >> 8) & 0x000F000Fu) | 0x43004300u;
    v[3] = ((x >> 12) & 0x000F000Fu) | 0x43004300u;
    return __builtin_bit_cast(bf16x8, v);
  }
  static __device__ inline f32x4 mfma(u32x4 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), b, c, 0, 0, 0);
  }
  static __device__ inline bf16x8 ones() {
    u32x4 v = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    return __builtin_bit_cast(bf16x8, v);
  }
  static __device__ inline float scale_to_float(uint32_t szw) { return __builtin_bit_cast(float, szw << 16); }
  static __device__ inline uint16_t to_bits(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }
};

template <typename T, int MT, int NT, int GPT, int D>
__global__ __launch_bounds__(256) void w4a16_stream_kernel(StreamArgs p) {
  using O = Ops<T>;
  constexpr int DPG = 4 / GPT;  // MFMAs (32-k steps) per quantisation group inside one tile
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int c = lane & 15, j = lane >> 4;
  const int grp = blockIdx.x * 4 + wave;  // column-tile group of this wave
  if (grp >= p.ngroups) return;           // wave-uniform; the kernel has no block-level barrier
  const int nt0 = grp * NT;
  const int split = blockIdx.y, mblock = blockIdx.z;
  const int kt_begin = (int)(((long)p.KT * split) / p.ksplit);
  const int kt_end = (int)(((long)p.KT * (split + 1)) / p.ksplit);
  const int m0 = mblock * (16 * MT);

  // per-lane base pointers
  const uint16_t* act = static_cast<const uint16_t*>(p.act);
  const uint16_t* arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int row = m0 + 16 * mt + c;
    row = row < p.M ? row : p.M - 1;  // padding rows re-read the last row; their results are never stored
    arow[mt] = act + (size_t)row * p.K + 8 * j;
  }
  const u32x4* wbase[NT];
  const uint32_t* szbase[NT];
  bool tile_ok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    int nt = nt0 + t;
    tile_ok[t] = nt < p.ntiles;
    nt = tile_ok[t] ? nt : p.ntiles - 1;
    wbase[t] = p.weight + (size_t)nt * p.KT * 64 + lane;
    szbase[t] = p.sz + (size_t)nt * p.G * 16 + c;
  }

  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // register ring of D k-tiles: weights, scale/zero words and activation fragments are fetched D tiles ahead
  u32x4 wq[D][NT];
  uint32_t szq[D][NT][GPT];
  u32x4 aq[D][MT][4];

  auto fetch = [&](int slot, int kt) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      wq[slot][t] = __builtin_nontemporal_load(wbase[t] + (size_t)kt * 64);
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi) szq[slot][t][gi] = szbase[t][(size_t)(kt * GPT + gi) * 16];
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int d = 0; d < 4; ++d)
        aq[slot][mt][d] = *reinterpret_cast<const u32x4*>(arow[mt] + (size_t)kt * kTileK + 32 * d);
  };

  auto consume = [&](int slot) {
    f32x4 R[MT][GPT];
    if constexpr (O::kBias) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int gi = 0; gi < GPT; ++gi) {
          f32x4 r = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int dd = 0; dd < DPG; ++dd) r = O::mfma(aq[slot][mt][gi * DPG + dd], Ops<__bf16>::ones(), r);
          R[mt][gi] = r;
        }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi) {
        const uint32_t szw = szq[slot][t][gi];
        const uint32_t z = szw >> 16;
        const uint32_t zc = z | (z << 16);
        const float s = O::scale_to_float(szw);
        f32x4 P[MT];
#pragma unroll
        for (int dd = 0; dd < DPG; ++dd) {
          const int d = gi * DPG + dd;
          auto b = O::unpack(wq[slot][t][d], zc);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            P[mt] = O::mfma(aq[slot][mt][d], b, dd == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : P[mt]);
        }
        if constexpr (O::kBias) {
          const float cz = -(128.0f + (float)z);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[mt][t][i] += s * (cz * R[mt][gi][i] + P[mt][i]);
        } else {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[mt][t][i] += s * P[mt][i];
        }
      }
    }
  };

  // Software pipeline.  The hardware retires loads in order and the compiler can only keep later prefetches in
  // flight across a wait when the number of loads issued after it is known statically, so every stage below is
  // straight-line code: a steady-state loop whose D fetches are all unconditional, and a tail specialised at
  // compile time on the remainder.
  const int ntile = kt_end - kt_begin;
  auto tail = [&](auto rc, int kt) {  // D tiles in flight in slots 0..D-1, R more to fetch from kt + D
    constexpr int R = decltype(rc)::value;
#pragma unroll
    for (int i = 0; i < D; ++i) {
      consume(i);
      if (i < R) fetch(i, kt + D + i);  // i and R are constants after unrolling
    }
#pragma unroll
    for (int i = 0; i < R; ++i) consume(i);
  };
  auto small = [&](auto nc) {  // fewer than D tiles in total
    constexpr int NS = decltype(nc)::value;
#pragma unroll
    for (int i = 0; i < NS; ++i) fetch(i, kt_begin + i);
#pragma unroll
    for (int i = 0; i < NS; ++i) consume(i);
  };
  if (ntile >= D) {
#pragma unroll
    for (int i = 0; i < D; ++i) fetch(i, kt_begin + i);
    int kt = kt_begin;
    for (int rounds = ntile / D; rounds >= 2; --rounds, kt += D) {
#pragma unroll
      for (int i = 0; i < D; ++i) {
        consume(i);
        fetch(i, kt + D + i);
      }
    }
    switch (ntile % D) {
      case 0: tail(std::integral_constant<int, 0>{}, kt); break;
      case 1: tail(std::integral_constant<int, (1 < D ? 1 : 0)>{}, kt); break;
      case 2: tail(std::integral_constant<int, (2 < D ? 2 : 0)>{}, kt); break;
      default: tail(std::integral_constant<int, (3 < D ? 3 : 0)>{}, kt); break;
    }
  } else {
    switch (ntile) {
      case 0: break;
      case 1: small(std::integral_constant<int, 1>{}); break;
      case 2: small(std::integral_constant<int, (2 < D ? 2 : 1)>{}); break;
      default: small(std::integral_constant<int, (3 < D ? 3 : 1)>{}); break;
    }
  }

  // ---- epilogue: lane (c, j) holds column 16*nt + c, rows m0 + 16*mt + 4*j + i
  uint16_t* out = static_cast<uint16_t*>(p.out);
  auto store_out = [&](int mt, int t, f32x4 v) {
    if (!tile_ok[t]) return;
    const int col = (nt0 + t) * 16 + c;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = m0 + 16 * mt + 4 * j + i;
      if (row < p.M) out[(size_t)row * p.N + col] = O::to_bits(v[i]);
    }
  };

  if (p.ksplit == 1) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < NT; ++t) store_out(mt, t, acc[mt][t]);
    return;
  }

  // split-K fix-up: every split parks its fp32 tiles, the last one to arrive adds them in split order
  // (deterministic) and writes the result.  Counters return to zero for the next launch.
  const size_t split_stride = (size_t)gridDim.z * p.ntiles * MT * 64;
  auto pidx = [&](int sp, int mt, int t) {
    int nt = nt0 + t;
    nt = nt < p.ntiles ? nt : p.ntiles - 1;
    return (size_t)sp * split_stride + (((size_t)mblock * p.ntiles + nt) * MT + mt) * 64 + lane;
  };
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t)
      if (tile_ok[t]) p.partial[pidx(split, mt, t)] = acc[mt][t];
  __threadfence();
  unsigned* ctr = p.counters + (size_t)mblock * p.ngroups + grp;
  unsigned arrived = 0;
  if (lane == 0) arrived = atomicAdd(ctr, 1u);
  arrived = __builtin_amdgcn_readfirstlane(arrived);
  if (arrived != (unsigned)(p.ksplit - 1)) return;
  __threadfence();
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (!tile_ok[t]) continue;
      f32x4 sum = {0.f, 0.f, 0.f, 0.f};
      for (int sp = 0; sp < p.ksplit; ++sp) {
        f32x4 v = p.partial[pidx(sp, mt, t)];
        sum += v;
      }
      store_out(mt, t, sum);
    }
  if (lane == 0) atomicExch(ctr, 0u);
}

template <typename T, int MT, int NT, int GPT>
void launch_one(const StreamArgs& a, dim3 grid, hipStream_t s) {
  constexpr int D = MT == 1 ? 4 : (MT == 2 ? 3 : 2);
  hipLaunchKernelGGL((w4a16_stream_kernel<T, MT, NT, GPT, D>), grid, dim3(256), 0, s, a);
}

template <typename T, int MT, int NT>
void launch_gpt(int gpt, const StreamArgs& a, dim3 grid, hipStream_t s) {
  if (gpt == 1) launch_one<T, MT, NT, 1>(a, grid, s);
  else launch_one<T, MT, NT, 2>(a, grid, s);
}

template <typename T, int MT>
void launch_nt(int nt, int gpt, const StreamArgs& a, dim3 grid, hipStream_t s) {
  if (nt == 1) launch_gpt<T, MT, 1>(gpt, a, grid, s);
  else launch_gpt<T, MT, 2>(gpt, a, grid, s);
}

template <typename T>
void launch_mt(int mt, int nt, int gpt, const StreamArgs& a, dim3 grid, hipStream_t s) {
  switch (mt) {
    case 1: launch_nt<T, 1>(nt, gpt, a, grid, s); break;
    case 2: launch_nt<T, 2>(nt, gpt, a, grid, s); break;
    case 3: launch_nt<T, 3>(nt, gpt, a, grid, s); break;
    default: launch_nt<T, 4>(nt, gpt, a, grid, s); break;
  }
}

}  // namespace

int w4a16_launch_stream(int dtype, const W4Plan& plan, void* out, const void* act, const void* weight,
                        const void* sz, size_t m, size_t n, size_t k, size_t g, void* workspace, hipStream_t s) {
  StreamArgs a{};
  a.weight = static_cast<const u32x4*>(weight);
  a.sz = static_cast<const uint32_t*>(sz);
  a.act = act;
  a.out = out;
  a.partial = static_cast<f32x4*>(workspace);
  a.M = (int)m;
  a.N = (int)n;
  a.K = (int)k;
  a.KT = (int)(k / kTileK);
  a.G = (int)(k / g);
  a.ntiles = (int)(n / kTileN);
  a.ngroups = (a.ntiles + plan.NT - 1) / plan.NT;
  a.ksplit = plan.ksplit;
  a.counters = nullptr;
  if (plan.ksplit > 1) {
    KSQ_REQUIRE(workspace != nullptr, KSQ_ERR_WORKSPACE, "split-K planned without a workspace");
    KSQ_REQUIRE((size_t)a.ngroups * plan.mblocks <= (size_t)kCountersPerSlot, KSQ_ERR_UNSUPPORTED,
                "too many tiles for the split-K counters");
    a.counters = counter_slot_device_ptr();
    if (!a.counters) return KSQ_ERR_HIP;
  }
  KSQ_REQUIRE(plan.mblocks <= 65535 && plan.ksplit <= 65535, KSQ_ERR_UNSUPPORTED, "grid too large");
  dim3 grid((unsigned)((a.ngroups + 3) / 4), (unsigned)plan.ksplit, (unsigned)plan.mblocks);
  const int gpt = (int)(kTileK / g);
  if (dtype == KSQ_F16) launch_mt<_Float16>(plan.MT, plan.NT, gpt, a, grid, s);
  else launch_mt<__bf16>(plan.MT, plan.NT, gpt, a, grid, s);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

}  // namespace ksq
