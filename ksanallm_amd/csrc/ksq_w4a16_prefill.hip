// W4A16 prefill kernel (large M, MFMA-bound).
//
// Workgroup tile 128 rows x 256 or 512 columns, four or eight waves side by side: every wave owns a 128 x 64 output
// tile (8 x 4 MFMA tiles of 16 x 16, fp32 accumulators in registers).  Activations go from global memory straight
// into LDS (no staging registers), 128 k at a time, two stages, one barrier per stage, in a layout that keeps both
// the global reads (four lanes per 64 contiguous bytes) and the LDS reads (no bank conflicts) at full rate.
// Weights never touch LDS: each wave
// reads its own column tiles straight from the fragment-order buffer (one 128-bit load per lane = the B operands of
// four 16x16x32 MFMAs), one k tile ahead, and dequantises them in registers once per 128 rows:
//   w = T((u - z) * s), rounded once -- the reference's dequantise-then-MMA semantics
//   (LK/cutlass_extensions/gemm/warp/mma_tensorop_dequantizer.h:206-245, 368-394), with no second rounding.
//   bit operations to 1024 + u / 64 + u, packed fp16 subtract of (bias + z) (exact), packed multiply by s.
// The matrix cores always run in fp16.  Rounding a dequantised weight to bf16 (8 significant bits) would cost up to
// 2^-8 per weight -- together with the bf16 rounding of the output more than the 1e-2 bound on the maximum relative
// error allows -- so bf16 activations are first re-encoded, exactly, as fp16 with one power-of-two exponent per row
// (a bf16 significand fits into fp16; the row exponent keeps every row inside the fp16 range whatever its
// magnitude); the row factor 2^e is applied to the fp32 accumulators in the epilogue.  The bf16 group scales are
// converted to fp16 after division by a power of two per column (the column's largest scale exponent, kept in
// every scale/zero word by the repack), which the epilogue puts back, so scales far outside the fp16 range work.
// Workgroups are numbered so that those sharing a row block of the activations run on the same XCD (own L2).
#include <cstdlib>
#include <type_traits>

#include "ksq_internal.h"
#include "ksq_epilogue.h"
#include "ksq_w4a16_ops.h"

namespace ksq {
namespace {

using namespace w4;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_ptr;

struct PrefillArgs {
  const void* weight;
  const void* sz;
  const void* act;
  void* out;
  const float* row_scale;  // bf16 route: 2^e per row of the re-encoded activations
  int M, N, K, KT, G, ntiles, mblocks, nblocks;
  int ksplit;          // grid.y: K split over workgroups
  float* partial;      // [ksplit][mblocks * rows per block][N] fp32, ksplit > 1 only
  Epilogue epi;
};

constexpr int kBM = 128;             // rows per workgroup
constexpr int kMT = 8;  // 16-row MFMA tiles per wave (the column tiles per wave are a template parameter)

// bf16 [M][K] -> fp16 [M][K] * 2^-e[row] (exact: power-of-two shift of an 8-bit significand into 11 bits), with
// e[row] chosen so that the row maximum lands at 2^14; row_scale[row] = 2^e.  One workgroup per row; the row stays
// in registers between the maximum and the conversion (R chunks of eight elements per lane), so it is read once.
template <int R>
__global__ __launch_bounds__(256) void bf16_rows_to_f16_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                               float* __restrict__ row_scale, int K) {
  __shared__ float smem[4];
  const size_t row = blockIdx.x;
  const u32x4* s = reinterpret_cast<const u32x4*>(src + row * K);
  u32x4* d = reinterpret_cast<u32x4*>(dst + row * K);
  const int nchunks = K / 8;  // K is a multiple of 128
  u32x4 v[R];
  float mx = 0.f;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int ch = threadIdx.x + i * 256;
    v[i] = ch < nchunks ? s[ch] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float lo = __builtin_fabsf(__builtin_bit_cast(float, v[i][q] << 16));
      const float hi = __builtin_fabsf(__builtin_bit_cast(float, v[i][q] & 0xFFFF0000u));
      mx = (lo == lo && lo < __builtin_inff()) ? __builtin_fmaxf(mx, lo) : mx;  // NaN / Inf do not set the exponent
      mx = (hi == hi && hi < __builtin_inff()) ? __builtin_fmaxf(mx, hi) : mx;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = __builtin_fmaxf(mx, __shfl_xor(mx, off));
  if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = __builtin_fmaxf(__builtin_fmaxf(smem[0], smem[1]), __builtin_fmaxf(smem[2], smem[3]));
  int e = 0;
  if (mx > 0.f) e = (int)((__builtin_bit_cast(uint32_t, mx) >> 23) & 0xFF) - 127 - 14;
  e = e < -100 ? -100 : e;  // keeps 2^-e and 2^e normal floats; rows that small lose bits that no output can show
  const float down = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);  // 2^-e, e in [-100, 113]
  const float up = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
  if (threadIdx.x == 0) row_scale[row] = up;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int ch = threadIdx.x + i * 256;
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float lo = __builtin_bit_cast(float, v[i][q] << 16) * down;
      const float hi = __builtin_bit_cast(float, v[i][q] & 0xFFFF0000u) * down;
      o[q] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) |
             ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
    }
    if (ch < nchunks) d[ch] = o;
  }
}

// the same for rows longer than 32768 elements: two passes over global memory, eight elements per load
__global__ __launch_bounds__(256) void bf16_rows_to_f16_long_kernel(const uint16_t* __restrict__ src,
                                                                    uint16_t* __restrict__ dst,
                                                                    float* __restrict__ row_scale, int K) {
  __shared__ float smem[4];
  const size_t row = blockIdx.x;
  const u32x4* s = reinterpret_cast<const u32x4*>(src + row * K);
  u32x4* d = reinterpret_cast<u32x4*>(dst + row * K);
  const int nchunks = K / 8;
  float mx = 0.f;
  for (int ch = threadIdx.x; ch < nchunks; ch += 256) {
    const u32x4 v = s[ch];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float lo = __builtin_fabsf(__builtin_bit_cast(float, v[q] << 16));
      const float hi = __builtin_fabsf(__builtin_bit_cast(float, v[q] & 0xFFFF0000u));
      mx = (lo == lo && lo < __builtin_inff()) ? __builtin_fmaxf(mx, lo) : mx;
      mx = (hi == hi && hi < __builtin_inff()) ? __builtin_fmaxf(mx, hi) : mx;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = __builtin_fmaxf(mx, __shfl_xor(mx, off));
  if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = mx;
  __syncthreads();
  mx = __builtin_fmaxf(__builtin_fmaxf(smem[0], smem[1]), __builtin_fmaxf(smem[2], smem[3]));
  int e = 0;
  if (mx > 0.f) e = (int)((__builtin_bit_cast(uint32_t, mx) >> 23) & 0xFF) - 127 - 14;
  e = e < -100 ? -100 : e;  // keeps 2^-e and 2^e normal floats; rows that small lose bits that no output can show
  const float down = __builtin_bit_cast(float, (uint32_t)(127 - e) << 23);
  const float up = __builtin_bit_cast(float, (uint32_t)(127 + e) << 23);
  if (threadIdx.x == 0) row_scale[row] = up;
  for (int ch = threadIdx.x; ch < nchunks; ch += 256) {
    const u32x4 v = s[ch];
    u32x4 o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float lo = __builtin_bit_cast(float, v[q] << 16) * down;
      const float hi = __builtin_bit_cast(float, v[q] & 0xFFFF0000u) * down;
      o[q] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)lo) |
             ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)hi) << 16);
    }
    d[ch] = o;
  }
}

// CT = column tiles per wave: 4 (64 columns: tiles of 256 or 512 columns) or 3 (48 columns: 192 or 384), for
// widths whose number of tiles falls better on the compute units (a partly filled last round costs a full one);
// 2 or 1 (tiles of 128 or 64 columns) where a single row block has to be spread over the device (65 to 128 rows).
template <typename T, int GPT, int NW, int KG = 1, int CT = 4>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void w4a16_prefill_kernel(PrefillArgs p) {
  static_assert(NW == 4 || NW == 8, "four or eight waves side by side");
  static_assert(CT >= 1 && CT <= 4, "one to four column tiles per wave");
  // KG = 2: two groups of four waves on the same 128 x 256 tile, the first on the even k tiles, the second on the
  // odd ones, each with its own pair of activation stages; the second group's accumulators reach the first through
  // LDS at the end.  For grids that put one workgroup on a CU: two waves per SIMD instead of one.
  static_assert(KG == 1 || (KG == 2 && NW == 4), "two k groups of four waves");
  constexpr int kFPW = 32 / NW;  // activation fragments of a stage that one wave brings in
  using O = Ops<_Float16>;  // the matrix cores run in fp16 for both element types
  using DQ = Dequant<T>;
  constexpr bool kBF16 = sizeof(T) == 2 && !__is_same(T, _Float16);
  constexpr int kStage = kMT * 4 * 64;  // 16-byte elements per activation stage (128 rows x 128 k) = 32 KiB
  constexpr int kEpiStride = 68;        // floats per row of the epilogue transpose (2-way conflicts at worst)
  // two activation stages as two separate objects: loads into one are then known not to alias reads of the other
  __shared__ u32x4 lds_a0[kStage];
  __shared__ u32x4 lds_a1[kStage];
  __shared__ u32x4 lds_a2[KG == 2 ? kStage : 1];
  __shared__ u32x4 lds_a3[KG == 2 ? kStage : 1];

  const int lane = threadIdx.x & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kg = KG == 2 ? wave_all >> 2 : 0;           // k group of this wave
  const int wave = KG == 2 ? wave_all & 3 : wave_all;  // its place among the waves side by side
  const int c = lane & 15, j = lane >> 4;

  int mb, nb;
  if (!tile_of(tile_logical_id(blockIdx.x, gridDim.x), p.mblocks, p.nblocks, &mb, &nb)) return;  // rounding of the grid
  const int m0 = mb * kBM;
  const int nt0 = (nb * NW + wave) * CT;

  __amdgpu_buffer_rsrc_t rs_w[CT], rs_sz[CT];
#pragma unroll
  for (int t = 0; t < CT; ++t) {
    const int nt = nt0 + t;
    const bool ok = nt < p.ntiles;
    const size_t ntc = ok ? (size_t)nt : 0;
    rs_w[t] = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(static_cast<const char*>(p.weight) + ntc * p.KT * 1024), 0, ok ? p.KT * 1024 : 0, 0x00020000);
    rs_sz[t] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(static_cast<const char*>(p.sz) + ntc * p.G * 64), 0,
                                                 ok ? p.G * 64 : 0, 0x00020000);
  }
  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.act), 0, (int)((size_t)p.M * p.K * 2), 0x00020000);
  // Activation stage in LDS: 32 blocks of 1 KiB, block (mt, q) = rows 4q .. 4q+3 of row tile mt, all 256 bytes of
  // the k tile.  A block is one global -> LDS load instruction (lane l lands at l * 16), with lane l on row l/4 % 4,
  // 32-k step l / 16 and 16-byte piece (l % 4) ^ q: every aligned group of four lanes reads 64 contiguous bytes of
  // one row (the memory pipeline then takes four lanes per clock instead of one), and the xor by q makes the 16
  // rows that one group of 16 lanes reads back for an MFMA operand (piece j of rows 0..15) fall on 16 different
  // bank groups.  Rows past M repeat row M - 1 (their results are never stored).  This wave brings in blocks
  // kFPW * wave .. kFPW * wave + kFPW - 1.
  unsigned a_off[8];  // kFPW of them in use: block i of this wave
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a_off[i] = 0u;
    if (i < kFPW) {
      const int blk = kFPW * wave + i, mt = blk >> 2, q = blk & 3;
      int row = m0 + 16 * mt + 4 * q + ((lane >> 2) & 3);
      row = row < p.M ? row : p.M - 1;
      a_off[i] = (unsigned)row * p.K * 2u + 64u * (lane >> 4) + 16u * ((lane & 3) ^ q);
    }
  }
  // where lane (c, j) finds piece j of row c of a (row tile, 32-k step) inside the stage, apart from
  // row tile * 256 + step * 16 (in 16-byte units)
  const int a_lane = (c >> 2) * 64 + (c & 3) * 4 + (j ^ (c >> 2));
  const unsigned w_voff = lane * 16u, sz_voff = c * 4u;

  f32x4 acc[kMT][CT];
#pragma unroll
  for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
    for (int t = 0; t < CT; ++t) acc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  struct BTile {
    u32x4 w[CT];
    uint32_t sz[CT][GPT];
  };
  BTile b0, b1;

  // The loads of the next k tile are issued a few at a time between the matrix instructions of the current one
  // (a burst of 16 memory instructions would hold the wave in the issue queue of the memory pipeline, and the
  // matrix cores with it).  Part q = 0..3 of a tile's loads, in four items: activation blocks (global -> LDS, no
  // registers; two with four waves, one with eight), the weight fragment of column tile q, its scale/zero words
  // (past the last k tile the resources return zero).
  auto load_item = [&](u32x4* buf, BTile& b, int kt, int q, int item) {
    if (item < 2) {
      if (item < kFPW / 4) {
        const int i = kFPW / 4 * q + item;
        // the scalar offset is not range-checked: a prefetch past K re-reads the last k tile (nobody uses it)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(buf + (kFPW * wave + i) * 64), 16, a_off[i],
                                                 (kt < p.KT ? kt : p.KT - 1) * 256, 0, 0);
      }
    } else if (q >= CT) {  // fewer than four column tiles per wave: the other parts carry activations only
    } else if (item == 2) {
      b.w[q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w[q], w_voff + kt * 1024u, 0, 0));
    } else {
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi)
        b.sz[q][gi] = __builtin_amdgcn_raw_buffer_load_b32(rs_sz[q], sz_voff + (kt * GPT + gi) * 64u, 0, 0);
    }
  };
  auto load_part = [&](u32x4* buf, BTile& b, int kt, int q) {
#pragma unroll
    for (int item = 0; item < 4; ++item) load_item(buf, b, kt, q, item);
  };

  uint32_t m_lo = Ops<_Float16>::kMaskLo, m_hi = Ops<_Float16>::kMaskHi, g_lo = Ops<_Float16>::kMagicLo,
           g_hi = Ops<_Float16>::kMagicHi;
  KSQ_PIN_SGPR(m_lo);
  KSQ_PIN_VGPR(g_lo);
  KSQ_PIN_VGPR(g_hi);
  KSQ_PIN_VGPR(m_hi);

  // Activation fragments are read from LDS four at a time (half of the row tiles of one 32-k step), one half ahead
  // of the matrix instructions that use them, so that the LDS latency hides behind 16 MFMAs.
  auto read_half = [&](u32x4 (&a)[4], const u32x4* buf, int ks, int h) {
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = buf[(4 * h + i) * 256 + ks * 16 + a_lane];
  };
  auto mfma_row = [&](const u32x4& a, const u32x4 (&b)[CT], int mt) {
#pragma unroll
    for (int t = 0; t < CT; ++t) acc[mt][t] = O::mfma(a, b[t], acc[mt][t]);
  };
  // One k tile.  On entry everything in flight (this tile's activations and weights) has landed and is visible to
  // the whole workgroup, and every wave is done with the other buffer.
  auto step = [&](const u32x4* cur, u32x4* nxt, const BTile& bt, BTile& bn, int kt) __attribute__((always_inline)) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    u32x4 a0[4], a1[4];
    read_half(a0, cur, 0, 0);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      u32x4 b[CT];
#pragma unroll
      for (int t = 0; t < CT; ++t) {
        const typename DQ::Consts k = DQ::prepare(bt.sz[t][GPT == 2 ? (ks >> 1) : 0]);
        b[t] = DQ::run(bt.w[t][ks], k, m_lo, m_hi, g_lo, g_hi);
      }
      read_half(a1, cur, ks, 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        mfma_row(a0[i], b, i);
        if (ks < 2) load_item(nxt, bn, kt + KG, 2 * ks, i);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (ks < 3) read_half(a0, cur, ks + 1, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        mfma_row(a1[i], b, 4 + i);
        if (ks < 2) load_item(nxt, bn, kt + KG, 2 * ks + 1, i);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // k tiles of this workgroup: all of them, or (K split over grid.y, for grids that would leave most compute units
  // without a tile) the range of its split, whose raw fp32 tile goes to the workspace for the reduction kernel
  int kt0, kt1;
  split_range(p.KT, blockIdx.y, p.ksplit, &kt0, &kt1);
  // The k loop of one k group over its pair of stages: k tiles kt0 + kg, kt0 + kg + KG, ...  Both groups make the same
  // number of steps (a step is one barrier); with an odd number of k tiles the second group's last step has no tile.
  // (everything here has to be inlined: a call would put the accumulators, captured by reference, into memory)
  auto k_loop = [&](u32x4* s0, u32x4* s1) __attribute__((always_inline)) {
    auto run = [&](const u32x4* cur, u32x4* nxt, const BTile& bt, BTile& bn, int kt) __attribute__((always_inline)) {
      if (KG == 1 || kt < kt1) {
        step(cur, nxt, bt, bn, kt);
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_s_barrier();
      }
    };
#pragma unroll
    for (int q = 0; q < 4; ++q) load_part(s0, b0, kt0 + kg, q);
    const int nsteps = (kt1 - kt0 + KG - 1) / KG;
    int st = 0;
    for (; st + 2 <= nsteps; st += 2) {
      run(s0, s1, b0, b1, kt0 + kg + st * KG);
      run(s1, s0, b1, b0, kt0 + kg + (st + 1) * KG);
    }
    if (st < nsteps) run(s0, s1, b0, b1, kt0 + kg + st * KG);
  };
  if (KG == 1 || kg == 0) k_loop(lds_a0, lds_a1);
  else k_loop(lds_a2, lds_a3);

  // ---- epilogue: transpose each 16-row slab through LDS so that every lane stores 16 contiguous bytes
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the last (unused) prefetch must not land on top of the transposes
  __syncthreads();
  float* epi = reinterpret_cast<float*>(wave < 4 ? lds_a0 : lds_a1) + (wave & 3) * (16 * kEpiStride);  // 4352 B
  if constexpr (KG == 2) {
    // wave w of the second group parks its accumulators in stage w; wave w of the first group, which owns the same
    // output tiles, adds them to its own and then uses that stage, and no other, for its transposes
    f32x4* park = reinterpret_cast<f32x4*>(wave == 0 ? lds_a0 : wave == 1 ? lds_a1 : wave == 2 ? lds_a2 : lds_a3);
    if (kg == 1) {
#pragma unroll
      for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
        for (int t = 0; t < CT; ++t) park[(mt * CT + t) * 64 + lane] = acc[mt][t];
    }
    __syncthreads();
    if (kg == 1) return;
#pragma unroll
    for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
      for (int t = 0; t < CT; ++t) acc[mt][t] += park[(mt * CT + t) * 64 + lane];
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): all of them read before the transposes overwrite the stage
    epi = reinterpret_cast<float*>(park);
  }
  uint16_t* out = static_cast<uint16_t*>(p.out);
  const int ncol0 = nt0 * 16;
  float cf[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};  // bf16 scales: 2^E of this lane's eight columns
  if constexpr (kBF16) {
    const int col = ncol0 + (lane & 7) * 8;
    if (col + 8 <= p.N && (lane & 7) * 8 < 16 * CT) column_factors(p.sz, p.G, col, cf);
  }
#pragma unroll
  for (int mt = 0; mt < kMT; ++mt) {
#pragma unroll
    for (int t = 0; t < CT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) epi[(4 * j + i) * kEpiStride + 16 * t + c] = acc[mt][t][i];
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      const int rr = (lane >> 3) + 8 * pass, cc = (lane & 7) * 8;
      const float* src = epi + rr * kEpiStride + cc;
      const int row = m0 + 16 * mt + rr, col = ncol0 + cc;
      if (p.ksplit > 1) {  // the fp32 segment of this split; the reduction kernel finishes it
        if (row < p.M && col + 8 <= p.N && cc < 16 * CT) {
          f32x4* dst = reinterpret_cast<f32x4*>(p.partial + ((size_t)blockIdx.y * p.mblocks * kBM + row) * p.N + col);
          dst[0] = f32x4{src[0], src[1], src[2], src[3]};
          dst[1] = f32x4{src[4], src[5], src[6], src[7]};
        }
        continue;
      }
      float rs = 1.f;
      if constexpr (kBF16) rs = p.row_scale[row < p.M ? row : p.M - 1];
      float vals[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) vals[q] = src[q] * rs * cf[q];
      epi_store_row8_wave<T>(p.epi, out, vals, row, col, p.N, row < p.M && col + 8 <= p.N && cc < 16 * CT, row < p.M, lane);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
  }
}

// The same GEMM for medium M, where 128-row tiles leave most CUs without work: workgroup tile 64 rows x 256 columns
// (four waves, every wave 4 x 4 MFMA tiles, two workgroups per CU) and, because such grids run one or two waves
// per SIMD with nobody to hide a memory round trip behind, everything three k tiles ahead: activations global -> LDS
// over four stages of 16 KiB (four separate objects), weights in a ring of four register tiles.
// What bounds such a grid is the length of the k loop (a k tile takes most of a microsecond however little work it
// carries), so while the output tiles alone leave workgroup slots empty K is split over grid.y: every split stores
// its fp32 partial tile into the workspace with plain stores and a second, ordinary kernel adds the splits in order
// (deterministic) and applies the epilogue.  Tens of megabytes of partial tiles through the agent-scope atomics that
// the decode kernels hand their few partial tiles over with were measured several times slower than the GEMM itself.
template <typename T, int GPT, int KNT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void w4a16_mid_kernel(PrefillArgs p) {
  using O = Ops<_Float16>;
  using DQ = Dequant<T>;
  constexpr bool kBF16 = sizeof(T) == 2 && !__is_same(T, _Float16);
  constexpr int kRows = 4;              // row tiles per workgroup
  constexpr int kStage = kRows * 4 * 64;  // 16-byte elements per activation stage (64 rows x 128 k) = 16 KiB
  constexpr int kEpiStride = 68;
  constexpr int kLoads = 4 + KNT * (1 + GPT);  // memory instructions per k tile and wave
  __shared__ u32x4 lds_a0[kStage];
  __shared__ u32x4 lds_a1[kStage];
  __shared__ u32x4 lds_a2[kStage];
  __shared__ u32x4 lds_a3[kStage];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, j = lane >> 4;

  int mb, nb;
  if (!tile_of(tile_logical_id(blockIdx.x, gridDim.x), p.mblocks, p.nblocks, &mb, &nb)) return;  // rounding of the grid
  const int m0 = mb * (16 * kRows);
  const int nt0 = (nb * 4 + wave) * KNT;

  __amdgpu_buffer_rsrc_t rs_w[KNT], rs_sz[KNT];
#pragma unroll
  for (int t = 0; t < KNT; ++t) {
    const int nt = nt0 + t;
    const bool ok = nt < p.ntiles;
    const size_t ntc = ok ? (size_t)nt : 0;
    rs_w[t] = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(static_cast<const char*>(p.weight) + ntc * p.KT * 1024), 0, ok ? p.KT * 1024 : 0, 0x00020000);
    rs_sz[t] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(static_cast<const char*>(p.sz) + ntc * p.G * 64), 0,
                                                 ok ? p.G * 64 : 0, 0x00020000);
  }
  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.act), 0, (int)((size_t)p.M * p.K * 2), 0x00020000);
  // activation blocks as in the 128-row kernel: block (mt, q) = rows 4q .. 4q+3 of row tile mt; this wave brings in
  // the four blocks of row tile `wave`
  unsigned a_off[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    int row = m0 + 16 * wave + 4 * q + ((lane >> 2) & 3);
    row = row < p.M ? row : p.M - 1;
    a_off[q] = (unsigned)row * p.K * 2u + 64u * (lane >> 4) + 16u * ((lane & 3) ^ q);
  }
  const int a_lane = (c >> 2) * 64 + (c & 3) * 4 + (j ^ (c >> 2));
  const unsigned w_voff = lane * 16u, sz_voff = c * 4u;

  f32x4 acc[kRows][KNT];
#pragma unroll
  for (int mt = 0; mt < kRows; ++mt)
#pragma unroll
    for (int t = 0; t < KNT; ++t) acc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  struct BTile {
    u32x4 w[KNT];
    uint32_t sz[KNT][GPT];
  };
  BTile b0, b1, b2, b3;

  // item 0..3 of part q: activation block q, weight fragment of column tile q, its scale/zero words (two items of
  // which the second is empty when a k tile is one group)
  auto load_item = [&](u32x4* buf, BTile& b, int kt, int q, int item) {
    if (item == 0) {
      // the scalar offset is not range-checked: a prefetch past K re-reads the last k tile (nobody uses it)
      const int kta = kt < p.KT ? kt : p.KT - 1;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(buf + (4 * wave + q) * 64), 16, a_off[q], kta * 256, 0, 0);
    } else if (q < KNT) {
      if (item == 1)
        b.w[q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w[q], w_voff + kt * 1024u, 0, 0));
      else if (item - 2 < GPT)
        b.sz[q][item - 2] = __builtin_amdgcn_raw_buffer_load_b32(rs_sz[q], sz_voff + (kt * GPT + item - 2) * 64u, 0, 0);
    }
  };
  auto load_tile = [&](u32x4* buf, BTile& b, int kt) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
#pragma unroll
      for (int item = 0; item < 4; ++item) load_item(buf, b, kt, q, item);
      __builtin_amdgcn_sched_barrier(0);  // keep the issue order: the waits below count on it
    }
  };

  uint32_t m_lo = Ops<_Float16>::kMaskLo, m_hi = Ops<_Float16>::kMaskHi, g_lo = Ops<_Float16>::kMagicLo,
           g_hi = Ops<_Float16>::kMagicHi;
  KSQ_PIN_SGPR(m_lo);
  KSQ_PIN_VGPR(g_lo);
  KSQ_PIN_VGPR(g_hi);
  KSQ_PIN_VGPR(m_hi);

  auto read_step = [&](u32x4 (&a)[kRows], const u32x4* buf, int ks) {
#pragma unroll
    for (int mt = 0; mt < kRows; ++mt) a[mt] = buf[mt * 256 + ks * 16 + a_lane];
  };
  // One k tile.  On entry all loads but those of the two youngest tiles have landed; after the barrier tile kt is
  // visible to every wave and every wave is done with the buffer that tile kt + 3 goes into.
  // In the steady state (`steady`) the wait leaves the loads of the two youngest tiles in flight and the step issues
  // those of tile kt + 3; the last steps of a workgroup issue nothing and wait for everything.
  auto step = [&](const u32x4* cur, u32x4* dst, const BTile& bt, BTile& bn, int kt, auto steady_tag) {
    constexpr bool kSteady = decltype(steady_tag)::value;
    constexpr int kCount = kSteady ? 2 * kLoads : 0;  // vmcnt: low four bits, high two bits in 15:14
    __builtin_amdgcn_s_waitcnt(0x0F70 | (kCount & 15) | ((kCount >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    u32x4 a0[kRows], a1[kRows];
    read_step(a0, cur, 0);
    // The dequantisation of 32-k step ks + 1 is spread between the MFMAs of step ks (one column tile after each row
    // of MFMAs): a wave that has a SIMD to itself then runs the vector ALU under the matrix pipeline instead of
    // before it.
    u32x4 b[2][KNT];
#pragma unroll
    for (int t = 0; t < KNT; ++t) {
      const typename DQ::Consts k = DQ::prepare(bt.sz[t][0]);
      b[0][t] = DQ::run(bt.w[t][0], k, m_lo, m_hi, g_lo, g_hi);
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks < 3) read_step((ks & 1) ? a0 : a1, cur, ks + 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < kRows; ++mt) {
        const u32x4 af = (ks & 1) ? a1[mt] : a0[mt];
#pragma unroll
        for (int t = 0; t < KNT; ++t) acc[mt][t] = O::mfma(af, b[ks & 1][t], acc[mt][t]);
        if (ks < 3 && mt < KNT) {
          const typename DQ::Consts k = DQ::prepare(bt.sz[mt][GPT == 2 ? ((ks + 1) >> 1) : 0]);
          b[(ks + 1) & 1][mt] = DQ::run(bt.w[mt][ks + 1], k, m_lo, m_hi, g_lo, g_hi);
        }
        if constexpr (kSteady) load_item(dst, bn, kt + 3, ks, mt);  // tile kt + 3, one load per four MFMAs
#pragma unroll
        for (int t = 0; t < KNT; ++t) {  // one MFMA, then its share of the vector work
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, (20 + KNT - 1) / KNT, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // k tiles of this split
  int kt0, kt1;
  split_range(p.KT, blockIdx.y, p.ksplit, &kt0, &kt1);
  load_tile(lds_a0, b0, kt0);
  load_tile(lds_a1, b1, kt0 + 1);
  load_tile(lds_a2, b2, kt0 + 2);
  // Whole groups of four tiles run in the steady state: every step issues the loads of the tile three ahead, also
  // past K (weights then read as zero without touching memory, activations as bytes that nobody uses), so that the
  // number of loads in flight at a step's wait is always the same.  The remaining one to three tiles issue nothing.
  int kt = kt0;
  for (; kt + 4 <= kt1; kt += 4) {
    step(lds_a0, lds_a3, b0, b3, kt, std::true_type{});
    step(lds_a1, lds_a0, b1, b0, kt + 1, std::true_type{});
    step(lds_a2, lds_a1, b2, b1, kt + 2, std::true_type{});
    step(lds_a3, lds_a2, b3, b2, kt + 3, std::true_type{});
  }
  if (kt < kt1) {
    step(lds_a0, lds_a3, b0, b3, kt, std::false_type{});
    if (kt + 1 < kt1) {
      step(lds_a1, lds_a0, b1, b0, kt + 1, std::false_type{});
      if (kt + 2 < kt1) step(lds_a2, lds_a1, b2, b1, kt + 2, std::false_type{});
    }
  }

  // ---- epilogue: transpose each 16-row slab through LDS so that every lane stores 16 contiguous bytes
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the unused prefetches must not land on top of the transposes
  __syncthreads();
  float* epi = reinterpret_cast<float*>(wave == 0 ? lds_a0 : wave == 1 ? lds_a1 : wave == 2 ? lds_a2 : lds_a3);
  uint16_t* out = static_cast<uint16_t*>(p.out);
  const int ncol0 = nt0 * 16;
  float cf[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};  // bf16 scales: 2^E of this lane's eight columns
  if constexpr (kBF16) {
    const int col = ncol0 + (lane & 7) * 8;
    if ((lane & 7) * 8 < 16 * KNT && col + 8 <= p.N) column_factors(p.sz, p.G, col, cf);
  }
#pragma unroll
  for (int mt = 0; mt < kRows; ++mt) {
#pragma unroll
    for (int t = 0; t < KNT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) epi[(4 * j + i) * kEpiStride + 16 * t + c] = acc[mt][t][i];
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      const int rr = (lane >> 3) + 8 * pass, cc = (lane & 7) * 8;
      const float* src = epi + rr * kEpiStride + cc;
      const int row = m0 + 16 * mt + rr, col = ncol0 + cc;
      float rs = 1.f;
      if constexpr (kBF16) rs = p.row_scale[row < p.M ? row : p.M - 1];
      const bool live = cc < 16 * KNT && row < p.M && col + 8 <= p.N;
      if (p.ksplit > 1) {  // the fp32 segment of this split; the reduction kernel finishes it
        if (live) {
          f32x4* dst = reinterpret_cast<f32x4*>(p.partial + ((size_t)blockIdx.y * p.mblocks * 64 + row) * p.N + col);
          dst[0] = f32x4{src[0], src[1], src[2], src[3]};
          dst[1] = f32x4{src[4], src[5], src[6], src[7]};
        }
        continue;
      }
      float vals[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) vals[q] = src[q] * rs * cf[q];
      epi_store_row8_wave<T>(p.epi, out, vals, row, col, p.N, live, row < p.M, lane);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
  }
}

// Second half of a K split of the 64-row kernel: out[row, col .. col + 7] = epilogue(row factor x sum over the splits,
// in split order), one thread per segment of eight columns.
template <typename T>
__global__ __launch_bounds__(256) void w4a16_splitk_reduce_kernel(const float* __restrict__ partial, size_t split_stride,
                                                                  int ksplit, const float* __restrict__ row_scale,
                                                                  const void* sz, int G, uint16_t* out, int M, int N,
                                                                  Epilogue epi) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t segs = (size_t)N / 8;
  const size_t row = idx / segs;
  if (row >= (size_t)M) return;
  const int col = (int)(idx - row * segs) * 8;
  const f32x4* src = reinterpret_cast<const f32x4*>(partial + row * N + col);
  f32x4 lo = src[0], hi = src[1];
  for (int sp = 1; sp < ksplit; ++sp) {
    lo += src[sp * (split_stride / 4)];
    hi += src[sp * (split_stride / 4) + 1];
  }
  const float rs = row_scale ? row_scale[row] : 1.f;
  float cf[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};
  if (sz) column_factors(sz, G, col, cf);  // bf16 scales: the column's 2^E
  const float vals[8] = {lo[0] * rs * cf[0], lo[1] * rs * cf[1], lo[2] * rs * cf[2], lo[3] * rs * cf[3],
                         hi[0] * rs * cf[4], hi[1] * rs * cf[5], hi[2] * rs * cf[6], hi[3] * rs * cf[7]};
  const float mx = epi_store_row8<T>(epi, out, vals, (int)row, col, N);
  if (epi.row_absmax) atomicMax(reinterpret_cast<unsigned*>(epi.row_absmax) + row, __builtin_bit_cast(unsigned, mx));
}

template <typename T>
void launch_typed(const PrefillArgs& a, int gpt, int nw, int kg, int ct, dim3 grid, dim3 block, hipStream_t s) {
  if (nw <= 0) {  // 64-row tiles; -nw = 16-column tiles per wave
    const int knt = -nw;
    if (gpt == 1) {
      if (knt == 4) hipLaunchKernelGGL((w4a16_mid_kernel<T, 1, 4>), grid, block, 0, s, a);
      else if (knt == 2) hipLaunchKernelGGL((w4a16_mid_kernel<T, 1, 2>), grid, block, 0, s, a);
      else hipLaunchKernelGGL((w4a16_mid_kernel<T, 1, 1>), grid, block, 0, s, a);
    } else {
      if (knt == 4) hipLaunchKernelGGL((w4a16_mid_kernel<T, 2, 4>), grid, block, 0, s, a);
      else if (knt == 2) hipLaunchKernelGGL((w4a16_mid_kernel<T, 2, 2>), grid, block, 0, s, a);
      else hipLaunchKernelGGL((w4a16_mid_kernel<T, 2, 1>), grid, block, 0, s, a);
    }
    return;
  }
#define KSQ_PF(GPT, NW, KG)                                                                              \
  do {                                                                                                   \
    if (ct == 1) hipLaunchKernelGGL((w4a16_prefill_kernel<T, GPT, NW, KG, 1>), grid, block, 0, s, a);    \
    else if (ct == 2) hipLaunchKernelGGL((w4a16_prefill_kernel<T, GPT, NW, KG, 2>), grid, block, 0, s, a); \
    else if (ct == 3) hipLaunchKernelGGL((w4a16_prefill_kernel<T, GPT, NW, KG, 3>), grid, block, 0, s, a); \
    else hipLaunchKernelGGL((w4a16_prefill_kernel<T, GPT, NW, KG, 4>), grid, block, 0, s, a);            \
  } while (0)
  if (nw == 4 && kg == 2) {
    if (gpt == 1) KSQ_PF(1, 4, 2);
    else KSQ_PF(2, 4, 2);
    return;
  }
  if (gpt == 1 && nw == 4) KSQ_PF(1, 4, 1);
  else if (gpt == 1) KSQ_PF(1, 8, 1);
  else if (nw == 4) KSQ_PF(2, 4, 1);
  else KSQ_PF(2, 8, 1);
#undef KSQ_PF
}

}  // namespace

bool w4a16_prefill_supported(int dtype, size_t m, size_t n, size_t k, size_t g, int cus) {
  (void)g;
  (void)dtype;
  // From 65 rows on.  33 to 64 rows as well where the columns alone fill the device several times over, or fill it
  // with a K long enough to split: there one 64-row block with the activations shared through LDS beats the decode
  // kernels, whose workgroups each pull all activations through their own loads (measured at M = 40 / 64: Llama-3-70B
  // gate_up 96 -> 77 / 109 -> 81..88 us, down 47 -> 44.5 / 53 -> 48, Llama-2-7B gate_up 27.5 -> 25.9 / 30.3 -> 28;
  // narrower shapes lose 10 to 60 %, and at 32 rows the decode kernel is 5 % ahead on the wide ones too).
  const size_t ntiles = n / kTileN, kt = k / kTileK;
  size_t min_m = (ntiles >= 4 * (size_t)cus || (ntiles >= 2 * (size_t)cus && kt >= 128)) ? 33 : 65;
  if (const char* e = tuning_env("KSQ_W4_PREFILL_MIN_M")) {  // tuning / test override
    const int v = atoi(e);
    if (v >= 1) min_m = (size_t)v;
  }
  return m >= min_m && n % 16 == 0 && m * k * 2 < 0x7FFFFF00ull && (k / kTileK) * 1024 < 0x7FFFFF00ull;
}

// bf16 route: fp16 copy of the activations + one float per row, in front of whatever else the plan needs
size_t w4a16_prefill_workspace_bytes(int dtype, size_t m, size_t k) {
  if (dtype != KSQ_BF16) return 0;
  return ((m * k * 2 + 255) / 256 * 256 + m * 4 + 255) / 256 * 256;
}

// Tile shapes and the K split of the 64-row kernel; `workspace_bytes` is what remains behind the bf16 front part.
PrefillPlan w4a16_prefill_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes) {
  PrefillPlan p{};
  p.kg = 1;
  p.ct = 4;
  const size_t ntiles = n / kTileN, kt = k / kTileK, mb128 = (m + 127) / 128;
  // Row tile of the workgroup and, for 128 rows, the waves per workgroup, by a cost model of how the tiles fall on the
  // compute units, in units of the time two 128 x 256 workgroups take side by side on one CU: workgroups run in
  // rounds of two per CU (one for the eight-wave 128 x 512 tiles); a last round that puts at most one workgroup on a
  // CU costs a little over half a round.  A 128 x 512 tile costs 1.85 of a 128 x 256 one, a 64 x 256 one 0.62 (the
  // dequantisation is shared by half the rows).  Measured on the Llama-2-7B and Llama-3-70B shapes at M = 96 .. 2048:
  // the choice is the fastest of the three or within 5 % of it wherever K is short enough not to ask for a K split,
  // which only the 64-row kernel has (long K with few column blocks: o / down projections).
  const size_t nb16 = (ntiles + 15) / 16, nb32 = (ntiles + 31) / 32, mb64 = (m + 63) / 64;
  auto rounds_of_two = [&](size_t wgs, double tile) {  // two workgroups per CU
    const size_t full = wgs / (2 * (size_t)cus), rem = wgs % (2 * (size_t)cus);
    return 2.0 * tile * (double)full + (rem == 0 ? 0.0 : rem <= (size_t)cus ? 1.1 * tile : 2.0 * tile);
  };
  // (a grid of at most one 128 x 256 workgroup per CU runs as two k groups of four waves: the price of a full tile)
  // Three column tiles per wave instead of four (tiles of 192 / 384 columns): a tile costs 0.88 of the wider one
  // (the activation stage and the barrier per k tile stay), so it pays where its grid still runs in one round --
  // which the narrower tiles often fill better -- or saves a round.  Measured at the Llama-2-7B shapes, fp16: qkv
  // M = 512 60.8 -> 52.5 us (192 workgroups of 128 x 256 -> 256 of 128 x 192), M = 1024 118.9 -> 103.9 (192 of
  // 128 x 512 -> 256 of 128 x 384); gate_up M = 256 60.5 -> 51.3, M = 512 107.1 -> 90.8; at M >= 2048 the wider
  // tiles win everywhere (4 to 13 %).
  double cost128w4 = 0, cost128w8 = 0;
  int ct_w4 = 4, ct_w8 = 4;
  for (int ct = 4; ct >= 3; --ct) {
    const double f = ct == 4 ? 1.0 : 0.88;
    const size_t nbw4 = (ntiles + 4 * ct - 1) / (4 * ct), nbw8 = (ntiles + 8 * ct - 1) / (8 * ct);
    const double c4 = (mb128 * nbw4 <= (size_t)cus && kt >= 4) ? f : rounds_of_two(mb128 * nbw4, f);
    const double c8 = 1.85 * f * (double)((mb128 * nbw8 + (size_t)cus - 1) / (size_t)cus);
    if (ct == 4 || c4 < 0.99 * cost128w4) {
      cost128w4 = c4;
      ct_w4 = ct;
    }
    if (ct == 4 || c8 < 0.99 * cost128w8) {
      cost128w8 = c8;
      ct_w8 = ct;
    }
  }
  (void)nb32;
  const double cost64 = rounds_of_two(mb64 * nb16, 0.62);
  // a K that the 64-row kernel would split (64 k tiles or more, fewer workgroups than CUs) stays with it
  const bool long_k_few_tiles = kt >= 64 && mb64 * nb16 < (size_t)cus;
  const double cost128 = cost128w8 < cost128w4 ? cost128w8 : cost128w4;
  // (ties go to the 128-row kernel: over 700 measured shapes x M the choice is the same on average either way, and
  // the worst case with a 3 % preference for the 64-row kernel was 8 % behind, a wide gate_up in three rounds)
  p.rows = (!long_k_few_tiles && cost128 < cost64) ? 128 : 64;
  if (const char* e = tuning_env("KSQ_W4_PREFILL_ROWS")) {  // tuning / test override
    const int v = atoi(e);
    if (v == 64 || v == 128) p.rows = v;
  }
  p.ksplit = 1;
  if (p.rows == 64) {
    const size_t mb = (m + 63) / 64;
    auto wgs = [&](int knt) { return mb * ((ntiles + 4 * knt - 1) / (4 * knt)); };
    // column tiles per wave (4, 2 or 1): the choice with the most workgroups that still run all at once, two per
    // CU (measured on the Llama-2 7B and 70B shapes at M = 128 .. 512: within 11 % of the best everywhere); the
    // widest tiles when even those need several rounds.
    int knt = 4;
    if (wgs(4) <= 2 * (size_t)cus) knt = wgs(2) <= 2 * (size_t)cus ? (wgs(1) <= 2 * (size_t)cus ? 1 : 2) : 4;
    // K split over workgroups, with the widest tiles.  Those are bound by their own instruction stream (about a
    // microsecond per k tile and workgroup), so a split pays where they leave CUs empty and K is long: from 64 k
    // tiles on and fewer workgroups than CUs, as many splits as fill two workgroup slots per CU, at least twelve k
    // tiles each, and the partial tiles (written and read once, about 4 TB/s) at most 40 % of the unsplit estimate
    // of 0.7 us per k tile.  Measured at the Llama-2 shapes, M = 128 .. 512: 7B down 52 -> 31, 54 -> 38, 61 -> 57 us;
    // 70B qkv 61 -> 46, 65 -> 55; 70B o 41 -> 39, 51 -> 47; 70B down 130 -> 100, 159 -> 125 us; K = 4096 never gains.
    size_t ks = 1;
    if (kt >= 64 && wgs(4) < (size_t)cus) {
      ks = 2 * (size_t)cus / wgs(4);
      if (ks > 8) ks = 8;
      if (ks > kt / 12) {  // too short for two workgroups per CU: one per CU if that fits, else what fits
        const size_t one = (size_t)cus / wgs(4);
        ks = one <= kt / 12 ? one : kt / 12;
      }
      auto traffic_us = [&](size_t c) { return 2.0 * (double)c * (double)(mb * 64) * (double)n * 4.0 / 4e6; };
      while (ks > 1 && traffic_us(ks) > 0.4 * 0.7 * (double)kt) --ks;
      if (ks < 1) ks = 1;
    }
    if (const char* e = tuning_env("KSQ_W4_PREFILL_KSPLIT")) {  // tuning / test override
      const size_t v = (size_t)atoi(e);
      if (v >= 1 && v <= 8 && v <= kt) ks = v;
    }
    auto need = [&](size_t x) { return x <= 1 ? (size_t)0 : x * mb * 64 * n * 4; };
    while (ks > 1 && need(ks) > workspace_bytes) --ks;
    if (ks > 1) knt = 4;
    if (const char* e = tuning_env("KSQ_W4_PREFILL_NT")) {  // tuning / test override
      const int v = atoi(e);
      if (v == 1 || v == 2 || v == 4) knt = v;
    }
    p.knt = knt;
    p.ksplit = (int)ks;
    p.partial_bytes = need(ks);
    // The 128-row kernel in its one-workgroup-per-CU form (four waves side by side, two k groups), with tiles of 64
    // to 256 columns and K split over workgroups like the 64-row kernel's: the dequantisation of a weight tile then
    // serves 128 rows instead of 64, which outweighs the rows that the taller tiles pad wherever both forms cover the
    // device in one round, and at 65 .. 128 rows the narrow tiles (128 x 128, 128 x 64) give one row block the
    // workgroups that two 64-row blocks get from their second block.  Chosen by an estimate in microseconds fitted
    // to sweeps over the Llama-2-7B/13B, Llama-3-8B/70B and Qwen-72B shapes at M = 65 .. 1024 (every form three
    // times; the fits within 4 to 7 % rms): per k tile of a workgroup 0.4 to 1.8 us for the 64-row form by tile width
    // and by one or two workgroups per CU; for the 128-row form 0.57 + 0.13 x, 0.68 + 0.25 x, 0.96 + 0.29 x and
    // 1.11 + 0.50 x us with one to four column tiles per wave (x = the share of the CUs in use: the per-tile time
    // grows as the device fills), a fixed part, and the partial tiles at 6 TB/s.  The 128-row form is taken where it
    // is estimated 5 % ahead, and only on grids that use three quarters of the CUs or more: every case of the fits
    // where it won has that, and on narrow shapes (N = 272 .. 2048) the estimate, extrapolated below it, chose the
    // form where it was 2 to 10 % slower.  Measured afterwards on those shapes and on three families the fit had not
    // seen (Qwen2.5-32B, Yi-34B, half of the 70B shapes), 448 cases at M = 65 .. 1024, against the better of the
    // 64-row kernel and the unsplit 128 x 192 .. 512 tiles: 5.4 % faster on average (8.4 % at M = 65 .. 128), the 266
    // cases that take one of these forms 9.2 % (-33 .. +4.6 %); e.g. Llama-2-7B down M = 512 62 -> 58 us,
    // M = 1024 107 -> 92; Llama-3-70B o M = 384 75 -> 66, down M = 512 276 -> 212; at M = 65 .. 128
    // Llama-2-7B qkv 27 -> 23.5 .. 27, 70B qkv 34 -> 30 .. 35, 13B gate_up 50 -> 43 .. 49.
    // (not for a single 64-row block: half of a 128-row tile would be padding, and the fits start at 65 rows)
    if (!tuning_env("KSQ_W4_PREFILL_ROWS") && !tuning_env("KSQ_W4_PREFILL_KSPLIT") && !tuning_env("KSQ_W4_PREFILL_NT") &&
        mb >= 2 && wgs(knt) * ks <= 2 * (size_t)cus) {
      const bool two = wgs(knt) * ks > (size_t)cus;
      const double b64 = knt == 1 ? (two ? 0.751 : 0.412) : knt == 2 ? (two ? 1.171 : 0.80) : (two ? 1.811 : 1.004);
      const double a64 = knt == 4 ? (two ? 9.0 : 6.9) : knt == 2 ? (two ? 3.1 : 4.0) : (two ? 3.0 : 4.8);
      auto partial_us = [&](size_t c, size_t rows) { return 3.0 + 2.0 * (double)c * (double)rows * (double)n * 4.0 / 6e6; };
      // (both kernels store and the reduction reads the rows below m only: the traffic follows m, not the blocks)
      const double est64 = a64 + b64 * (double)((kt + ks - 1) / ks) + (ks > 1 ? partial_us(ks, m) : 0.0);
      auto need128 = [&](size_t x) { return x <= 1 ? (size_t)0 : x * mb128 * 128 * n * 4; };
      static const double kTile[5] = {0, 0.569, 0.682, 0.962, 1.106}, kFill[5] = {0, 0.129, 0.250, 0.292, 0.495},
                          kFixed[5] = {0, 5.1, 6.3, 6.75, 7.35};
      double best = 0.95 * est64;
      for (int ct = 4; ct >= 1; --ct) {
        if (ct <= 2 && mb128 > 3) break;  // the narrow tiles were fitted at up to 384 rows (narrow shapes at 512 and
                                          // 1000 rows: chosen there, they ran 4 to 14 % behind the 64-row form)
        const size_t w = mb128 * ((ntiles + (size_t)(4 * ct) - 1) / (size_t)(4 * ct));
        // (workgroup ids go to the 8 XCDs in turn, y-slab after y-slab: what has to fit is every XCD's share)
        for (size_t c = 1; c <= 8 && (w + 7) / 8 * c <= (size_t)cus / 8 && kt / c >= 8; ++c) {
          if (need128(c) > workspace_bytes) break;
          if (4 * w * c < 3 * (size_t)cus) continue;  // the fits know nothing below three quarters of the CUs in use
          const double fill = (double)(w * c) / (double)cus;
          const double est = kFixed[ct] + (kTile[ct] + kFill[ct] * fill) * (double)((kt + c - 1) / c) +
                             (c > 1 ? partial_us(c, m) : 0.0);
          if (est < best) {
            best = est;
            p.rows = 128;
            p.nw = 4;
            p.kg = 2;
            p.ct = ct;
            p.ksplit = (int)c;
            p.partial_bytes = need128(c);
          }
        }
      }
    }
  } else {
    p.nw = cost128w8 < cost128w4 ? 8 : 4;
    p.ct = p.nw == 8 ? ct_w8 : ct_w4;
    if (const char* e = tuning_env("KSQ_W4_PREFILL_WAVES")) {  // tuning / test override
      const int v = atoi(e);
      if (v == 4 || v == 8) {
        p.nw = v;
        p.ct = v == 8 ? ct_w8 : ct_w4;
      }
    }
    if (const char* e = tuning_env("KSQ_W4_PREFILL_CT")) {  // tuning / test override
      const int v = atoi(e);
      if (v >= 1 && v <= 4) p.ct = v;
    }
    // one workgroup per CU at most: two k groups of four waves each
    const size_t nbw = (ntiles + (size_t)(4 * p.ct) - 1) / (size_t)(4 * p.ct);
    p.kg = (p.nw == 4 && mb128 * nbw <= (size_t)cus && kt >= 4) ? 2 : 1;
    // (a K split of this form is the planner's choice only from the 64-row side, above)
    size_t ks = 1;
    if (const char* e = tuning_env("KSQ_W4_PREFILL_KSPLIT")) {  // tuning / test override
      const size_t v = (size_t)atoi(e);
      if (v >= 1 && v <= 8 && v <= kt) ks = v;
    }
    auto need128 = [&](size_t x) { return x <= 1 ? (size_t)0 : x * mb128 * 128 * n * 4; };
    while (ks > 1 && need128(ks) > workspace_bytes) --ks;
    p.ksplit = (int)ks;
    p.partial_bytes = need128(ks);
    if (const char* e = tuning_env("KSQ_W4_PREFILL_KG")) {  // tuning / test override
      const int v = atoi(e);
      if (v == 1 || (v == 2 && kt >= 2)) p.kg = v;
    }
    if (p.nw == 8) p.kg = 1;
  }
  return p;
}

int w4a16_launch_prefill(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m,
                         size_t n, size_t k, size_t g, void* workspace, size_t workspace_bytes, hipStream_t s,
                         const Epilogue& epi) {
  KSQ_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15) == 0 && n % 8 == 0, KSQ_ERR_INVALID_ARGUMENT,
              "prefill output must be 16-byte aligned");
  PrefillArgs a{};
  a.epi = epi;
  a.weight = weight;
  a.sz = sz;
  a.act = act;
  a.out = out;
  a.row_scale = nullptr;
  a.M = (int)m;
  a.N = (int)n;
  a.K = (int)k;
  a.KT = (int)(k / kTileK);
  a.G = (int)(k / g);
  a.ntiles = (int)(n / kTileN);
  const DeviceInfo* di = device_info();
  KSQ_REQUIRE(di != nullptr, KSQ_ERR_HIP, "no device");
  const size_t front = w4a16_prefill_workspace_bytes(dtype, m, k);
  KSQ_REQUIRE(front == 0 || (workspace != nullptr && workspace_bytes >= front), KSQ_ERR_WORKSPACE,
              "bf16 prefill needs its workspace");
  const PrefillPlan plan = w4a16_prefill_plan(m, n, k, di->cus, workspace ? workspace_bytes - front : 0);
  a.ksplit = plan.ksplit;
  a.partial = plan.ksplit > 1 ? reinterpret_cast<float*>(static_cast<char*>(workspace) + front) : nullptr;
  int nw = 0;  // > 0: waves of the 128-row kernel; <= 0: minus the column tiles per wave of the 64-row kernel
  dim3 grid, block(256);
  if (plan.rows == 64) {
    a.mblocks = (int)((m + 63) / 64);
    const int knt = plan.knt;
    nw = -knt;
    a.nblocks = (a.ntiles + 4 * knt - 1) / (4 * knt);
    KSQ_REQUIRE((size_t)a.mblocks * a.nblocks < (1ull << 30), KSQ_ERR_UNSUPPORTED, "grid too large");
    grid = dim3(tile_grid(a.mblocks, a.nblocks), (unsigned)plan.ksplit);
  } else {
    a.mblocks = (int)((m + kBM - 1) / kBM);
    nw = plan.nw;
    const int bnt = nw * plan.ct;
    a.nblocks = (a.ntiles + bnt - 1) / bnt;
    KSQ_REQUIRE((size_t)a.mblocks * a.nblocks < (1ull << 30), KSQ_ERR_UNSUPPORTED, "grid too large");
    grid = dim3(tile_grid(a.mblocks, a.nblocks), (unsigned)plan.ksplit);
    block = dim3(64 * nw * plan.kg);
  }
  const int gpt = (int)(kTileK / g);
  if (dtype != KSQ_F16) note_launch("bf16_rows_to_f16_kernel grid=(%zu)", m);
  if (plan.rows == 64)
    note_launch("w4a16_mid_kernel<gpt=%d,knt=%d> grid=(%u,%u)", gpt, plan.knt, grid.x, grid.y);
  else
    note_launch("w4a16_prefill_kernel<gpt=%d,nw=%d,kg=%d,ct=%d> grid=(%u,%u)", gpt, plan.nw, plan.kg, plan.ct, grid.x, grid.y);
  if (plan.ksplit > 1) note_launch("w4a16_splitk_reduce_kernel");
  if (dtype == KSQ_F16) {
    launch_typed<_Float16>(a, gpt, nw, plan.kg, plan.ct, grid, block, s);
  } else {
    uint16_t* a16 = static_cast<uint16_t*>(workspace);
    float* row_scale = reinterpret_cast<float*>(static_cast<char*>(workspace) + (m * k * 2 + 255) / 256 * 256);
    const uint16_t* a_in = static_cast<const uint16_t*>(act);
    const dim3 rows((unsigned)m), lanes(256);
    if (k <= 2048) hipLaunchKernelGGL(bf16_rows_to_f16_kernel<1>, rows, lanes, 0, s, a_in, a16, row_scale, (int)k);
    else if (k <= 4096) hipLaunchKernelGGL(bf16_rows_to_f16_kernel<2>, rows, lanes, 0, s, a_in, a16, row_scale, (int)k);
    else if (k <= 8192) hipLaunchKernelGGL(bf16_rows_to_f16_kernel<4>, rows, lanes, 0, s, a_in, a16, row_scale, (int)k);
    else if (k <= 16384) hipLaunchKernelGGL(bf16_rows_to_f16_kernel<8>, rows, lanes, 0, s, a_in, a16, row_scale, (int)k);
    else if (k <= 32768) hipLaunchKernelGGL(bf16_rows_to_f16_kernel<16>, rows, lanes, 0, s, a_in, a16, row_scale, (int)k);
    else hipLaunchKernelGGL(bf16_rows_to_f16_long_kernel, rows, lanes, 0, s, a_in, a16, row_scale, (int)k);
    a.act = a16;
    a.row_scale = row_scale;
    launch_typed<__bf16>(a, gpt, nw, plan.kg, plan.ct, grid, block, s);
  }
  if (plan.ksplit > 1) {  // add the splits up and store
    const size_t stride = (size_t)a.mblocks * (plan.rows == 64 ? 64 : kBM) * n;
    const dim3 rgrid((unsigned)((m * (n / 8) + 255) / 256));
    uint16_t* o = static_cast<uint16_t*>(out);
    if (dtype == KSQ_F16)
      hipLaunchKernelGGL(w4a16_splitk_reduce_kernel<_Float16>, rgrid, dim3(256), 0, s, a.partial, stride, plan.ksplit,
                         a.row_scale, (const void*)nullptr, a.G, o, (int)m, (int)n, epi);
    else
      hipLaunchKernelGGL(w4a16_splitk_reduce_kernel<__bf16>, rgrid, dim3(256), 0, s, a.partial, stride, plan.ksplit,
                         a.row_scale, sz, a.G, o, (int)m, (int)n, epi);
  }
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

}  // namespace ksq
