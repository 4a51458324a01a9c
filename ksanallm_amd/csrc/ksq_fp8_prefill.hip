// FP8 e4m3 GEMM, large M (MFMA-bound): out[m,n] = T((sum_k a[m,k] * w[n,k]) * w_scale[n] * a_scale[m]).
//
// Workgroup tile 128 rows x 256 columns, four waves side by side, every wave 8 x 4 MFMA tiles of 16 x 16 with fp32
// accumulators, K = 128 per instruction (v_mfma_f32_16x16x128_f8f6f4, both operands OCP e4m3, no block scaling).
// Activations go from global memory straight into LDS in fragment order (one 128-row x 128-k stage = 16 KiB, four
// stages in flight as four separate objects, loaded two stages ahead, one barrier per stage); weights are read by
// each wave for its own 64 columns straight from the [N][K] tensor into registers, one stage ahead.  The loads of
// the coming stages are issued one at a time between the matrix instructions.
// Inside one instruction lane (r, j) holds bytes [16j, 16j+16) and [64+16j, 64+16j+16) of row r's 128-byte k
// slice -- the same assignment on both operands, so the products pair up, and every 128-bit load of a 16-lane
// group covers 64 contiguous bytes of a row.  K must be a multiple of 128 (other K take the streaming kernel).
#include <cstdlib>

#include "ksq_epilogue.h"
#include "ksq_internal.h"

namespace ksq {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) void* lds_ptr;

struct Fp8PrefillArgs {
  const uint8_t* aq;  // [M][K]
  const uint8_t* wq;  // [N][K]
  const float* a_scale;
  const float* w_scale;
  void* out;
  int M, N, K, KS /* 128-byte k stages */, mblocks, nblocks;
  int a_scale_per_row, w_scale_per_col;
  // 256 x 256 kernel only: this launch covers the logical tile ids lid_begin .. of the whole grid; with ksplit > 1
  // it is the launch for the tiles of a last, mostly empty round: K is split over grid.y and every split stores its
  // raw fp32 tile to `partial` [split][tile - lid_begin][256][256] for fp8_tail_reduce_kernel
  int lid_begin, ksplit, tail_tiles;
  float* partial;
  Epilogue epi;
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

// A global -> LDS load of 16 bytes per lane (lane l lands at lds + 16 l) written as an assembly statement, so that the
// compiler does not know it to be one: it would otherwise wait for *every* outstanding vector memory load before an
// LDS read that follows (it cannot always tell which LDS bytes a pending load writes), which empties a ring of stages
// that are deliberately left in flight.  The statement sets M0 (LDS address of lane 0) itself; the kernel that uses it
// has no other user of M0.  Ordering against the LDS reads is the kernel's business (s_waitcnt vmcnt + s_barrier).
__device__ inline u32x4 raw_rsrc(const void* base, size_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  return u32x4{(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
}
#if defined(KSQ_EMU)
typedef uintptr_t lds_addr_t;  // host build: LDS is host memory
__device__ inline lds_addr_t lds_addr(const void* p) { return reinterpret_cast<uintptr_t>(p); }
__device__ inline void load_lds_opaque(u32x4 rsrc, lds_addr_t lds, uint32_t voff, uint32_t soff) {
  const uint64_t base = (uint64_t)rsrc[0] | ((uint64_t)(rsrc[1] & 0xffffu) << 32);
  const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(base), 0, (int)rsrc[2], 0);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_ptr) reinterpret_cast<void*>(lds), 16, voff, soff, 0, 0);
}
#else
typedef uint32_t lds_addr_t;
__device__ inline lds_addr_t lds_addr(const void* p) {
  return (uint32_t)reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)p);
}
__device__ inline void load_lds_opaque(u32x4 rsrc, lds_addr_t lds, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds), "v"(voff), "s"(rsrc), "s"(soff)
               : "memory");
}
#endif

__device__ inline i32x8 join(u32x4 lo, u32x4 hi) {
  i32x8 v;
  v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
  v[4] = hi[0]; v[5] = hi[1]; v[6] = hi[2]; v[7] = hi[3];
  return v;
}

template <typename T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void fp8_prefill_kernel(Fp8PrefillArgs p) {
  constexpr int kStage = kMT * 2 * 64;  // 16-byte elements per activation stage (16 KiB)
  constexpr int kEpiStride = 68;
  // four stages as four separate objects: loads into one are then known not to alias reads of another
  __shared__ u32x4 lds0[kStage];
  __shared__ u32x4 lds1[kStage];
  __shared__ u32x4 lds2[kStage];
  __shared__ u32x4 lds3[kStage];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, j = lane >> 4;

  int mb, nb;
  if (!tile_of(tile_logical_id(blockIdx.x, gridDim.x), p.mblocks, p.nblocks, &mb, &nb)) return;  // rounding of the grid
  const int m0 = mb * kBM, n0 = nb * kBN + wave * (kNT * 16);

  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.aq), 0, (int)((size_t)p.M * p.K), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.wq), 0, (int)((size_t)p.N * p.K), 0x00020000);
  // Staging role of this wave: fragments f = 4 * wave + i (row tile f >> 1, half f & 1) of a stage, this lane's 16
  // bytes; rows past M repeat row M - 1 (their results are never stored).
  unsigned a_off[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    int row = m0 + 16 * (2 * wave + h) + r;
    row = row < p.M ? row : p.M - 1;
    a_off[h] = (unsigned)row * p.K + 16 * j;
  }
  unsigned w_off[kNT];  // rows past N read as zero
#pragma unroll
  for (int t = 0; t < kNT; ++t) {
    const int row = n0 + 16 * t + r;
    w_off[t] = row < p.N ? (unsigned)row * p.K + 16 * j : 0x80000000u;
  }

  f32x4 acc[kMT][kNT];
#pragma unroll
  for (int mt = 0; mt < kMT; ++mt)
#pragma unroll
    for (int t = 0; t < kNT; ++t) acc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  struct BStage {
    u32x4 w[kNT][2];
  };
  BStage b0, b1;

  // item i < 4: activation fragment 4 * wave + i of stage s -> buf.  The scalar offset is not range-checked: a
  // prefetch past K re-reads the last stage (nobody uses it).
  auto load_a_item = [&](u32x4* buf, int s, int i) {
    const int sc = s < p.KS ? s : p.KS - 1;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(buf + (4 * wave + i) * 64), 16, a_off[i >> 1],
                                             sc * 128 + (i & 1) * 64, 0, 0);
  };
  // item i < 8: weight piece (column tile i >> 1, half i & 1) of stage s; a stage past K is never used
  auto load_b_item = [&](BStage& b, int s, int i) {
    const int t = i >> 1, h = i & 1;
    b.w[t][h] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w, w_off[t] + s * 128u + 64u * h, 0, 0));
  };
  auto read_a = [&](const u32x4* buf, int mt) {
    return join(buf[(mt * 2 + 0) * 64 + lane], buf[(mt * 2 + 1) * 64 + lane]);
  };

  // One stage.  On entry all loads but the four newest (the activations of stage s + 1) have landed; after the
  // barrier stage s is visible to every wave and every wave is done with the buffer that stage s + 2 goes into.
  auto step = [&](const u32x4* cur, u32x4* dst, const BStage& bc, BStage& bn, int s) {
    __builtin_amdgcn_s_waitcnt(0x0F74);  // vmcnt(4)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    i32x8 bf[kNT];
#pragma unroll
    for (int t = 0; t < kNT; ++t) bf[t] = join(bc.w[t][0], bc.w[t][1]);
    i32x8 a_cur = read_a(cur, 0), a_nxt = read_a(cur, 1);
#pragma unroll
    for (int mt = 0; mt < kMT; ++mt) {
      const i32x8 af = a_cur;
      a_cur = a_nxt;
      if (mt + 2 < kMT) a_nxt = read_a(cur, mt + 2);
      load_b_item(bn, s + 1, mt);  // weights of the next stage first ...
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < kNT; ++t)
        acc[mt][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af, bf[t], acc[mt][t], 0, 0, 0, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) load_a_item(dst, s + 2, i);  // ... then the activations two stages ahead
    __builtin_amdgcn_sched_barrier(0);
  };

#pragma unroll
  for (int i = 0; i < 4; ++i) load_a_item(lds0, 0, i);
#pragma unroll
  for (int i = 0; i < 8; ++i) load_b_item(b0, 0, i);
#pragma unroll
  for (int i = 0; i < 4; ++i) load_a_item(lds1, 1, i);
  int s = 0;
  for (; s + 4 <= p.KS; s += 4) {
    step(lds0, lds2, b0, b1, s);
    step(lds1, lds3, b1, b0, s + 1);
    step(lds2, lds0, b0, b1, s + 2);
    step(lds3, lds1, b1, b0, s + 3);
  }
  if (s < p.KS) {
    step(lds0, lds2, b0, b1, s);
    if (s + 1 < p.KS) {
      step(lds1, lds3, b1, b0, s + 1);
      if (s + 2 < p.KS) step(lds2, lds0, b0, b1, s + 2);
    }
  }

  // ---- epilogue: scales, then a transpose through LDS so that every lane stores 16 contiguous bytes
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the last (unused) prefetches must not land on top of the transposes
  __syncthreads();
  float* epi = reinterpret_cast<float*>(wave == 0 ? lds0 : wave == 1 ? lds1 : wave == 2 ? lds2 : lds3);
  epi_elem_t<T>* out = static_cast<epi_elem_t<T>*>(p.out);
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
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      const int rr = (lane >> 3) + 8 * pass, cc = (lane & 7) * 8;
      const float* src = epi + rr * kEpiStride + cc;
      const int row = m0 + 16 * mt + rr, col = n0 + cc;
      const float as = p.a_scale[p.a_scale_per_row ? (row < p.M ? row : p.M - 1) : 0];
      float vals[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) vals[q] = src[q] * as;
      epi_store_row8_wave<T>(p.epi, out, vals, row, col, p.N, row < p.M && col + 8 <= p.N, row < p.M, lane);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // ... and its reads, before the next row tile overwrites the slab
  }
}


// The same GEMM with a 256 x 256 workgroup tile: eight waves as 2 x 4, every wave 128 rows x 64 columns.  Both
// operands go from global memory straight into LDS (one stage = 256 rows x 128 k of each = 32 KiB per operand; two
// stages of activations, three of weights = all 160 KiB), so
// each byte crosses the CU's vector memory path once per workgroup: 128 x 256 tiles need 46 B/clk per CU at the
// matrix cores' FP8 rate, this one 32.  One workgroup per CU.
// WN = 4: the whole tile, waves as 2 x 4.  WN = 1: a quarter of it, 256 rows x 64 columns, waves as 8 x 1 (every wave 32
// rows x 64 columns), four workgroups to a tile: for the tiles of a last round that is mostly empty, which then fill
// the device without a K split (no partial tiles through memory).  Its weight stage is 8 KiB, one block per wave.
template <typename T, int WN = 4>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void fp8_prefill256_kernel(Fp8PrefillArgs p) {
  static_assert(WN == 4 || WN == 1, "whole tiles or column quarters");
  constexpr int kMTW = WN == 4 ? 8 : 2;      // row tiles per wave
  constexpr int kHalf = 16 * 2 * 64;         // 16-byte elements of an activation stage (32 KiB)
  constexpr int kHalfB = 4 * WN * 2 * 64;    // ... of a weight stage (32 or 8 KiB)
  constexpr int kEpiStride = 68;
  __shared__ u32x4 lds_a0[kHalf];
  __shared__ u32x4 lds_a1[kHalf];
  __shared__ u32x4 lds_b0[kHalfB];
  __shared__ u32x4 lds_b1[kHalfB];
  __shared__ u32x4 lds_b2[kHalfB];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = WN == 4 ? wave >> 2 : wave, wn = WN == 4 ? wave & 3 : 0;
  const int r = lane & 15, j = lane >> 4;

  // this launch covers the logical tile ids lid_begin .. of the whole grid (with WN = 1: four workgroups to a tile)
  const int unit = tile_logical_id(blockIdx.x, gridDim.x);
  const int lid = p.lid_begin + (WN == 4 ? unit : unit >> 2);
  int mb, nb;
  if (!tile_of(lid, p.mblocks, p.nblocks, &mb, &nb)) return;  // rounding of the grid
  const int m0 = mb * 256, n0 = nb * 256 + (WN == 4 ? 0 : 64 * (unit & 3));

  const u32x4 rs_a = raw_rsrc(p.aq, (size_t)p.M * p.K), rs_w = raw_rsrc(p.wq, (size_t)p.N * p.K);
  // Operand stage in LDS: 32 blocks of 1 KiB per operand, block (tile, q) = rows 8q .. 8q+7 of a 16-row tile, all
  // 128 bytes of the stage.  A block is one global -> LDS load instruction (lane l lands at l * 16) with lane l on
  // row l/4 % 8, half l / 32 of the 128 bytes and 16-byte piece (l % 4) ^ x(row, q): every aligned group of four
  // lanes reads 64 contiguous bytes of one row (the memory pipeline then takes four lanes per clock instead of one),
  // and the xor makes the 16 rows that one group of 16 lanes reads back for an MFMA operand fall on 16 different
  // bank groups.  Rows past M / N repeat the last row (their results are never stored).  This wave brings in
  // blocks 4 * wave .. 4 * wave + 3 of each operand, i.e. tiles 2 * wave and 2 * wave + 1.
  unsigned a_off[4], w_off[4];
  {
    const int rr = (lane >> 2) & 7, hh = lane >> 5;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = i & 1, x = (rr >> 2) | (q << 1);
      const unsigned kb = 64u * hh + 16u * ((lane & 3) ^ x);
      int row = m0 + 16 * (2 * wave + (i >> 1)) + 8 * q + rr;
      row = row < p.M ? row : p.M - 1;
      a_off[i] = (unsigned)row * p.K + kb;
      // weight blocks: four per wave of the 32, or (WN = 1) block `wave` of the 8: tile wave / 2, rows 8 (wave % 2) ..
      const int wq8 = WN == 4 ? q : (wave & 1), wx = (rr >> 2) | (wq8 << 1);
      const unsigned wkb = 64u * hh + 16u * ((lane & 3) ^ wx);
      int col = WN == 4 ? n0 + 16 * (2 * wave + (i >> 1)) + 8 * q + rr : n0 + 16 * (wave >> 1) + 8 * (wave & 1) + rr;
      col = col < p.N ? col : p.N - 1;
      w_off[i] = (unsigned)col * p.K + wkb;
    }
  }
  // where lane (r, j) finds piece j of half 0 of row r of a tile inside the stage, apart from tile * 128 and
  // half * 32 (in 16-byte units)
  const int f_lane = (r >> 3) * 64 + (r & 7) * 4 + (j ^ (((r & 7) >> 2) | ((r >> 3) << 1)));

  f32x4 acc[kMTW][kNT];
#pragma unroll
  for (int mt = 0; mt < kMTW; ++mt)
#pragma unroll
    for (int t = 0; t < kNT; ++t) acc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Rows past M: the activation rows 32 * wave .. 32 * wave + 31 that this wave stages are not loaded when all of them
  // lie past M (what the LDS then holds feeds only output rows that are never stored), and a wave whose 128 output
  // rows all lie past M issues its share of the loads and no matrix instruction.  Both are uniform over the wave; a
  // step's `vmcnt` keeps its meaning, since the loads that may stay in flight are the step's weight loads.
  const bool a_live = m0 + 32 * wave < p.M, rows_live = m0 + 16 * kMTW * wm < p.M;
  // item i of a step's loads: i < 4 activations of stage sa, else weights of stage sb (four, or one with WN = 1)
  constexpr int kItems = 4 + WN;
  auto load_item = [&](u32x4* abuf, u32x4* bbuf, int sa, int sb, int i) __attribute__((always_inline)) {
    const int f = i & 3;
    // the scalar offset is not range-checked: past K, the last stage again (nobody uses it)
    const int sac = sa < p.KS ? sa : p.KS - 1, sbc = sb < p.KS ? sb : p.KS - 1;
    if (i < 4) {
      if (a_live) load_lds_opaque(rs_a, lds_addr(abuf + (4 * wave + f) * 64), a_off[f], sac * 128);
    } else if (i < kItems) {
      load_lds_opaque(rs_w, lds_addr(bbuf + (WN * wave + f) * 64), w_off[f], sbc * 128);
    }
  };
  auto read_frag = [&](const u32x4* buf, int tile) __attribute__((always_inline)) {
    return join(buf[tile * 128 + f_lane], buf[tile * 128 + 32 + f_lane]);
  };

  // One stage.  Weights (they come from HBM) are requested two stages ahead into a ring of three buffers, activations
  // (mostly L2 hits: every row block is shared by all column blocks) one stage ahead into a ring of two.  Loads
  // retire in order and a step issues its activation loads before its weight loads, so on entry everything but the
  // four weight loads of the previous step (stage s + 1) has to have landed.
  //
  // WN = 4: the two halves of the workgroup (waves 0-3 = rows 0..127, waves 4-7 = rows 128..255; one wave of each on
  // every SIMD) run half a step apart, so that on every SIMD one wave issues matrix instructions while the other
  // waits for its first LDS reads after a barrier.  Every wave passes two barriers per step, one at its start and
  // one in the middle (after four of its eight row tiles); the second half passed one more before its first step,
  // the first half passes one more after its last.  A half stages exactly the activation rows it reads itself, so
  // only the weight buffers tie the halves together: stage s is complete when the first half starts step s because
  // the second half waits for its share of it before the barrier in the middle of its step s - 1 (all but the eight
  // loads of that step have landed), and the buffer that the first half refills during step s (stage s - 1) was
  // copied into registers by the second half before that same barrier.
  auto mid_wait = [&]() __attribute__((always_inline)) {
    if (wm == 1) {
      if (a_live) __builtin_amdgcn_s_waitcnt(0x0F78);  // vmcnt(8): this step's loads may be in flight
      else __builtin_amdgcn_s_waitcnt(0x0F74);         // vmcnt(4): this wave loads weights only
    }
  };
  auto step = [&](const u32x4* acur, const u32x4* bcur, u32x4* anxt, u32x4* bnxt2, int s) __attribute__((always_inline)) {
    // vmcnt(4) / vmcnt(1): the weight loads of the step before may be in flight.  lgkmcnt(0) costs nothing here (the
    // matrix instructions of the step before have consumed every LDS read) and tells the compiler that no scalar
    // load is pending: LDS reads and scalar loads share that counter, and while it believes one of the latter may be
    // in flight it turns the first LDS wait of the step into a wait for all 14 reads instead of the first four.
    if constexpr (WN == 4) __builtin_amdgcn_s_waitcnt(0x0074);
    else __builtin_amdgcn_s_waitcnt(0x0071);
    __builtin_amdgcn_s_barrier();        // ... everyone's share has landed, and everyone is done with the stage before
    __builtin_amdgcn_sched_barrier(0);
    if (!rows_live) {
#pragma unroll
      for (int i = 0; i < kItems; ++i) load_item(anxt, bnxt2, s + 1, s + 2, i);
      if constexpr (WN == 4) {
        mid_wait();
        __builtin_amdgcn_s_barrier();
      }
      __builtin_amdgcn_sched_barrier(0);
      return;
    }
    // the operands of the first matrix instruction first
    i32x8 bf[kNT];
    i32x8 a_cur = read_frag(acur, kMTW * wm + 0);
#pragma unroll
    for (int t = 0; t < kNT; ++t) bf[t] = read_frag(bcur, 4 * wn + t);
    i32x8 a_nxt = read_frag(acur, kMTW * wm + 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int mt = 0; mt < kMTW; ++mt) {
      if constexpr (WN == 4) {
        if (mt == 4) {
          mid_wait();
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      const i32x8 af = a_cur;
      a_cur = a_nxt;
      if (mt + 2 < kMTW) a_nxt = read_frag(acur, kMTW * wm + mt + 2);
      if constexpr (WN == 4) {
        if (mt < 4) {  // the loads go out in the first half: activations first, then weights
          load_item(anxt, bnxt2, s + 1, s + 2, mt < 2 ? 2 * mt : 4 + 2 * (mt - 2));
          load_item(anxt, bnxt2, s + 1, s + 2, mt < 2 ? 2 * mt + 1 : 4 + 2 * (mt - 2) + 1);
        }
      } else {  // two row tiles: the four activation loads with the first, the weight load with the second
        if (mt == 0) {
#pragma unroll
          for (int i = 0; i < 4; ++i) load_item(anxt, bnxt2, s + 1, s + 2, i);
        } else {
          load_item(anxt, bnxt2, s + 1, s + 2, 4);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < kNT; ++t)
        acc[mt][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af, bf[t], acc[mt][t], 0, 0, 0, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // k stages of this launch's split (all of them unless this is the tail launch)
  int s_begin, s_end;
  split_range(p.KS, blockIdx.y, p.ksplit, &s_begin, &s_end);
#pragma unroll
  for (int i = 0; i < 4; ++i) load_item(lds_a0, lds_b0, s_begin, s_begin, i);
#pragma unroll
  for (int i = 4; i < kItems; ++i) load_item(lds_a0, lds_b0, s_begin, s_begin, i);
#pragma unroll
  for (int i = 4; i < kItems; ++i) load_item(lds_a0, lds_b1, s_begin, s_begin + 1, i);
  if constexpr (WN == 4) {
    if (wm == 1) {  // the second half starts half a step late; its share of the first weight stage has landed
      __builtin_amdgcn_s_waitcnt(0x0F74);
      __builtin_amdgcn_s_barrier();
    }
  }
  int s = s_begin;
  for (; s + 6 <= s_end; s += 6) {
    step(lds_a0, lds_b0, lds_a1, lds_b2, s);
    step(lds_a1, lds_b1, lds_a0, lds_b0, s + 1);
    step(lds_a0, lds_b2, lds_a1, lds_b1, s + 2);
    step(lds_a1, lds_b0, lds_a0, lds_b2, s + 3);
    step(lds_a0, lds_b1, lds_a1, lds_b0, s + 4);
    step(lds_a1, lds_b2, lds_a0, lds_b1, s + 5);
  }
  // the remaining zero to five stages, same rotation (their prefetches past the end re-read a stage nobody uses)
  if (s < s_end) step(lds_a0, lds_b0, lds_a1, lds_b2, s);
  if (s + 1 < s_end) step(lds_a1, lds_b1, lds_a0, lds_b0, s + 1);
  if (s + 2 < s_end) step(lds_a0, lds_b2, lds_a1, lds_b1, s + 2);
  if (s + 3 < s_end) step(lds_a1, lds_b0, lds_a0, lds_b2, s + 3);
  if (s + 4 < s_end) step(lds_a0, lds_b1, lds_a1, lds_b0, s + 4);
  if constexpr (WN == 4) {
    if (wm == 0) __builtin_amdgcn_s_barrier();  // the barrier in the middle of the second half's last step
  }

  // ---- epilogue: scales, then a transpose through LDS so that every lane stores 16 contiguous bytes
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the last (unused) prefetch must not land on top of the transposes
  __syncthreads();
  float* epi = reinterpret_cast<float*>(wave < 4 ? lds_a0 : lds_a1) + (wave & 3) * (16 * kEpiStride);
  epi_elem_t<T>* out = static_cast<epi_elem_t<T>*>(p.out);
  const int mw = m0 + 16 * kMTW * wm, nw = n0 + 64 * wn;
  float ws[kNT];
#pragma unroll
  for (int t = 0; t < kNT; ++t) {
    const int col = nw + 16 * t + r;
    ws[t] = p.ksplit > 1 ? 1.f : p.w_scale[p.w_scale_per_col ? (col < p.N ? col : p.N - 1) : 0];
  }
  // split launch: the raw fp32 tile of this split, rows of 256 floats, for the reduction kernel
  float* part = p.ksplit > 1 ? p.partial + ((size_t)blockIdx.y * p.tail_tiles + (lid - p.lid_begin)) * 65536 : nullptr;
#pragma unroll
  for (int mt = 0; mt < kMTW; ++mt) {
#pragma unroll
    for (int t = 0; t < kNT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) epi[(4 * j + i) * kEpiStride + 16 * t + r] = acc[mt][t][i] * ws[t];
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
      const int rr = (lane >> 3) + 8 * pass, cc = (lane & 7) * 8;
      const float* src = epi + rr * kEpiStride + cc;
      const int row = mw + 16 * mt + rr, col = nw + cc;
      if (part) {
        if (row < p.M) {  // the reduction kernel reads no row past M either (whole tiles only: WN = 4)
          f32x4* dst = reinterpret_cast<f32x4*>(part + (16 * kMTW * wm + 16 * mt + rr) * 256 + 64 * wn + cc);
          dst[0] = f32x4{src[0], src[1], src[2], src[3]};
          dst[1] = f32x4{src[4], src[5], src[6], src[7]};
        }
        continue;
      }
      const float as = p.a_scale[p.a_scale_per_row ? (row < p.M ? row : p.M - 1) : 0];
      float vals[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) vals[q] = src[q] * as;
      epi_store_row8_wave<T>(p.epi, out, vals, row, col, p.N, row < p.M && col + 8 <= p.N, row < p.M, lane);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
  }
}

// Second half of the split tail launch of the 256 x 256 kernel: one thread per eight consecutive columns of a tail
// tile; adds the splits in order, applies the scales and the epilogue.
template <typename T>
__global__ __launch_bounds__(256) void fp8_tail_reduce_kernel(Fp8PrefillArgs p) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;  // [tail tile][256 rows][32 segments]
  const int tile = (int)(idx >> 13), rr = (int)(idx >> 5) & 255, seg = (int)idx & 31;
  if (tile >= p.tail_tiles) return;
  int mb, nb;
  if (!tile_of(p.lid_begin + tile, p.mblocks, p.nblocks, &mb, &nb)) return;
  const int row = mb * 256 + rr, col = nb * 256 + seg * 8;
  if (row >= p.M || col + 8 > p.N) return;
  const f32x4* src = reinterpret_cast<const f32x4*>(p.partial + (size_t)tile * 65536 + rr * 256 + seg * 8);
  const size_t stride = (size_t)p.tail_tiles * 65536 / 4;
  f32x4 lo = src[0], hi = src[1];
  for (int sp = 1; sp < p.ksplit; ++sp) {
    lo += src[sp * stride];
    hi += src[sp * stride + 1];
  }
  const float as = p.a_scale[p.a_scale_per_row ? row : 0];
  float vals[8];
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const float w = p.w_scale[p.w_scale_per_col ? col + q : 0];
    vals[q] = ((q < 4 ? lo[q] : hi[q - 4]) * w) * as;  // the order of the one-launch epilogue: column scale, then row scale
  }
  const float mx = epi_store_row8<T>(p.epi, static_cast<epi_elem_t<T>*>(p.out), vals, row, col, p.N);
  if (p.epi.row_absmax) atomicMax(reinterpret_cast<unsigned*>(p.epi.row_absmax) + row, __builtin_bit_cast(unsigned, mx));
}

}  // namespace

// A grid of 256 x 256 tiles runs in rounds of one workgroup per CU.  When the last round is at most half full and K
// is long, its tiles go out as a launch of their own with K split so that it fills the device: every split stores its
// raw fp32 tile with plain stores and a reduction kernel finishes (the Qwen-72B qkv shape at M = 2048 is 320 tiles
// on 256 CUs: a second round a quarter full).  Returns the split count (1 = no split) and the tiles in the tail.
static int fp8_tail_split(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes, int* tail_tiles, size_t* need,
                          bool* quarters) {
  *tail_tiles = 0;
  *need = 0;
  *quarters = false;
  if (cus <= 0 || cus % 8 != 0) return 1;  // the main launch's tile count has to stay a multiple of eight
  const size_t total = ((m + 255) / 256) * ((n + 255) / 256), per_round = (size_t)cus;
  if (total <= per_round) {
    // A single round.  With at most half the CUs holding a tile and K long, the whole grid is the "tail": K split
    // so that the splits fill the device, 12 k stages each at least (Qwen-72B qkv at M = 256: 40 tiles, 86 us unsplit;
    // a sweep of every split count at M = 96 .. 1024: with 16 stages at least, o at M = 96 .. 256 ran 5 to 8 % and a
    // K = 11008, N = 4096 shape 8 to 11 % behind their best, with 10 qkv loses 3 %).
    size_t ks = per_round / total;
    if (ks > 8) ks = 8;
    if (ks > k / 128 / 12) ks = k / 128 / 12;
    if (const char* e = tuning_env("KSQ_FP8_TAIL_KSPLIT")) {  // tuning / test override (1 switches the split off)
      const int v = atoi(e);
      if (v >= 1 && v <= 8 && (size_t)v <= k / 128) ks = (size_t)v;
    }
    const size_t bytes = ks * total * 65536 * 4;
    if (ks <= 1 || bytes > workspace_bytes) return 1;
    *tail_tiles = (int)total;
    *need = bytes;
    return (int)ks;
  }
  const size_t rem = total % per_round;
  // A last round that covers at most a quarter of the CUs goes out as column quarters of its tiles (256 x 64, four
  // workgroups to a tile, no K split and nothing through memory)
  bool use_quarters = rem != 0 && 4 * rem <= per_round;
  if (const char* e = tuning_env("KSQ_FP8_TAIL_QUARTERS")) use_quarters = use_quarters && atoi(e) != 0;  // tuning switch
  if (use_quarters) {
    *tail_tiles = (int)rem;
    *quarters = true;
    return 1;
  }
  // measured at the Qwen-72B shapes, M = 2048: qkv (one full round + a quarter) 194 -> 186 us; gate_up (seven rounds
  // + a quarter) no gain, so grids of four rounds or more are left alone
  if (rem == 0 || 2 * rem > per_round || k / 128 < 32 || total >= 4 * per_round) return 1;
  size_t ks = per_round / rem;
  if (ks > 4) ks = 4;
  if (const char* e = tuning_env("KSQ_FP8_TAIL_KSPLIT")) {  // tuning / test override (1 switches the split off)
    const int v = atoi(e);
    if (v >= 1 && v <= 8 && (size_t)v <= k / 128) ks = (size_t)v;
  }
  const size_t bytes = ks * rem * 65536 * 4;
  if (ks <= 1 || bytes > workspace_bytes) return 1;
  *tail_tiles = (int)rem;
  *need = bytes;
  return (int)ks;
}

size_t fp8_prefill_workspace_bytes(size_t m, size_t n, size_t k, int cus) {
  int tail = 0;
  size_t need = 0;
  bool quarters = false;
  fp8_tail_split(m, n, k, cus, (size_t)-1, &tail, &need, &quarters);
  return need;
}

bool fp8_prefill_supported(size_t m, size_t n, size_t k, int cus) {
  // From 65 rows on (the decode kernels end at 64; the streaming fallback is several times slower than a padded
  // 256-row tile with K split over the grid).  From 17 rows on shapes whose columns fill the device several times
  // over, or fill it with a K long enough to split (measured on the Qwen-72B shapes against the decode kernel:
  // gate_up 111 -> 99 us at M = 17 .. 32 and 139 -> 101 .. 117 at M = 64, down 73 -> 56 and 89 -> 59; qkv and o lose
  // 10 to 50 %, and so do the wide shapes at 16 rows and fewer).
  const size_t ntiles = n / 16, ks = k / 128;
  size_t min_m = (ntiles >= 4 * (size_t)cus || (ntiles >= 2 * (size_t)cus && ks >= 128)) ? 17 : 65;
  if (const char* e = tuning_env("KSQ_FP8_PREFILL_MIN_M")) {  // tuning / test override
    const int v = atoi(e);
    if (v >= 1) min_m = (size_t)v;
  }
  return m >= min_m && n % 8 == 0 && k % 128 == 0 && m * k < 0x7FFFFF00ull && n * k < 0x7FFFFF00ull;
}

int fp8_launch_prefill(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                       const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                       void* workspace, size_t workspace_bytes, hipStream_t s, const Epilogue& epi) {
  KSQ_REQUIRE((reinterpret_cast<uintptr_t>(out) & 15) == 0, KSQ_ERR_INVALID_ARGUMENT, "output must be 16-byte aligned");
  Fp8PrefillArgs a{};
  a.epi = epi;
  a.aq = static_cast<const uint8_t*>(act_q);
  a.wq = static_cast<const uint8_t*>(w_q);
  a.a_scale = act_scale;
  a.w_scale = w_scale;
  a.out = out;
  a.M = (int)m;
  a.N = (int)n;
  a.K = (int)k;
  a.KS = (int)(k / 128);
  a.a_scale_per_row = act_scale_count > 1;
  a.w_scale_per_col = w_scale_count > 1;
  // 256 x 256 tiles (one workgroup of eight waves per CU): measured on the Qwen-72B shapes that kernel sustains 1.7
  // times the rate of the 128 x 256 one and is the faster one from M = 128 on (at M = 128, where half of every tile
  // is padding, by 8 to 18 %; it also has the K split that partly empty grids need).  The 128 x 256 kernel stays
  // reachable through the override, which the parity tests use.
  int tile = 256;
  if (const char* e = tuning_env("KSQ_FP8_PREFILL_TILE")) {  // tuning / test override
    const int v = atoi(e);
    if (v == 128 || v == 256) tile = v;
  }
  a.lid_begin = 0;
  a.ksplit = 1;
  a.tail_tiles = 0;
  a.partial = nullptr;
  if (tile == 256) {
    a.mblocks = (int)((m + 255) / 256);
    a.nblocks = (int)((n + 255) / 256);
    const size_t total = (size_t)a.mblocks * a.nblocks;
    KSQ_REQUIRE(total < (1ull << 30), KSQ_ERR_UNSUPPORTED, "grid too large");
    const DeviceInfo* di = device_info();
    KSQ_REQUIRE(di != nullptr, KSQ_ERR_HIP, "no device");
    int tail_tiles = 0;
    size_t need = 0;
    const bool ws_ok = workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0;
    bool quarters = false;
    const int ks = fp8_tail_split(m, n, k, di->cus, ws_ok ? workspace_bytes : 0, &tail_tiles, &need, &quarters);
    // without a tail launch the one launch covers everything, rounded up to a multiple of eight; with one, the main
    // launch covers whole rounds (a multiple of eight by itself)
    const size_t main_tiles = (ks > 1 || quarters) ? total - (size_t)tail_tiles : tile_grid(a.mblocks, a.nblocks);
    if (main_tiles) note_launch("fp8_prefill256_kernel grid=(%zu)", main_tiles);
    if (quarters) note_launch("fp8_prefill256_kernel<quarters> tiles=%d", tail_tiles);
    else if (ks > 1) note_launch("fp8_prefill256_kernel<ksplit=%d> tiles=%d + fp8_tail_reduce_kernel", ks, tail_tiles);
#define KSQ_BY_TYPE(KERNEL, GRID, BLOCK, ARGS)                                                  \
  do {                                                                                        \
    if (out_dtype == KSQ_F16) hipLaunchKernelGGL((KERNEL<_Float16>), GRID, BLOCK, 0, s, ARGS); \
    else if (out_dtype == KSQ_F32) hipLaunchKernelGGL((KERNEL<float>), GRID, BLOCK, 0, s, ARGS); \
    else hipLaunchKernelGGL((KERNEL<__bf16>), GRID, BLOCK, 0, s, ARGS);                        \
  } while (0)
    if (main_tiles == 0) {
      // every tile is in the split launch
    } else {
      KSQ_BY_TYPE(fp8_prefill256_kernel, dim3((unsigned)main_tiles), dim3(512), a);
    }
    if (quarters) {
      Fp8PrefillArgs t = a;
      t.lid_begin = (int)main_tiles;
      const dim3 qgrid((unsigned)((4 * (size_t)tail_tiles + 7) / 8 * 8));
      if (out_dtype == KSQ_F16)
        hipLaunchKernelGGL((fp8_prefill256_kernel<_Float16, 1>), qgrid, dim3(512), 0, s, t);
      else if (out_dtype == KSQ_F32)
        hipLaunchKernelGGL((fp8_prefill256_kernel<float, 1>), qgrid, dim3(512), 0, s, t);
      else
        hipLaunchKernelGGL((fp8_prefill256_kernel<__bf16, 1>), qgrid, dim3(512), 0, s, t);
    } else if (ks > 1) {
      Fp8PrefillArgs t = a;
      t.lid_begin = (int)main_tiles;
      t.ksplit = ks;
      t.tail_tiles = tail_tiles;
      t.partial = static_cast<float*>(workspace);
      const dim3 tgrid((unsigned)((tail_tiles + 7) / 8 * 8), (unsigned)ks), rgrid((unsigned)((size_t)tail_tiles * 8192 / 256));
      KSQ_BY_TYPE(fp8_prefill256_kernel, tgrid, dim3(512), t);
      KSQ_BY_TYPE(fp8_tail_reduce_kernel, rgrid, dim3(256), t);
    }
  } else {
    a.mblocks = (int)((m + kBM - 1) / kBM);
    a.nblocks = (int)((n + kBN - 1) / kBN);
    KSQ_REQUIRE((size_t)a.mblocks * a.nblocks < (1ull << 30), KSQ_ERR_UNSUPPORTED, "grid too large");
    const dim3 grid(tile_grid(a.mblocks, a.nblocks));
    note_launch("fp8_prefill_kernel grid=(%u)", grid.x);
    KSQ_BY_TYPE(fp8_prefill_kernel, grid, dim3(256), a);
  }
#undef KSQ_BY_TYPE
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

}  // namespace ksq
