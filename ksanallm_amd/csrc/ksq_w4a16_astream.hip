// W4A16 decode kernel for 17 <= M <= 64: accumulator-stationary, both operands streamed.
//
// With two to four 16-row tiles the activations of a decode step no longer fit into the registers of one workgroup
// for the whole of K, so here nothing but the accumulators stays: a workgroup (8 waves, two per SIMD) owns CNT
// column tiles for all of K, wave w owns a contiguous slice of the k tiles, and for every k tile of its slice it
// streams the activation fragments of all MT row tiles (from the L2: every workgroup reads all activations once) and
// the CNT weight tiles (from HBM, once per device), one k tile ahead for the weights and half a k tile ahead for the
// activations.  No barrier and no LDS until the end, where the 8 k slices of every (column tile, row tile) are
// summed through LDS in a fixed order.
//
// Every workgroup reads all activations of its k range from the L2, M x K x 2 bytes for one to four weight tiles of
// K x 8 bytes each: with few column tiles per compute unit that is most of what a compute unit moves.  K is then
// split over grid.y as well (two or four ways), which divides that traffic; the partial tiles of the splits go
// through the workspace and the last workgroup to arrive at a tile adds them in split order (deterministic).
//
// Activation loads put lane l on row l / 4 and 16-byte piece l % 4 of a 32-k step, so that every aligned group of
// four lanes reads 64 contiguous bytes (the memory pipeline then takes four lanes per clock instead of one); a lane
// permutation gives the MFMA operand layout (lane 16 j + c = row c, piece j).
//
// Arithmetic, bf16: biased nibbles by bit operations (every nibble as bias + u with one bias); fp32 sums over 64 k
// of a (bias + u) by MFMA, the bias and the zero point removed through the row sums of the activations (one more
// MFMA per row tile and 32-k step, shared by all column tiles), scaled by s[g,n]: the weights stay exact, which bf16
// needs.  fp16: the weights are dequantised to T((u - z) s) in registers and accumulated directly.
#include <cstdlib>

#include "ksq_epilogue.h"
#include "ksq_internal.h"
#include "ksq_w4a16_ops.h"

namespace ksq {
namespace {

using namespace w4;

struct AstreamArgs {
  const void* weight;  // [ntiles][KT][64] x 16 B
  const void* sz;      // [ntiles][G][16] x 4 B
  const void* act;     // [M][K] T
  void* out;           // [M][N] T
  int M, N, K, KT, G, ntiles;
  int ksplit;          // grid.y
  f32x4* partial;      // [ksplit][ntiles][MT][64], ksplit > 1 only
  unsigned* counters;  // [ntiles][MT], zero between launches
  Epilogue epi;
};

// k tiles [begin, end) of wave `wave` of the workgroup of split blockIdx.y
struct KRange {
  int wg_begin, begin, end;
};
__device__ inline KRange astream_k_range(const AstreamArgs& p, int wave) {
  KRange r;
  int wg_end;
  split_range(p.KT, blockIdx.y, p.ksplit, &r.wg_begin, &wg_end);
  const int slice = (wg_end - r.wg_begin + 7) / 8;
  r.begin = r.wg_begin + wave * slice;
  r.end = r.begin + slice < wg_end ? r.begin + slice : wg_end;
  // The 64-bit divisions above run on the vector unit, and a value that crosses a basic block in a vector register
  // counts as divergent from there on: every global -> LDS load whose scalar offset derives from it would be wrapped
  // in a readfirstlane loop.  The values are uniform; say so.
  r.wg_begin = __builtin_amdgcn_readfirstlane(r.wg_begin);
  r.begin = __builtin_amdgcn_readfirstlane(r.begin);
  r.end = __builtin_amdgcn_readfirstlane(r.end);
  return r;
}

// What a wave does with output tile (column tile nt, row tile mt) once the k slices of its workgroup are summed:
// store it, or with K split over workgroups park it and, as the last split to arrive, add all of them up first.
// Every lane of the wave makes the call.
template <typename T, int MT>
__device__ inline void astream_finish_tile(const AstreamArgs& p, f32x4 sum, int nt, int mt, int lane) {
  bool store = true;
  if (p.ksplit > 1) {
    const size_t stride = (size_t)p.ntiles * MT * 64;
    const size_t tile = ((size_t)nt * MT + mt) * 64 + lane;
    store_agent(p.partial + (size_t)blockIdx.y * stride + tile, sum);
    unsigned* counter = p.counters + nt * MT + mt;
    store = splitk_arrive_last(counter, lane, p.ksplit);
    if (store) {
      sum = f32x4{0.f, 0.f, 0.f, 0.f};
      for (int sp = 0; sp < p.ksplit; ++sp) sum += load_agent(p.partial + (size_t)sp * stride + tile);
      if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (store)
    epi_store_acc<T>(p.epi, static_cast<uint16_t*>(p.out), sum, 16 * mt + 4 * (lane >> 4), nt * 16 + (lane & 15), p.M,
                     p.N, true);
}

template <typename T, int GPT, int MT, int CNT>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void w4a16_astream_kernel(AstreamArgs p) {
  using O = Ops<T>;
  constexpr int kWaves = 8;
  constexpr int kTiles = CNT * MT;  // output tiles of the workgroup
  __shared__ f32x4 red[kTiles * kWaves * 64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, j = lane >> 4;
  const int nt_begin = blockIdx.x * CNT;
  int count = p.ntiles - nt_begin;
  count = count < CNT ? count : CNT;
  // k slice of this wave (the loop below prefetches one tile ahead; tiles past the end are parked out of range and
  // read as zero)
  const KRange kr = astream_k_range(p, wave);
  const int kt_begin = kr.begin, kt_end = kr.end;

  // Resources cover exactly this workgroup's column tiles: tiles past `count` read as zero without traffic.
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(p.weight) + (size_t)nt_begin * p.KT * 1024), 0,
      count > 0 ? count * p.KT * 1024 : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_sz = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(p.sz) + (size_t)nt_begin * p.G * 64), 0, count > 0 ? count * p.G * 64 : 0,
      0x00020000);
  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.act), 0, (int)((size_t)p.M * p.K * 2), 0x00020000);
  const unsigned w_stride = (unsigned)p.KT * 1024u, sz_stride = (unsigned)p.G * 64u;
  const unsigned w_lane = lane * 16u, sz_lane = c * 4u;
  // loading lane: row l / 4 of the row tile, piece l % 4 of the 32-k step
  unsigned a_row[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int row = 16 * mt + (lane >> 2);
    a_row[mt] = row < p.M ? ((unsigned)row * p.K + 8u * (lane & 3)) * 2u : 0x80000000u;
  }
  const int from = (4 * c + j) * 4;  // lane 16 j + c takes what lane 4 c + j loaded

  struct WTile {
    u32x4 w[CNT];
    uint32_t sz[CNT][GPT];
  };
  // The per-lane part of every address is a loop constant and the moving part (k tile, column tile) goes into the
  // scalar offset of the buffer instruction, which costs no vector arithmetic.  The hardware checks only the vector
  // offset against the resource's range, so whatever must read as zero (a k tile past the slice, a column tile past
  // the workgroup's range, a row past M) is parked there, at an offset that is out of range by itself.
  auto load_w = [&](WTile& t, int kt) {
    const bool ok = kt < kt_end;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const bool live = ok && i < count;  // uniform
      t.w[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w, live ? w_lane : 0x80000000u,
                                                                               __builtin_amdgcn_readfirstlane(live ? kt * 1024 + i * (int)w_stride : 0), 2));
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi)
        t.sz[i][gi] = __builtin_amdgcn_raw_buffer_load_b32(rs_sz, live ? sz_lane : 0x80000000u,
                                                           __builtin_amdgcn_readfirstlane(live ? (kt * GPT + gi) * 64 + i * (int)sz_stride : 0), 0);
    }
  };
  // half h of k tile kt: 32-k steps 2h and 2h + 1 of all row tiles, as loaded (before the lane permutation)
  auto load_a = [&](u32x4 (&a)[MT][2], int kt, int h) {
    const bool ok = kt < kt_end;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int dd = 0; dd < 2; ++dd)
        a[mt][dd] = __builtin_bit_cast(
            u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_a, ok ? a_row[mt] : 0x80000000u,
                                                         ok ? (kt * kTileK + 32 * (2 * h + dd)) * 2 : 0, 0));
  };
  auto permute = [&](u32x4 (&a)[MT][2]) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int dd = 0; dd < 2; ++dd)
#pragma unroll
        for (int q = 0; q < 4; ++q) a[mt][dd][q] = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)a[mt][dd][q]);
  };

  uint32_t m_lo = O::kMaskLo, m_hi = O::kMaskHi, c_lo = O::kMagicLo, c_hi = O::kMagicHi;
  KSQ_PIN_SGPR(m_lo);
  KSQ_PIN_VGPR(c_lo);
  KSQ_PIN_VGPR(c_hi);
  KSQ_PIN_VGPR(m_hi);

  f32x4 acc[CNT][MT];
#pragma unroll
  for (int i = 0; i < CNT; ++i)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[i][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // 64 k of all column tiles against all row tiles
  // sum_k a (u - z) = sum_k a (bias + u) - (bias + z) sum_k a: the row sums of the activations (an MFMA against
  // ones) serve every column tile, so the bias and the zero point cost one multiply-add per output.
  auto compute_half = [&](const u32x4 (&a)[MT][2], const WTile& t, int h) {
    if constexpr (__is_same(T, _Float16)) {
      // fp16: the weights are dequantised (T((u - z) s), rounded once) and multiplied straight into the
      // accumulators: with two or four row tiles that is fewer instructions than scaling every output per group
#pragma unroll
      for (int i = 0; i < CNT; ++i) {
        const typename Dequant<_Float16>::Consts k = Dequant<_Float16>::prepare(t.sz[i][GPT == 2 ? h : 0]);
#pragma unroll
        for (int dd = 0; dd < 2; ++dd) {
          const u32x4 bw = Dequant<_Float16>::run(t.w[i][2 * h + dd], k, m_lo, m_hi, c_lo, c_hi);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[i][mt] = O::mfma(a[mt][dd], bw, acc[i][mt]);
        }
      }
      return;
    }
    const u32x4 ones = {O::kOnes, O::kOnes, O::kOnes, O::kOnes};
    f32x4 S[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) S[mt] = O::mfma(a[mt][0], ones, f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) S[mt] = O::mfma(a[mt][1], ones, S[mt]);
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const uint32_t szw = t.sz[i][GPT == 2 ? h : 0];
      const float s = O::scale_to_float(szw);
      const float nsz = -s * (O::kBias + (float)((szw >> 16) & 15u));  // exact: 11 x 11 significant bits
      f32x4 P[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) P[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dd = 0; dd < 2; ++dd) {
        const u32x4 bw = O::unpack_uniform(t.w[i][2 * h + dd], m_lo, c_lo);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) P[mt] = O::mfma(a[mt][dd], bw, P[mt]);
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i][mt][e] += s * P[mt][e] + nsz * S[mt][e];
    }
  };

  // One k tile: its weights (wc) and first activation half (a0) were requested a step earlier; request the second
  // half, the next tile's weights and first half, and run the two halves.
  u32x4 a0[MT][2], a1[MT][2];
  WTile w0, w1;
  auto tile = [&](WTile& wc, WTile& wn, int kt, int kt_next) {
    load_a(a1, kt, 1);
    load_w(wn, kt_next);
    __builtin_amdgcn_sched_barrier(0);
    permute(a0);
    compute_half(a0, wc, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_a(a0, kt_next, 0);
    __builtin_amdgcn_sched_barrier(0);
    permute(a1);
    compute_half(a1, wc, 1);
    __builtin_amdgcn_sched_barrier(0);
  };

  load_w(w0, kt_begin);
  load_a(a0, kt_begin, 0);
  __builtin_amdgcn_sched_barrier(0);
  for (int kt = kt_begin; kt < kt_end; kt += 2) {
    tile(w0, w1, kt, kt + 1);
    if (kt + 1 >= kt_end) break;  // odd slice: what was prefetched for the missing tile is zeros
    tile(w1, w0, kt + 1, kt + 2);
  }

  // ---- sum the 8 k slices of every output tile (fixed order: deterministic), one tile per wave and turn
#pragma unroll
  for (int i = 0; i < CNT; ++i)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) red[((i * MT + mt) * kWaves + wave) * 64 + lane] = acc[i][mt];
  __syncthreads();
  for (int q = wave; q < kTiles; q += kWaves) {
    const int i = q / MT, mt = q - i * MT;
    // all eight reads first (one LDS round trip instead of four), then the sum in wave order
    f32x4 part[kWaves];
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) part[ww] = red[(q * kWaves + ww) * 64 + lane];
    __builtin_amdgcn_sched_barrier(0);
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) sum += part[ww];
    if (i < count) astream_finish_tile<T, MT>(p, sum, nt_begin + i, mt, lane);
  }
}

// The same decomposition with the activations staged through LDS: every wave owns two buffers of half a k tile
// (all MT row tiles x 64 k) and fills them with global -> LDS loads (no registers, no lane permutation), one half ahead;
// the MFMA operands are then plain 16-byte LDS reads.  A block of 1 KiB is one load instruction = one 32-k step of
// one row tile: lane l brings piece (l & 3) ^ (l >> 4) of row l >> 2 and lands at l * 16, so that every aligned group
// of four lanes reads 64 contiguous bytes from memory and the sixteen lanes that later read piece j of rows 0..15
// hit sixteen different bank groups.  Nothing is shared between waves, so the only synchronisation is the wave's own
// vmcnt; the buffers of all waves together are reused for the final reduction.
typedef __attribute__((address_space(3))) void* lds_ptr;

// s_waitcnt vmcnt(N) alone, N a constant expression (6-bit count in bits 3:0 and 15:14 of the immediate, the other
// counters at their maxima).  Expanded in place with literal immediates: the builtin takes no value-dependent
// argument, and a call from a __device__ helper template loses the kernel's host-side stub.
#define KSQ_WAIT_VMCNT(N) \
  if constexpr ((N) == 0) __builtin_amdgcn_s_waitcnt(0x0F70); \
  else if constexpr ((N) == 1) __builtin_amdgcn_s_waitcnt(0x0F71); \
  else if constexpr ((N) == 2) __builtin_amdgcn_s_waitcnt(0x0F72); \
  else if constexpr ((N) == 3) __builtin_amdgcn_s_waitcnt(0x0F73); \
  else if constexpr ((N) == 4) __builtin_amdgcn_s_waitcnt(0x0F74); \
  else if constexpr ((N) == 5) __builtin_amdgcn_s_waitcnt(0x0F75); \
  else if constexpr ((N) == 6) __builtin_amdgcn_s_waitcnt(0x0F76); \
  else if constexpr ((N) == 7) __builtin_amdgcn_s_waitcnt(0x0F77); \
  else if constexpr ((N) == 8) __builtin_amdgcn_s_waitcnt(0x0F78); \
  else if constexpr ((N) == 9) __builtin_amdgcn_s_waitcnt(0x0F79); \
  else if constexpr ((N) == 10) __builtin_amdgcn_s_waitcnt(0x0F7A); \
  else if constexpr ((N) == 11) __builtin_amdgcn_s_waitcnt(0x0F7B); \
  else if constexpr ((N) == 12) __builtin_amdgcn_s_waitcnt(0x0F7C); \
  else if constexpr ((N) == 13) __builtin_amdgcn_s_waitcnt(0x0F7D); \
  else if constexpr ((N) == 14) __builtin_amdgcn_s_waitcnt(0x0F7E); \
  else if constexpr ((N) == 15) __builtin_amdgcn_s_waitcnt(0x0F7F); \
  else if constexpr ((N) == 16) __builtin_amdgcn_s_waitcnt(0x4F70); \
  else if constexpr ((N) == 17) __builtin_amdgcn_s_waitcnt(0x4F71); \
  else if constexpr ((N) == 18) __builtin_amdgcn_s_waitcnt(0x4F72); \
  else if constexpr ((N) == 19) __builtin_amdgcn_s_waitcnt(0x4F73); \
  else if constexpr ((N) == 20) __builtin_amdgcn_s_waitcnt(0x4F74); \
  else static_assert((N) <= 20, "add the immediate")

// 16-byte elements of each of the two LDS objects: the activation halves of eight waves, or half of the final
// reduction (8 partial tiles per output tile), whichever is larger
template <int MT, int CNT>
struct AstreamLds {
  static constexpr int kHalf = MT * 2 * 64;
  static constexpr int kRedHalf = (CNT * MT + 1) / 2 * 8 * 64;
  static constexpr int value = 8 * kHalf > kRedHalf ? 8 * kHalf : kRedHalf;
};

template <typename T, int GPT, int MT, int CNT>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void w4a16_astream_lds_kernel(AstreamArgs p) {
  using O = Ops<T>;
  constexpr int kWaves = 8;
  constexpr int kTiles = CNT * MT;          // output tiles of the workgroup
  constexpr int kHalf = MT * 2 * 64;        // 16-byte elements of half a k tile of activations (MT x 2 blocks)
  // two separate objects: loads into one are then known not to alias reads of the other
  __shared__ u32x4 buf0[AstreamLds<MT, CNT>::value];
  __shared__ u32x4 buf1[AstreamLds<MT, CNT>::value];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, j = lane >> 4;
  const int nt_begin = blockIdx.x * CNT;
  int count = p.ntiles - nt_begin;
  count = count < CNT ? count : CNT;
  const KRange kr = astream_k_range(p, wave);
  const int kt_begin = kr.begin, kt_end = kr.end;

  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(p.weight) + (size_t)nt_begin * p.KT * 1024), 0,
      count > 0 ? count * p.KT * 1024 : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_sz = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(p.sz) + (size_t)nt_begin * p.G * 64), 0, count > 0 ? count * p.G * 64 : 0,
      0x00020000);
  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.act), 0, (int)((size_t)p.M * p.K * 2), 0x00020000);
  const unsigned w_stride = (unsigned)p.KT * 1024u, sz_stride = (unsigned)p.G * 64u;
  const unsigned w_lane = lane * 16u, sz_lane = c * 4u;
  // loading lane: row l / 4 of the row tile (rows past M repeat row M - 1: their results are never stored), piece
  // (l & 3) ^ (l >> 4) of the 32-k step
  unsigned a_row[4];  // MT of them in use (a fixed size: with a dependent one the kernel loses its host-side stub)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int row = 16 * mt + (lane >> 2);
    row = row < p.M ? row : p.M - 1;
    a_row[mt] = ((unsigned)row * p.K + 8u * ((lane & 3) ^ (lane >> 4))) * 2u;
  }
  // where lane (c, j) finds piece j of row c inside a block, in 16-byte units
  const int a_lane = c * 4 + (j ^ (c >> 2));

  struct WTile {
    u32x4 w[CNT];
    uint32_t sz[CNT][GPT];
  };
  auto load_w = [&](WTile& t, int kt) {
    const bool ok = kt < kt_end;
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const bool live = ok && i < count;  // uniform
      t.w[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w, live ? w_lane : 0x80000000u,
                                                                               __builtin_amdgcn_readfirstlane(live ? kt * 1024 + i * (int)w_stride : 0), 2));
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi)
        t.sz[i][gi] = __builtin_amdgcn_raw_buffer_load_b32(rs_sz, live ? sz_lane : 0x80000000u,
                                                           __builtin_amdgcn_readfirstlane(live ? (kt * GPT + gi) * 64 + i * (int)sz_stride : 0), 0);
    }
  };
  // half h of k tile kt into this wave's part of `buf`.  A tile past the slice repeats the slice's first tile (the
  // workgroup's first for a wave whose slice is empty): its weights read as zero, so whatever finite activations stand in for it
  // contribute nothing.  The scalar offset is not range-checked by the hardware, hence the clamp.
  const int kt_safe = kt_begin < kt_end ? kt_begin : kr.wg_begin;
  auto load_a = [&](u32x4* buf, int kt, int h) {
    const int ktc = kt < kt_end ? kt : kt_safe;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int dd = 0; dd < 2; ++dd)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(buf + wave * kHalf + (mt * 2 + dd) * 64), 16, a_row[mt],
                                                 (ktc * kTileK + 32 * (2 * h + dd)) * 2, 0, 0);
  };
  auto read_a = [&](u32x4 (&a)[MT][2], const u32x4* buf) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int dd = 0; dd < 2; ++dd) a[mt][dd] = buf[wave * kHalf + (mt * 2 + dd) * 64 + a_lane];
  };

  uint32_t m_lo = O::kMaskLo, m_hi = O::kMaskHi, c_lo = O::kMagicLo, c_hi = O::kMagicHi;
  KSQ_PIN_SGPR(m_lo);
  KSQ_PIN_VGPR(c_lo);
  KSQ_PIN_VGPR(c_hi);
  KSQ_PIN_VGPR(m_hi);

  f32x4 acc[CNT][MT];
#pragma unroll
  for (int i = 0; i < CNT; ++i)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[i][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto compute_half = [&](const u32x4 (&a)[MT][2], const WTile& t, int h) {
    if constexpr (__is_same(T, _Float16)) {
#pragma unroll
      for (int i = 0; i < CNT; ++i) {
        const typename Dequant<_Float16>::Consts k = Dequant<_Float16>::prepare(t.sz[i][GPT == 2 ? h : 0]);
#pragma unroll
        for (int dd = 0; dd < 2; ++dd) {
          const u32x4 bw = Dequant<_Float16>::run(t.w[i][2 * h + dd], k, m_lo, m_hi, c_lo, c_hi);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) acc[i][mt] = O::mfma(a[mt][dd], bw, acc[i][mt]);
        }
      }
      return;
    }
    const u32x4 ones = {O::kOnes, O::kOnes, O::kOnes, O::kOnes};
    f32x4 S[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) S[mt] = O::mfma(a[mt][0], ones, f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) S[mt] = O::mfma(a[mt][1], ones, S[mt]);
#pragma unroll
    for (int i = 0; i < CNT; ++i) {
      const uint32_t szw = t.sz[i][GPT == 2 ? h : 0];
      const float s = O::scale_to_float(szw);
      const float nsz = -s * (O::kBias + (float)((szw >> 16) & 15u));
      f32x4 P[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) P[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int dd = 0; dd < 2; ++dd) {
        const u32x4 bw = O::unpack_uniform(t.w[i][2 * h + dd], m_lo, c_lo);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) P[mt] = O::mfma(a[mt][dd], bw, P[mt]);
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i][mt][e] += s * P[mt][e] + nsz * S[mt][e];
    }
  };

  // One k tile.  On entry its weights (wc) and its first activation half (buf0) were requested a step earlier.  Of the
  // memory instructions issued since a half was requested, the ones still allowed in flight when it is read:
  // the other half (MT x 2 loads) and one weight tile (CNT x (1 + GPT) loads).
  u32x4 a[MT][2];
  WTile w0, w1;
  auto tile = [&](WTile& wc, WTile& wn, int kt, int kt_next) {
    load_a(buf1, kt, 1);
    load_w(wn, kt_next);
    __builtin_amdgcn_sched_barrier(0);
    KSQ_WAIT_VMCNT(MT * 2 + CNT * (1 + GPT));
    read_a(a, buf0);
    compute_half(a, wc, 0);
    __builtin_amdgcn_sched_barrier(0);
    load_a(buf0, kt_next, 0);  // the reads of buf0 have returned: the MFMAs above consumed them
    __builtin_amdgcn_sched_barrier(0);
    KSQ_WAIT_VMCNT(MT * 2 + CNT * (1 + GPT));
    read_a(a, buf1);
    compute_half(a, wc, 1);
    __builtin_amdgcn_sched_barrier(0);
  };

  load_w(w0, kt_begin);
  load_a(buf0, kt_begin, 0);
  __builtin_amdgcn_sched_barrier(0);
  for (int kt = kt_begin; kt < kt_end; kt += 2) {
    tile(w0, w1, kt, kt + 1);
    if (kt + 1 >= kt_end) break;  // odd slice: what was prefetched for the missing tile is zeros
    tile(w1, w0, kt + 1, kt + 2);
  }

  // ---- sum the 8 k slices of every output tile (fixed order: deterministic), one tile per wave and turn.  The
  // activation buffers are free once every wave's last loads have landed and every wave has left the loop.
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the last (unused) prefetch
  __syncthreads();
  f32x4* red0 = reinterpret_cast<f32x4*>(buf0);
  f32x4* red1 = reinterpret_cast<f32x4*>(buf1);
  constexpr int kFirst = (kTiles + 1) / 2;  // tiles parked in buf0, the rest in buf1
#pragma unroll
  for (int i = 0; i < CNT; ++i)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int q = i * MT + mt;
      if (q < kFirst) red0[(q * kWaves + wave) * 64 + lane] = acc[i][mt];
      else red1[((q - kFirst) * kWaves + wave) * 64 + lane] = acc[i][mt];
    }
  __syncthreads();
  for (int q = wave; q < kTiles; q += kWaves) {
    const int i = q / MT, mt = q - i * MT;
    const f32x4* src = q < kFirst ? red0 + q * kWaves * 64 : red1 + (q - kFirst) * kWaves * 64;
    // all eight reads first (one LDS round trip instead of four), then the sum in wave order
    f32x4 part[kWaves];
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) part[ww] = src[ww * 64 + lane];
    __builtin_amdgcn_sched_barrier(0);
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ww = 0; ww < kWaves; ++ww) sum += part[ww];
    if (i < count) astream_finish_tile<T, MT>(p, sum, nt_begin + i, mt, lane);
  }
}

// Column tiles per workgroup that 256 registers per lane hold without spilling.  Weight-side dequantisation (fp16)
// and staging the activations in LDS both leave more registers for accumulators.
template <typename T, int GPT>
constexpr int cnt_max_of(int mt, bool lds) {
  if (mt == 2 || __is_same(T, _Float16)) return 4;
  if (lds) return GPT == 1 ? 4 : 3;
  return GPT == 1 ? 3 : 2;
}

// false: no instantiation for (mt, cnt, lds) -- nothing was launched
template <typename T, int GPT>
bool launch(int mt, int cnt, bool lds, const AstreamArgs& a, dim3 grid, hipStream_t s) {
  const dim3 block(512);
  bool launched = false;
#define KSQ_GO(MT, CNT)                                                                         \
  do {                                                                                          \
    if (lds) {                                                                                  \
      if constexpr (CNT <= cnt_max_of<T, GPT>(MT, true)) {                                      \
        hipLaunchKernelGGL((w4a16_astream_lds_kernel<T, GPT, MT, CNT>), grid, block, 0, s, a);  \
        launched = true;                                                                        \
      }                                                                                         \
    } else {                                                                                    \
      if constexpr (CNT <= cnt_max_of<T, GPT>(MT, false)) {                                     \
        hipLaunchKernelGGL((w4a16_astream_kernel<T, GPT, MT, CNT>), grid, block, 0, s, a);      \
        launched = true;                                                                        \
      }                                                                                         \
    }                                                                                           \
  } while (0)
  if (mt <= 2) {
    if (cnt == 1) KSQ_GO(2, 1);
    else if (cnt == 2) KSQ_GO(2, 2);
    else if (cnt == 3) KSQ_GO(2, 3);
    else if (cnt == 4) KSQ_GO(2, 4);
  } else if (mt == 3) {
    if (cnt == 1) KSQ_GO(3, 1);
    else if (cnt == 2) KSQ_GO(3, 2);
    else if (cnt == 3) KSQ_GO(3, 3);
    else if (cnt == 4) KSQ_GO(3, 4);
  } else {
    if (cnt == 1) KSQ_GO(4, 1);
    else if (cnt == 2) KSQ_GO(4, 2);
    else if (cnt == 3) KSQ_GO(4, 3);
    else if (cnt == 4) KSQ_GO(4, 4);
  }
#undef KSQ_GO
  return launched;
}

template <typename T, int GPT>
bool plan_and_launch(int mt, int cus, const AstreamArgs& a, hipStream_t s) {
  // column tiles per workgroup: one workgroup per CU (per CU and split) if that needs no more than fit, else the
  // split into whole rounds of workgroups that wastes least
  const int wgs = cus / a.ksplit > 0 ? cus / a.ksplit : 1;
  auto plan = [&](int cnt_max) {
    int cnt = (a.ntiles + wgs - 1) / wgs;
    if (cnt > cnt_max) {
      const int rounds = (a.ntiles + cnt_max * wgs - 1) / (cnt_max * wgs);
      cnt = (a.ntiles + rounds * wgs - 1) / (rounds * wgs);
    }
    if (const char* e = tuning_env("KSQ_W4_ASTREAM_CNT")) {  // tuning / test override
      const int v = atoi(e);
      if (v > 0) cnt = v;
    }
    cnt = cnt < 1 ? 1 : cnt;
    return cnt > cnt_max ? cnt_max : cnt;
  };
  // Activations through LDS once a k tile carries enough work (three column tiles or more) to hide the longer
  // global -> LDS -> register chain; through registers and a lane permutation below that (measured: 3 to 11 %
  // faster with three or four tiles, up to 8 % slower with one).
  int cnt = plan(cnt_max_of<T, GPT>(mt, true));
  bool lds = cnt >= 3;
  if (const char* e = tuning_env("KSQ_W4_ASTREAM_LDS")) lds = atoi(e) != 0;  // tuning / test override
  cnt = plan(cnt_max_of<T, GPT>(mt, lds));  // the limit of the form that runs, whichever way it was chosen
  const dim3 grid((unsigned)((a.ntiles + cnt - 1) / cnt), (unsigned)a.ksplit);
  note_launch("%s<mt=%d,cnt=%d,gpt=%d> grid=(%u,%u)", lds ? "w4a16_astream_lds_kernel" : "w4a16_astream_kernel", mt,
              cnt, GPT, grid.x, grid.y);
  return launch<T, GPT>(mt, cnt, lds, a, grid, s);
}

}  // namespace

bool w4a16_astream_supported(size_t m, size_t n, size_t k) {
  return m >= 17 && m <= 64 && m * k * 2 < 0x7FFFFF00ull && 4 * (k / kTileK) * 1024 < 0x7FFFFF00ull && n / kTileN < (1u << 30);
}

// K is split in two over workgroups while the column tiles alone give a compute unit at most two of them and the
// kernel is long enough for the hand-over through memory (about 3 us) to pay: always with four row tiles, from 80 k
// tiles on with two (measured on the o and down projections of Llama-2 7B and 70B: 3 to 29 % faster, four splits
// never better than two).  The element type plays no part, so the workspace can be sized without it.
AstreamPlan w4a16_astream_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes) {
  AstreamPlan p{};
  p.mt = m <= 32 ? 2 : (m <= 48 ? 3 : 4);  // row tiles past M cost their activation loads and matrix instructions
  if (const char* e = tuning_env("KSQ_W4_ASTREAM_MT")) {  // tuning / test override: never fewer than the rows need
    const int v = atoi(e);
    if (v >= 2 && v <= 4 && (size_t)v * 16 >= m) p.mt = v;
  }
  const size_t ntiles = n / kTileN, kt = k / kTileK;
  size_t ks = (ntiles <= 2 * (size_t)cus && kt >= 16 && (p.mt >= 3 || kt >= 80)) ? 2 : 1;
  if (const char* e = tuning_env("KSQ_W4_ASTREAM_KSPLIT")) {  // tuning / test override
    const size_t v = (size_t)atoi(e);
    if (v >= 1 && v <= 8 && v <= kt) ks = v;
  }
  if (ntiles * p.mt > (size_t)kCountersPerSlot) ks = 1;
  auto need = [&](size_t x) { return x <= 1 ? (size_t)0 : x * ntiles * p.mt * 64 * 16; };
  while (ks > 1 && need(ks) > workspace_bytes) --ks;
  p.ksplit = (int)ks;
  p.partial_bytes = need(ks);
  return p;
}

int w4a16_launch_astream(int dtype, const AstreamPlan& plan, void* out, const void* act, const void* weight,
                         const void* sz, size_t m, size_t n, size_t k, size_t g, int cus, void* workspace,
                         hipStream_t s, const Epilogue& epi) {
  AstreamArgs a{};
  a.epi = epi;
  a.weight = weight;
  a.sz = sz;
  a.act = act;
  a.out = out;
  a.M = (int)m;
  a.N = (int)n;
  a.K = (int)k;
  a.KT = (int)(k / kTileK);
  a.G = (int)(k / g);
  a.ntiles = (int)(n / kTileN);
  a.ksplit = plan.ksplit;
  a.partial = static_cast<f32x4*>(workspace);
  a.counters = nullptr;
  if (plan.ksplit > 1) {
    KSQ_REQUIRE(workspace != nullptr, KSQ_ERR_WORKSPACE, "split-K planned without a workspace");
    a.counters = counter_slot_device_ptr(s);
    KSQ_REQUIRE(a.counters != nullptr, KSQ_ERR_HIP, "split-K planned for a stream without arrival counters");
  }
  const int mt = plan.mt;
  const int gpt = (int)(kTileK / g);
  bool launched;
  if (dtype == KSQ_F16) {
    launched = gpt == 1 ? plan_and_launch<_Float16, 1>(mt, cus, a, s) : plan_and_launch<_Float16, 2>(mt, cus, a, s);
  } else {
    launched = gpt == 1 ? plan_and_launch<__bf16, 1>(mt, cus, a, s) : plan_and_launch<__bf16, 2>(mt, cus, a, s);
  }
  KSQ_REQUIRE(launched, KSQ_ERR_UNSUPPORTED, "no accumulator-stationary kernel for %d row tiles of this element type", mt);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

}  // namespace ksq
