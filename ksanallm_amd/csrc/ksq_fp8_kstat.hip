// FP8 e4m3 GEMM for M <= 64 (HBM-bound): k-stationary.
//
// A workgroup is 16 waves (8 for more than two row tiles, or for one row tile with a long K: twice the registers each).  Wave w keeps the activation fragments of its own TPW k stages (128 bytes of k each)
// for all MT row tiles in registers for the whole kernel and streams the weight rows of the workgroup's column
// range, for its own stages only, straight from HBM into a register ring, one batch of NB column tiles ahead.
// Nothing is re-read.  After every batch the 16 partial tiles of a (column tile, row tile) -- one per wave = per k
// slice -- are summed through LDS in a fixed order.  K beyond waves x TPW stages is split over grid.y and finished by
// the last-arriving workgroup through the workspace (partials in split order: deterministic).
//
// v_mfma_f32_16x16x128_f8f6f4 with both operands OCP e4m3 and no block scaling: lane (r, j) holds bytes
// [16j, 16j+16) and [64+16j, 64+16j+16) of row r's 128-byte stage, on both operands.  Pieces past K read as zero on
// both sides (K is a multiple of 16).  out = T(acc * w_scale[n] * a_scale[m]).
#include <cstdlib>

#include "ksq_epilogue.h"
#include "ksq_fp8_ops.h"
#include "ksq_internal.h"

namespace ksq {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x8 __attribute__((ext_vector_type(8)));

struct Fp8KstatArgs {
  const uint16_t* a_src;  // fused quantisation: the activations [M][K] as T, M <= 8; aq and a_scale are then unused
  const uint8_t* aq;  // [M][K]
  const uint8_t* wq;  // [N][K]
  const float* a_scale;
  const float* w_scale;
  void* out;           // [M][N] T
  f32x4* partial;      // [ksplit][ntiles][MT][64]
  unsigned* counters;  // [ntiles][MT]
  int M, N, K, KS /* stages, rounded up */, ntiles, ksplit, nt_per_wg;
  int a_scale_per_row, w_scale_per_col;
  Epilogue epi;
};

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

// FUSED: the kernel quantises its own activations (per token: one scale per row, Fp8E4m3Quantize of the reference
// with num_channels = m) instead of reading e4m3 bytes and scales: every workgroup takes the row maxima over the
// whole K, quantises the k range it works on into LDS -- the same arithmetic as the quantisation kernel, so the
// bytes are the same -- and its waves read their operand fragments from there.  Up to eight rows.
constexpr int kFusedRows = 8;
constexpr int kFusedRowBytes = 64 * 128 + 16;  // 64 stages per workgroup at most; 16 bytes of padding spread the banks

// AR = activation rows that one load instruction covers: 16 (lane l on row l / 4), or 4 for M <= 4 (lane l on row
// l / 4 % 4 of 64-byte chunk l / 16: four half stages per instruction instead of one; every vector memory instruction
// costs the compute unit the same whatever its lanes carry, and at one token the activation loads were a quarter of
// all loads of a workgroup).
template <typename T, int MT, int TPW, int NB, int NW, bool FUSED, int AR = 16>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(NW / 4))) void fp8_kstat_kernel(Fp8KstatArgs p) {
  static_assert(AR == 16 || (AR == 4 && MT == 1 && !FUSED), "narrow activation loads: one row tile, at most four rows");
  constexpr int D = NB * TPW;  // ring depth = one batch
  constexpr int NL = (2 * TPW + 3) / 4;  // AR = 4: load instructions for the 2 * TPW half stages of a wave
  static_assert(NB * MT * NW <= 64 && NB * MT <= NW, "two reduction buffers of at most 64 KiB, one tile per wave");
  static_assert(!FUSED || (MT == 1 && NB <= 2 && NW == 16 && TPW <= 4), "fused quantisation: one row tile, 64 KiB of LDS left");
  __shared__ f32x4 red[2 * NB * MT * NW * 64];
  __shared__ __attribute__((aligned(16))) uint8_t aq_lds[FUSED ? kFusedRows * kFusedRowBytes : 16];
  __shared__ float row_part[FUSED ? kFusedRows * NW : 1];
  __shared__ float row_scale[FUSED ? kFusedRows : 1];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, j = lane >> 4;
  const int split = blockIdx.y;
  int wg_begin, wg_end;
  split_range(p.KS, split, p.ksplit, &wg_begin, &wg_end);
  const int s0 = wg_begin + wave * TPW;  // first stage of this wave
  const int nt_begin = blockIdx.x * p.nt_per_wg;
  int count = p.ntiles - nt_begin;
  count = count < p.nt_per_wg ? count : p.nt_per_wg;
  const int nbatches = (p.nt_per_wg + NB - 1) / NB;  // same for every workgroup

  // The weight resource covers exactly the rows of this workgroup's column tiles (clipped to N): column tiles
  // past the range and rows past N read as zero without touching memory.
  int rows = count * 16;
  if (nt_begin * 16 + rows > p.N) rows = p.N - nt_begin * 16;
  if (rows < 0) rows = 0;
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(p.wq) + (size_t)nt_begin * 16 * p.K, 0, (int)((size_t)rows * p.K), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.aq), 0, (int)((size_t)p.M * p.K), 0x00020000);
  // Loads are issued with lane l on row l / 4 and 16-byte piece l % 4 of a 64-byte half stage, so that every aligned
  // group of four lanes reads 64 contiguous bytes (the memory pipeline then takes four lanes per clock instead of
  // one); a lane permutation (lane 16 j + r takes what lane 4 r + j loaded) gives the MFMA operand layout.
  // per stage and half: offset of the loading lane's 16 bytes inside its row, or out of range (stage past the
  // split's end, piece past K)
  const int lr = lane >> 2, lp = lane & 3;
  unsigned k_off[TPW][2];
#pragma unroll
  for (int t = 0; t < TPW; ++t)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const unsigned kb = (unsigned)(s0 + t) * 128u + 64u * h + 16u * lp;
      k_off[t][h] = (s0 + t < wg_end && kb + 16u <= (unsigned)p.K) ? kb : 0x80000000u;
    }
  // offset of this lane's piece of (stage t, half h) inside column tile 0; a parked offset stays out of range for
  // every column tile (the range of one workgroup is below 2^30 bytes)
  unsigned w_off[TPW][2];
#pragma unroll
  for (int t = 0; t < TPW; ++t)
#pragma unroll
    for (int h = 0; h < 2; ++h) w_off[t][h] = k_off[t][h] + (unsigned)lr * p.K;
  const unsigned w_stride = 16u * (unsigned)p.K;
  const int from = (4 * r + j) * 4;
  auto to_operand = [&](u32x4 lo, u32x4 hi) {
    i32x8 v;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      v[q] = __builtin_amdgcn_ds_bpermute(from, (int)lo[q]);
      v[4 + q] = __builtin_amdgcn_ds_bpermute(from, (int)hi[q]);
    }
    return v;
  };

  // activation fragments of this wave's stages: registers for the whole kernel
  i32x8 af[MT][TPW];
  u32x4 araw[AR == 4 ? NL : 1];
  if constexpr (AR == 4) {
#pragma unroll
    for (int u = 0; u < NL; ++u) {
      const int hs = 4 * u + (lane >> 4), t = hs >> 1, h = hs & 1, row = (lane >> 2) & 3;
      const unsigned kb = (unsigned)(s0 + t) * 128u + 64u * h + 16u * lp;
      const bool ok = hs < 2 * TPW && s0 + t < wg_end && kb + 16u <= (unsigned)p.K && row < p.M;
      araw[u] = __builtin_bit_cast(
          u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_a, ok ? (unsigned)row * p.K + kb : 0x80000000u, 0, 0));
    }
  } else if constexpr (!FUSED) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        const int row = 16 * mt + lr;
        u32x4 piece[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const unsigned ao = (row < p.M && k_off[t][h] != 0x80000000u) ? (unsigned)row * p.K + k_off[t][h] : 0x80000000u;
          piece[h] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_a, ao, 0, 0));
        }
        af[mt][t] = join(piece[0], piece[1]);
      }
  }

  // Fused quantisation, first half (before the weight stream starts, so that these loads are not queued behind
  // it): row maxima over the whole K.  Every thread takes one 16-byte chunk of each row per round, all rows' loads
  // of a round in flight together; rows past M cost no instruction.
  constexpr int TH = 64 * NW;
  const int tid = threadIdx.x;
  const __amdgpu_buffer_rsrc_t rs_src = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(FUSED ? p.a_src : nullptr), 0, FUSED ? (int)((size_t)p.M * p.K * 2) : 0, 0x00020000);
  const int chunks = p.K / 8;  // per row
  u32x4 v[FUSED ? kFusedRows : 1];
  float mx[FUSED ? kFusedRows : 1];
  if constexpr (FUSED) {
#pragma unroll
    for (int row = 0; row < kFusedRows; ++row) {
      mx[row] = 0.f;
      v[row] = u32x4{0u, 0u, 0u, 0u};
    }
    for (int base = 0; base < chunks; base += TH) {
      const int ch = base + tid;
#pragma unroll
      for (int row = 0; row < kFusedRows; ++row)
        if (row < p.M) {
          const unsigned off = ch < chunks ? ((unsigned)row * p.K + (unsigned)ch * 8u) * 2u : 0x80000000u;
          v[row] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_src, off, 0, 0));
        }
      if (base + TH < chunks) {  // more rounds follow: fold this one in now (the last round's chunks stay in v)
#pragma unroll
        for (int row = 0; row < kFusedRows; ++row) {
          float f[8];
          fp8ops::unpack8<T>(v[row], f);
          mx[row] = fp8ops::absmax8(f, mx[row]);
        }
      }
    }
  }

  u32x4 wq[D][2];
  auto fetch = [&](int slot, int i /* column tile inside the workgroup */, int t) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
      wq[slot][h] = __builtin_bit_cast(
          u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w, w_off[t][h] + i * w_stride, 0, 2));
  };

  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int q = 0; q < D; ++q) {
    fetch(q, q / TPW, q % TPW);
    __builtin_amdgcn_sched_barrier(0);
  }

  if constexpr (AR == 4) {
    // operand lane 16 j + r takes piece j of row r from the lane that loaded it: row r < 4 of half stage hs sits in
    // lane 16 * (hs % 4) + 4 r + j of load hs / 4; rows 4 .. 15 are zero
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      i32x8 v;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int hs = 2 * t + h;
        const int src = (16 * (hs & 3) + 4 * (r & 3) + j) * 4;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int x = __builtin_amdgcn_ds_bpermute(src, (int)araw[hs >> 2][q]);
          v[4 * h + q] = r < 4 ? x : 0;
        }
      }
      af[0][t] = v;
    }
  } else if constexpr (!FUSED) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        u32x4 lo, hi;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          lo[q] = (uint32_t)af[mt][t][q];
          hi[q] = (uint32_t)af[mt][t][4 + q];
        }
        af[mt][t] = to_operand(lo, hi);
      }
  } else {
    // ---- second half: the weight stream is under way.  Fold the last round of chunks in, reduce over the workgroup.
#pragma unroll
    for (int row = 0; row < kFusedRows; ++row) {
      float f[8];
      fp8ops::unpack8<T>(v[row], f);
      mx[row] = fp8ops::absmax8(f, mx[row]);
    }
#pragma unroll
    for (int row = 0; row < kFusedRows; ++row) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) mx[row] = fmaxf(mx[row], __shfl_xor(mx[row], off));
      if (lane == 0) row_part[row * NW + wave] = mx[row];
    }
    __syncthreads();
    if (tid < kFusedRows) {
      float m = row_part[tid * NW];
#pragma unroll
      for (int w = 1; w < NW; ++w) m = fmaxf(m, row_part[tid * NW + w]);
      row_scale[tid] = fmaxf(m / fp8ops::kE4m3Max, fp8ops::kMinScale);
    }
    __syncthreads();
    // ---- quantise the k range of this workgroup into LDS: one chunk per thread and row (at most 64 stages = 1024
    // chunks).  With one split and a row of at most 1024 chunks the registers still hold exactly these chunks.
    const int kw0 = wg_begin * 16, kwn = (wg_end - wg_begin) * 16;  // first chunk and chunk count of the range
    if (!(p.ksplit == 1 && chunks <= TH)) {
#pragma unroll
      for (int row = 0; row < kFusedRows; ++row)
        if (row < p.M) {
          const unsigned off = tid < kwn ? ((unsigned)row * p.K + (unsigned)(kw0 + tid) * 8u) * 2u : 0x80000000u;
          v[row] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_src, off, 0, 0));
        }
    }
#pragma unroll
    for (int row = 0; row < kFusedRows; ++row)
      if (row < p.M) {  // uniform: rows past M cost nothing (the division is the expensive part)
        float f[8];
        fp8ops::unpack8<T>(v[row], f);
        const fp8ops::u32x2 q = fp8ops::quantize8(f, row_scale[row]);
        if (tid < kwn) *reinterpret_cast<fp8ops::u32x2*>(aq_lds + row * kFusedRowBytes + tid * 8) = q;
      }
    __syncthreads();
    // ---- operand fragments straight from LDS: lane (r, j) takes bytes [16j, 16j+16) and [64+16j, ..) of row r
#pragma unroll
    for (int t = 0; t < TPW; ++t) {
      const bool ok = r < p.M && s0 + t < wg_end;
      const uint8_t* src = aq_lds + (r & (kFusedRows - 1)) * kFusedRowBytes + (ok ? (s0 + t - wg_begin) * 128 : 0) + 16 * j;
      u32x4 lo = *reinterpret_cast<const u32x4*>(src), hi = *reinterpret_cast<const u32x4*>(src + 64);
      if (!ok) lo = hi = u32x4{0u, 0u, 0u, 0u};
      af[0][t] = join(lo, hi);
    }
  }

  epi_elem_t<T>* out = static_cast<epi_elem_t<T>*>(p.out);
  for (int b = 0; b < nbatches; ++b) {
    f32x4 accb[NB][MT];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) accb[i][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        const int slot = i * TPW + t;
        const i32x8 bw = to_operand(wq[slot][0], wq[slot][1]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          accb[i][mt] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af[mt][t], bw, accb[i][mt], 0, 0, 0, 0, 0, 0);
        fetch(slot, (b + 1) * NB + i, t);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- sum the k slices of every tile of the batch (fixed order: deterministic).  The reduction buffer is
    // double-buffered, so one barrier per batch is enough: whoever writes buffer b & 1 again (batch b + 2) has passed
    // the barrier of batch b + 1, which the readers of batch b reach only after their reads.
    f32x4* rb = red + (b & 1) * (NB * MT * NW * 64);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) rb[((i * MT + mt) * NW + wave) * 64 + lane] = accb[i][mt];
    __syncthreads();
    if (wave < NB * MT) {  // one (column tile, row tile) per wave
      const int i = wave / MT, mt = wave - i * MT;
      const int nt = nt_begin + b * NB + i;
      const bool valid = b * NB + i < count && 16 * mt < p.M;
      // added in wave order (deterministic), eight reads in flight at a time: the weight ring is live in registers
      // here, so all NW at once do not fit, but every group of reads is one LDS round trip on the way to the store
      // (where the activation fragments and the ring leave the registers for it: otherwise the reads would spill)
      constexpr int kOperandRegs = (MT * TPW + D) * 8;
      constexpr int kRB = ((NW == 16 && kOperandRegs <= 48) || (NW == 8 && kOperandRegs <= 160)) ? 8 : 4;
      f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w0 = 0; w0 < NW; w0 += kRB) {
        f32x4 part[kRB];
#pragma unroll
        for (int ww = 0; ww < kRB; ++ww) part[ww] = rb[(wave * NW + w0 + ww) * 64 + lane];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ww = 0; ww < kRB; ++ww) sum += part[ww];
        __builtin_amdgcn_sched_barrier(0);
      }
      bool store = valid;
      if (p.ksplit > 1 && valid) {
        // split across workgroups: park the fp32 tile, the last split to arrive adds them in split order
        const size_t stride = (size_t)p.ntiles * MT * 64;
        const size_t tile = ((size_t)nt * MT + mt) * 64 + lane;
        store_agent(p.partial + (size_t)split * stride + tile, sum);
        unsigned* counter = p.counters + nt * MT + mt;
        store = splitk_arrive_last(counter, lane, p.ksplit);
        if (store) {
          sum = f32x4{0.f, 0.f, 0.f, 0.f};
          for (int sp = 0; sp < p.ksplit; ++sp) sum += load_agent(p.partial + (size_t)sp * stride + tile);
          if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      if (store) {
        const int col = nt * 16 + r, row0 = 16 * mt + 4 * j;
        const float ws = p.w_scale[p.w_scale_per_col ? (col < p.N ? col : p.N - 1) : 0];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int row = row0 + e;
          float as;
          if constexpr (FUSED) as = row_scale[row < p.M ? row : 0];
          else as = p.a_scale[p.a_scale_per_row ? (row < p.M ? row : p.M - 1) : 0];
          sum[e] = sum[e] * ws * as;
        }
        epi_store_acc<T>(p.epi, out, sum, row0, col, p.M, p.N, col < p.N);
      }
    }
  }
}

// The same decomposition for a K too long for one pass at one to eight rows (more stages than the waves hold as
// activation fragments): the workgroup walks K in phases of 16 x TPW stages instead of sharing it with other workgroups
// through partial tiles in memory.  Every wave keeps one fp32 tile per column tile of the workgroup across the phases,
// swaps in the activation fragments of its next TPW stages (requested a phase ahead, as loaded) and streams the weight
// rows through the same ring; one reduction over the 16 waves at the end.  No workspace, no counters.
// AR as above: 4 (at most four rows, one load instruction per phase) or 16.
template <typename T, int NB, int AR>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4))) void fp8_kphase_kernel(Fp8KstatArgs p) {
  constexpr int NW = 16, TPW = 2, D = NB * TPW, KP = NW * TPW;
  static_assert(AR == 4 || AR == 16, "activation rows per load instruction");
  __shared__ f32x4 red[NB * NW * 64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, j = lane >> 4;
  const int nt_begin = blockIdx.x * NB;
  int count = p.ntiles - nt_begin;
  count = count < NB ? count : NB;
  const int nphases = (p.KS + KP - 1) / KP;
  const int s0 = wave * TPW;  // first stage of this wave in phase 0; phase ph adds ph * KP

  int rows = count * 16;
  if (nt_begin * 16 + rows > p.N) rows = p.N - nt_begin * 16;
  if (rows < 0) rows = 0;
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(p.wq) + (size_t)nt_begin * 16 * p.K, 0, (int)((size_t)rows * p.K), 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(p.aq), 0, (int)((size_t)p.M * p.K), 0x00020000);
  const int lr = lane >> 2, lp = lane & 3;
  const unsigned w_stride = 16u * (unsigned)p.K;
  // this lane's 16 bytes of (stage s0 + ph * KP + t, half h) inside a row, or out of range (stage past K, piece past K)
  auto k_byte = [&](int ph, int t, int h) {
    const int st = s0 + ph * KP + t;
    const unsigned kb = (unsigned)st * 128u + 64u * h + 16u * lp;
    return (st < p.KS && kb + 16u <= (unsigned)p.K) ? kb : 0x80000000u;
  };

  u32x4 wq[D][2];
  auto fetch = [&](int slot, int i, int t, int ph) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const unsigned kb = k_byte(ph, t, h);
      const unsigned off = kb != 0x80000000u ? kb + (unsigned)lr * p.K + i * w_stride : 0x80000000u;
      wq[slot][h] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w, off, 0, 2));
    }
  };
  // the next phase's activations as loaded.  AR = 16: araw[2 t + h], lane l on row l / 4, piece l % 4 of the half
  // stage; AR = 4: araw[0], lane l on row l / 4 % 4 of half stage l / 16
  u32x4 araw[AR == 4 ? 1 : 2 * TPW];
  auto load_a = [&](int ph) {
    if constexpr (AR == 4) {
      const int hs = lane >> 4, row = (lane >> 2) & 3;
      const unsigned kb = k_byte(ph, hs >> 1, hs & 1);
      const bool ok = kb != 0x80000000u && row < p.M;
      araw[0] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_a, ok ? (unsigned)row * p.K + kb : 0x80000000u, 0, 0));
    } else {
#pragma unroll
      for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const unsigned kb = k_byte(ph, t, h);
          const bool ok = kb != 0x80000000u && lr < p.M;
          araw[2 * t + h] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_a, ok ? (unsigned)lr * p.K + kb : 0x80000000u, 0, 0));
        }
    }
  };
  const int from = (4 * r + j) * 4;
  auto to_operand = [&](u32x4 lo, u32x4 hi) {
    i32x8 v;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      v[q] = __builtin_amdgcn_ds_bpermute(from, (int)lo[q]);
      v[4 + q] = __builtin_amdgcn_ds_bpermute(from, (int)hi[q]);
    }
    return v;
  };

  load_a(0);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int q = 0; q < D; ++q) {
    fetch(q, q / TPW, q % TPW, 0);
    __builtin_amdgcn_sched_barrier(0);
  }

  f32x4 acc[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int ph = 0; ph < nphases; ++ph) {
    i32x8 af[TPW];
    if constexpr (AR == 4) {
      // operand lane 16 j + r takes piece j of row r from lane 16 * hs + 4 r + j of the one load; rows 4 .. 15 are zero
#pragma unroll
      for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int src = (16 * (2 * t + h) + 4 * (r & 3) + j) * 4;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int x = __builtin_amdgcn_ds_bpermute(src, (int)araw[0][q]);
            af[t][4 * h + q] = r < 4 ? x : 0;
          }
        }
    } else {
#pragma unroll
      for (int t = 0; t < TPW; ++t) af[t] = to_operand(araw[2 * t], araw[2 * t + 1]);
    }
    __builtin_amdgcn_sched_barrier(0);
    load_a(ph + 1);  // a phase past the end is parked: nothing is read
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        const int slot = i * TPW + t;
        const i32x8 bw = to_operand(wq[slot][0], wq[slot][1]);
        acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af[t], bw, acc[i], 0, 0, 0, 0, 0, 0);
        fetch(slot, i, t, ph + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
  }

  // ---- the 16 k slices of every column tile, summed in wave order by wave i of tile i
#pragma unroll
  for (int i = 0; i < NB; ++i) red[(i * NW + wave) * 64 + lane] = acc[i];
  __syncthreads();
  if (wave < NB) {
    f32x4 part[NW];
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) part[ww] = red[(wave * NW + ww) * 64 + lane];
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) sum += part[ww];
    const int col = (nt_begin + wave) * 16 + r, row0 = 4 * j;
    const float ws = p.w_scale[p.w_scale_per_col ? (col < p.N ? col : p.N - 1) : 0];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int row = row0 + e;
      const float as = p.a_scale[p.a_scale_per_row ? (row < p.M ? row : p.M - 1) : 0];
      sum[e] = sum[e] * ws * as;
    }
    // every lane makes the call (the epilogue may exchange lanes); a column tile past the range stores nothing
    epi_store_acc<T>(p.epi, static_cast<epi_elem_t<T>*>(p.out), sum, row0, col, p.M, p.N, wave < count && col < p.N);
  }
}

template <typename T>
bool launch_kphase(int nb, int m, const Fp8KstatArgs& a, dim3 grid, hipStream_t s) {
#define KSQ_PH(NB)                                                                                    \
  do {                                                                                                \
    if (m <= 4) hipLaunchKernelGGL((fp8_kphase_kernel<T, NB, 4>), grid, dim3(1024), 0, s, a);         \
    else hipLaunchKernelGGL((fp8_kphase_kernel<T, NB, 16>), grid, dim3(1024), 0, s, a);               \
  } while (0)
  if (nb == 1) KSQ_PH(1);
  else if (nb == 2) KSQ_PH(2);
  else if (nb == 3) KSQ_PH(3);
  else if (nb == 4) KSQ_PH(4);
  else return false;
#undef KSQ_PH
  return true;
}

// one row tile and at most four rows: the narrow activation loads
#define KSQ_GO(MT, TPW, NB, NW)                                                                                   \
  do {                                                                                                            \
    if (MT == 1 && a.M <= 4)                                                                                      \
      hipLaunchKernelGGL((fp8_kstat_kernel<T, 1, TPW, NB, NW, false, 4>), grid, dim3(64 * NW), 0, s, a);          \
    else                                                                                                          \
      hipLaunchKernelGGL((fp8_kstat_kernel<T, MT, TPW, NB, NW, false>), grid, dim3(64 * NW), 0, s, a);            \
  } while (0)
#define KSQ_GO_FUSED(TPW, NB) hipLaunchKernelGGL((fp8_kstat_kernel<T, 1, TPW, NB, 16, true>), grid, dim3(1024), 0, s, a)
template <typename T>
bool launch_fused(int tpw, int nb, const Fp8KstatArgs& a, dim3 grid, hipStream_t s) {
  if (tpw == 4 && nb == 1) KSQ_GO_FUSED(4, 1);
  else if (tpw == 4 && nb == 2) KSQ_GO_FUSED(4, 2);
  else if (tpw == 2 && nb == 1) KSQ_GO_FUSED(2, 1);
  else if (tpw == 2 && nb == 2) KSQ_GO_FUSED(2, 2);
  else if (tpw == 1 && nb == 1) KSQ_GO_FUSED(1, 1);
  else if (tpw == 1 && nb == 2) KSQ_GO_FUSED(1, 2);
  else return false;
  return true;
}
#undef KSQ_GO_FUSED

template <typename T>
void launch(int mt, int tpw, int nb, const Fp8KstatArgs& a, dim3 grid, hipStream_t s) {
  if (mt == 1 && tpw == 8) {
    if (nb == 1) KSQ_GO(1, 8, 1, 8);
    else KSQ_GO(1, 8, 2, 8);
  } else if (mt == 1) {
    if (tpw == 4) {
      if (nb == 1) KSQ_GO(1, 4, 1, 16);
      else KSQ_GO(1, 4, 2, 16);
    } else if (tpw == 2) {
      if (nb == 1) KSQ_GO(1, 2, 1, 16);
      else if (nb == 2) KSQ_GO(1, 2, 2, 16);
      else KSQ_GO(1, 2, 4, 16);
    } else {
      if (nb == 1) KSQ_GO(1, 1, 1, 16);
      else if (nb == 2) KSQ_GO(1, 1, 2, 16);
      else KSQ_GO(1, 1, 4, 16);
    }
  } else if (mt == 2) {
    if (tpw == 2) {
      if (nb == 1) KSQ_GO(2, 2, 1, 16);
      else KSQ_GO(2, 2, 2, 16);
    } else {
      if (nb == 1) KSQ_GO(2, 1, 1, 16);
      else KSQ_GO(2, 1, 2, 16);
    }
  } else {
    if (tpw == 4) {
      if (nb == 1) KSQ_GO(4, 4, 1, 8);
      else KSQ_GO(4, 4, 2, 8);
    } else if (tpw == 2) {
      if (nb == 1) KSQ_GO(4, 2, 1, 8);
      else KSQ_GO(4, 2, 2, 8);
    } else {
      KSQ_GO(4, 1, 2, 8);
    }
  }
}
#undef KSQ_GO

}  // namespace

// Plan: row tiles (1, 2 or 4), waves per workgroup (8 with four row tiles or one row tile and a long K, else 16),
// stages per wave (1, 2, 4 or 8; at most 2 with two row tiles: the activations of waves x TPW stages live in
// registers), split count, column tiles per workgroup and per batch.
Fp8KstatPlan fp8_kstat_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes, bool fused) {
  Fp8KstatPlan p{};
  const size_t ntiles = (n + 15) / 16, stages = (k + 127) / 128;
  p.ok = m >= 1 && m <= 64 && ntiles * 4 <= (size_t)kCountersPerSlot && m * k < 0x7FFFFF00ull;
  if (!p.ok) return p;
  p.mt = m <= 16 ? 1 : (m <= 32 ? 2 : 4);
  // One row tile and a K that has to be split over workgroups anyway (more than 64 stages): 8 waves with 8 stages
  // each and a ring of two column tiles instead of 16 waves with 4 stages and a ring of one -- twice the bytes in
  // flight per CU (measured at K = 29568: 15 % faster; no gain for K <= 8192).
  bool wide = p.mt == 1 && stages > 64;
  if (const char* e = tuning_env("KSQ_FP8_WIDE")) wide = atoi(e) != 0 && p.mt == 1;  // tuning / test override
  if (fused) wide = false;  // the kernel that quantises its own activations: 16 waves, LDS for two column tiles a batch
  const size_t nw = (p.mt == 4 || wide) ? 8 : 16;
  const size_t cap = nw * (wide ? 8u : (p.mt == 2 ? 2u : 4u));
  size_t ksplit = (stages + cap - 1) / cap;
  auto need = [&](size_t ks) { return ks <= 1 ? (size_t)0 : ks * ntiles * p.mt * 64 * 16; };
  // Five to sixteen rows and between one and two column tiles per CU: K split in two (four tiles per workgroup in
  // batches of two, half the stages each) where the workspace allows, instead of two tiles one after the other
  // (measured at K = N = 8192: 20.5 -> 18.4 us at M = 8, 21.0 -> 18.7 at M = 16; at four rows and fewer the
  // one-tile workgroups below are faster still, and with 2.5 tiles per CU, N = 10240, the split loses 10 %)
  if (p.mt == 1 && m > 4 && ksplit == 1 && !fused && stages >= 64 && ntiles > (size_t)cus && ntiles <= 2 * (size_t)cus &&
      need(2) <= workspace_bytes)
    ksplit = 2;
  if (const char* e = tuning_env("KSQ_FP8_KSPLIT")) {  // tuning / test override; never below what the registers need
    const size_t v = (size_t)atoi(e);
    if (v > ksplit && v <= stages) ksplit = v;
  }
  // One to eight rows and a K that one pass does not cover: phases inside the workgroup instead of a split across
  // workgroups, where the column tiles alone give every CU one to four of them (see fp8_kphase_kernel)
  bool phases = p.mt == 1 && m <= 8 && !fused && ksplit >= 2 && ntiles * 4 >= 3 * (size_t)cus && ntiles <= 4 * (size_t)cus;
  if (const char* e = tuning_env("KSQ_FP8_KPHASE")) {  // tuning / test switch: 0 = never, 1 = whenever the kernel can
    phases = atoi(e) != 0 && p.mt == 1 && m <= 8 && !fused && ntiles <= 4 * (size_t)cus && stages >= 2;
  }
  if (phases) {
    p.phases = true;
    p.ksplit = 1;
    p.tpw = 2;
    p.nb = (int)((ntiles + (size_t)cus - 1) / (size_t)cus);
    p.nt_per_wg = p.nb;
    p.grid_x = (int)((ntiles + p.nb - 1) / p.nb);
    p.partial_bytes = 0;
    return p;
  }
  if (need(ksplit) > workspace_bytes) {
    p.ok = false;
    return p;
  }
  const size_t per_split = (stages + ksplit - 1) / ksplit;
  const size_t tpw = (per_split + nw - 1) / nw;
  p.tpw = wide ? 8 : (tpw <= 1 ? 1 : (tpw <= 2 ? 2 : 4));
  p.ksplit = (int)ksplit;
  size_t wgs = (size_t)cus / ksplit;
  if (wgs < 1) wgs = 1;
  if (wgs > ntiles) wgs = ntiles;
  p.nt_per_wg = (int)((ntiles + wgs - 1) / wgs);
  // At most four rows (their activation loads are a handful of instructions) and between one and two column tiles
  // per CU: one tile per workgroup, two workgroups side by side on a CU, instead of two tiles one after the other
  // (measured at K = 8192, one token: N = 8192 20.2 -> 17.4 us, N = 6144 16.5 -> 15.7; with 16 rows it loses)
  if (m <= 4 && ksplit == 1 && p.mt == 1 && !wide && !fused && ntiles > (size_t)cus && ntiles <= 2 * (size_t)cus)
    p.nt_per_wg = 1;
  if (const char* e = tuning_env("KSQ_FP8_NT_PER_WG")) {  // tuning / test override
    const int v = atoi(e);
    if (v >= 1 && (size_t)v <= ntiles) p.nt_per_wg = v;
  }
  p.grid_x = (int)((ntiles + p.nt_per_wg - 1) / p.nt_per_wg);
  // a single row tile reduces after every column tile when the ring is deep enough without batching (measured:
  // finer batches overlap the reduction of one tile with the stream of the next); more row tiles batch by two
  // (four row tiles: one column tile a batch; measured at M = 64, K = 8192: N = 10240 34.6 -> 29.6 us, N = 8192
  // 28.7 -> 25.0; with two row tiles batches of two are 10 % ahead)
  p.nb = p.mt == 4 ? 1 : (p.mt == 2 ? 2 : (p.tpw == 4 ? 1 : (p.tpw == 2 ? 2 : 4)));
  if (wide) p.nb = 2;
  if (p.nb > p.nt_per_wg) p.nb = p.nt_per_wg >= 2 ? 2 : 1;
  if (const char* e = tuning_env("KSQ_FP8_NB")) {  // tuning override
    const int v = atoi(e);
    if (v == 1 || v == 2 || (v == 4 && p.mt == 1 && p.tpw < 4)) p.nb = v;
    if (wide && p.nb > 2) p.nb = 2;
  }
  if (fused && p.nb > 2) p.nb = 2;
  p.partial_bytes = need(ksplit);
  return p;
}

int fp8_launch_kstat(int out_dtype, const Fp8KstatPlan& plan, void* out, const void* act_q, const float* act_scale,
                     size_t act_scale_count, const void* w_q, const float* w_scale, size_t w_scale_count, size_t m,
                     size_t n, size_t k, void* workspace, hipStream_t s, const Epilogue& epi, const void* act_src) {
  KSQ_REQUIRE(((size_t)plan.nt_per_wg + 8) * 16 * k < 0x3FFFFF00ull, KSQ_ERR_UNSUPPORTED,
              "column range of one workgroup larger than 1 GiB");
  KSQ_REQUIRE(act_src == nullptr || (m <= (size_t)kFusedRows && k % 128 == 0 && plan.mt == 1 && plan.nb <= 2 &&
                                     plan.tpw <= 4 && m * k * 2 < 0x7FFFFF00ull),
              KSQ_ERR_UNSUPPORTED, "fused activation quantisation: at most %d rows, k a multiple of 128", kFusedRows);
  Fp8KstatArgs a{};
  a.epi = epi;
  a.a_src = static_cast<const uint16_t*>(act_src);
  a.aq = static_cast<const uint8_t*>(act_q);
  a.wq = static_cast<const uint8_t*>(w_q);
  a.a_scale = act_scale;
  a.w_scale = w_scale;
  a.out = out;
  a.partial = static_cast<f32x4*>(workspace);
  a.M = (int)m;
  a.N = (int)n;
  a.K = (int)k;
  a.KS = (int)((k + 127) / 128);
  a.ntiles = (int)((n + 15) / 16);
  a.ksplit = plan.ksplit;
  a.nt_per_wg = plan.nt_per_wg;
  a.a_scale_per_row = act_scale_count > 1;
  a.w_scale_per_col = w_scale_count > 1;
  a.counters = nullptr;
  if (plan.ksplit > 1) {
    KSQ_REQUIRE(workspace != nullptr, KSQ_ERR_WORKSPACE, "split-K planned without a workspace");
    a.counters = counter_slot_device_ptr(s);
    KSQ_REQUIRE(a.counters != nullptr, KSQ_ERR_HIP, "split-K planned for a stream without arrival counters");
  }
  dim3 grid((unsigned)plan.grid_x, (unsigned)plan.ksplit, 1);
  if (plan.phases) {
    KSQ_REQUIRE(act_src == nullptr, KSQ_ERR_UNSUPPORTED, "no fused quantisation in the phase kernel");
    note_launch("fp8_kphase_kernel<nb=%d,ar=%d> grid=(%d)", plan.nb, m <= 4 ? 4 : 16, plan.grid_x);
    const bool ok = out_dtype == KSQ_F16   ? launch_kphase<_Float16>(plan.nb, (int)m, a, grid, s)
                    : out_dtype == KSQ_F32 ? launch_kphase<float>(plan.nb, (int)m, a, grid, s)
                                           : launch_kphase<__bf16>(plan.nb, (int)m, a, grid, s);
    KSQ_REQUIRE(ok, KSQ_ERR_UNSUPPORTED, "no phase kernel for %d column tiles per workgroup", plan.nb);
    KSQ_HIP_TRY(hipGetLastError());
    return KSQ_OK;
  }
  note_launch("fp8_kstat_kernel<mt=%d,tpw=%d,nb=%d%s> grid=(%d,%d) nt_per_wg=%d", plan.mt, plan.tpw, plan.nb,
              act_src ? ",fused" : "", plan.grid_x, plan.ksplit, plan.nt_per_wg);
  if (act_src != nullptr) {
    KSQ_REQUIRE(out_dtype != KSQ_F32, KSQ_ERR_UNSUPPORTED, "the kernel that quantises its own activations reads 16-bit ones");
    const bool ok = out_dtype == KSQ_F16 ? launch_fused<_Float16>(plan.tpw, plan.nb, a, grid, s)
                                         : launch_fused<__bf16>(plan.tpw, plan.nb, a, grid, s);
    KSQ_REQUIRE(ok, KSQ_ERR_UNSUPPORTED, "no fused kernel for %d stages per wave, %d column tiles per batch", plan.tpw,
                plan.nb);
  } else if (out_dtype == KSQ_F16) {
    launch<_Float16>(plan.mt, plan.tpw, plan.nb, a, grid, s);
  } else if (out_dtype == KSQ_F32) {
    launch<float>(plan.mt, plan.tpw, plan.nb, a, grid, s);
  } else {
    launch<__bf16>(plan.mt, plan.tpw, plan.nb, a, grid, s);
  }
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

}  // namespace ksq
