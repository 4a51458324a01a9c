// W4A16 decode kernel for M <= 64: k-stationary.
//
// A workgroup is 16 waves (one 16-row tile of activations) or 8 waves with twice the registers each (two or four row
// tiles).  Wave w keeps the activation fragments of its own TPW k tiles, for all MT row tiles, in registers for the
// whole kernel (the activations of a decode step are small) and streams the weight tiles (n tile, its k tiles) of
// the workgroup's column range straight from HBM into a register ring, one batch of NB column tiles ahead.  Nothing
// is re-read: no activation traffic per weight tile, no LDS on the streaming path.  After every batch the partial
// tiles of a (column tile, row tile) -- one per wave = per k slice -- are summed through LDS in a fixed order, one
// tile per wave.  Because k is covered inside the workgroup, narrow N needs no split across workgroups; only K
// beyond waves x TPW tiles is split over grid.y and finished by the last-arriving workgroup through the workspace.
//
// Arithmetic as in the streaming kernel: biased nibbles by bit operations, a correction MFMA with -(bias + z),
// fp32 group sums scaled by s[g,n].
#include <cstdlib>

#include "ksq_internal.h"
#include "ksq_epilogue.h"
#include "ksq_w4a16_ops.h"

namespace ksq {
namespace {

using namespace w4;

struct KstatArgs {
  const void* weight;  // [ntiles][KT][64] x 16 B
  const void* sz;      // [ntiles][G][16] x 4 B
  const void* act;     // [M][K] T
  void* out;           // [M][N] T
  f32x4* partial;      // [ksplit][ntiles][MT][64]
  unsigned* counters;  // [ntiles][MT]
  int M, N, K, KT, G, ntiles, ksplit, nt_per_wg, act_barrier;
  Epilogue epi;
};

// PPI = 16-byte pieces of one activation row that one load instruction brings in (4, 8 or 16): a load covers 64 / PPI
// rows, so with few rows (M <= 8, M <= 4) a k tile takes two or one instruction instead of four.  The memory pipeline
// of a compute unit holds a limited number of instructions in flight, whatever their size or lane mask, and at the
// start of this kernel that window is what every wave waits for.
template <typename T, int GPT, int MT, int TPW, int NB, int NW, int PPI>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(NW / 4))) void w4a16_kstat_kernel(KstatArgs p) {
  static_assert(PPI == 4 || ((PPI == 8 || PPI == 16) && MT == 1), "wide activation loads: one row tile only");
  constexpr int API = 16 / PPI;  // activation load instructions per k tile
  using O = Ops<T>;
  constexpr int DPG = 4 / GPT;
  constexpr int D = NB * TPW;  // ring depth = one batch
  constexpr bool kRowSums = MT == 1 && TPW * GPT <= 2 && D <= 4;  // see the prologue (where the registers allow)
  static_assert(NB * MT * NW <= 64 && NB * MT <= NW && NW % (NB * MT) == 0, "reduction: two buffers of <= 64 KiB");
  __shared__ f32x4 red[2 * NB * MT * NW * 64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, j = lane >> 4;
  const int split = blockIdx.y;
  int wg_begin, wg_end;
  split_range(p.KT, split, p.ksplit, &wg_begin, &wg_end);
  const int kt0 = wg_begin + wave * TPW;  // first k tile of this wave
  const int nt_begin = blockIdx.x * p.nt_per_wg;
  int count = p.ntiles - nt_begin;
  count = count < p.nt_per_wg ? count : p.nt_per_wg;
  const int nbatches = (p.nt_per_wg + NB - 1) / NB;  // same for every workgroup

  // Resources start at (nt_begin, kt0) and end with the wave's live k tiles of the last column tile of the workgroup,
  // so column tiles past the range read as zero: the prefetch of column tile `count` lands KT tiles further on, and
  // KT >= live.  (With TPW in place of `live` a wave with fewer live k tiles than TPW -- K = 128 under an
  // instantiation with two k tiles per wave -- had tile `count` in range, and the last workgroup read 1 KiB past the
  // end of the weights and 64 GPT bytes past the scale/zero words.)  k tiles past the end of the split are parked at
  // an offset that stays out of range for every column tile (the range is far below 2^31 bytes).
  const size_t kt0c = kt0 < p.KT ? (size_t)kt0 : (size_t)p.KT - 1;
  const char* wb = static_cast<const char*>(p.weight) + ((size_t)nt_begin * p.KT + kt0c) * 1024;
  const char* sb = static_cast<const char*>(p.sz) + ((size_t)nt_begin * p.G + kt0c * GPT) * 64;
  const bool any = count > 0 && kt0 < wg_end;
  const int live = wg_end - kt0 < TPW ? wg_end - kt0 : TPW;
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(wb), 0, any ? ((count - 1) * p.KT + live) * 1024 : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_sz = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(sb), 0, any ? ((count - 1) * p.G + live * GPT) * 64 : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.act), 0, (int)((size_t)p.M * p.K * 2), 0x00020000);
  unsigned w_off[TPW];
#pragma unroll
  for (int t = 0; t < TPW; ++t) w_off[t] = kt0 + t < wg_end ? t * 1024u + lane * 16u : 0x80000000u;
  const unsigned w_stride = (unsigned)p.KT * 1024u, sz_stride = (unsigned)p.G * 64u;
  // The scale/zero words of one batch -- NB column tiles x the wave's TPW * GPT groups x 16 columns -- are fetched
  // with one word per lane: the words of one column tile are contiguous (its groups follow each other), so SZR
  // instructions cover the batch instead of one instruction per (column tile, group).  Flat word f = 64 r + lane
  // belongs to column tile f / (16 GW), group (f / 16) % GW, column f % 16.  The memory pipeline takes about as long
  // for a one-word-per-lane instruction as for a weight tile, so this matters.
  constexpr int GW = TPW * GPT;                  // groups per column tile that this wave needs
  constexpr int SZR = (NB * GW * 16 + 63) / 64;  // instructions per batch
  unsigned sz_off[SZR];
#pragma unroll
  for (int r = 0; r < SZR; ++r) {
    const int f = 64 * r + lane, i = f / (16 * GW), gq = (f >> 4) % GW;
    const bool ok = i < NB && kt0 + gq / GPT < wg_end;
    sz_off[r] = ok ? (unsigned)i * sz_stride + (unsigned)gq * 64u + (unsigned)c * 4u : 0x80000000u;
  }

  // Activation fragments of this wave's k tiles: registers for the whole kernel.  Load instruction i of a k tile has
  // lane l on row l / PPI, 16-byte piece i * PPI + l % PPI of the tile's 16, so that every aligned group of four lanes
  // reads 64 contiguous bytes (the memory pipeline then takes four lanes per clock instead of one); the MFMA operand
  // layout (lane 16 j + c = row c, piece 4 d + j for the 32-k step d) comes from a lane permutation further down.
  u32x4 af[MT][TPW][4];
  {
    const int lr = lane / PPI, lp = lane % PPI;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int i = 0; i < API; ++i) {
          const int row = 16 * mt + lr;
          const bool ok = row < p.M && kt0 + t < wg_end;
          const unsigned ao = ok ? ((unsigned)row * p.K + (kt0 + t) * kTileK + 8 * (i * PPI + lp)) * 2u : 0x80000000u;
          af[mt][t][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_a, ao, 0, 0));
        }
  }

  u32x4 wq[D];
  uint32_t szraw[SZR];  // the next batch's words as loaded, one per lane
  auto fetch = [&](int slot, int i /* column tile inside the workgroup */, int t) {
    wq[slot] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w, w_off[t] + i * w_stride, 0, 2));
  };
  auto fetch_sz = [&](int batch) {
#pragma unroll
    for (int r = 0; r < SZR; ++r)
      szraw[r] = __builtin_amdgcn_raw_buffer_load_b32(rs_sz, sz_off[r] + (unsigned)(batch * NB) * sz_stride, 0, 0);
  };

  uint32_t m_lo = O::kMaskLo, m_hi = O::kMaskHi, c_lo = O::kMagicLo, c_hi = O::kMagicHi;
  KSQ_PIN_SGPR(m_lo);
  KSQ_PIN_VGPR(c_lo);
  KSQ_PIN_VGPR(c_hi);
  KSQ_PIN_VGPR(m_hi);

  __builtin_amdgcn_sched_barrier(0);
  // With more than one batch per workgroup, every wave's activation loads are issued before any wave's weight
  // loads: the memory pipeline of a compute unit returns data in the order of issue, so activations (cache hits)
  // queued behind another wave's weight tiles (HBM) would hold their wave back by the whole first batch.
  if (p.act_barrier) __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  fetch_sz(0);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int q = 0; q < D; ++q) {
    fetch(q, q / TPW, q % TPW);
    __builtin_amdgcn_sched_barrier(0);
  }

  {  // lane 16 j + c takes piece 4 d + j of row c: loaded by instruction (4 d + j) / PPI, lane c * PPI + (4 d + j) % PPI
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        u32x4 got[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int piece = 4 * d + j;
          const int from = (c * PPI + piece % PPI) * 4;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            uint32_t v = 0;
            if constexpr (PPI == 4) {
              v = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)af[mt][t][d][q]);
            } else if constexpr (PPI == 8) {  // instruction 0 for d < 2, instruction 1 for d >= 2
              v = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)af[mt][t][d >> 1][q]);
              v = c < 8 ? v : 0u;  // rows 8..15 were not loaded
            } else {
              v = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)af[mt][t][0][q]);
              v = c < 4 ? v : 0u;
            }
            got[d][q] = v;
          }
        }
#pragma unroll
        for (int d = 0; d < 4; ++d) af[mt][t][d] = got[d];
      }
  }

  // Bias and zero point: the nibbles enter the matrix instruction as bias + u, so every (column, group) owes
  // -sum_k a_k (bias_k + z).  With one row tile and few k tiles per wave the two sums over the wave's activations,
  // sum_k a_k and -sum_k a_k bias_k (the bias alternates between 1024 and 64 inside a word for fp16), are computed
  // once here, by the matrix cores against constant operands, and every (column tile, group) starts its
  // accumulator from -z sum_k a_k - sum_k a_k bias_k: half the matrix instructions of the loop.  Elsewhere the
  // registers for the sums are not there, and the correction stays a second matrix instruction per 32-k step.
  f32x4 asum[kRowSums ? TPW : 1][GPT], abias[kRowSums ? TPW : 1][GPT];
  if constexpr (kRowSums) {
    const uint32_t ones = O::kOnes;
    const u32x4 one4 = {ones, ones, ones, ones}, nbias = O::correction(0u);
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi) {
        asum[t][gi] = f32x4{0.f, 0.f, 0.f, 0.f};
        abias[t][gi] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dd = 0; dd < DPG; ++dd) {
          asum[t][gi] = O::mfma(af[0][t][gi * DPG + dd], one4, asum[t][gi]);
          abias[t][gi] = O::mfma(af[0][t][gi * DPG + dd], nbias, abias[t][gi]);
        }
      }
  }

  uint16_t* out = static_cast<uint16_t*>(p.out);
  const int sz_lane = c * 4;
  for (int b = 0; b < nbatches; ++b) {
    // every lane takes the words of its column: word (i, gq) sits in lane 16 * (f / 16 % 4) + c of instruction f / 64
    uint32_t szq[D][GPT];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int gi = 0; gi < GPT; ++gi) {
          const int f16 = (i * TPW + t) * GPT + gi;  // flat word index / 16
          szq[i * TPW + t][gi] =
              (uint32_t)__builtin_amdgcn_ds_bpermute(sz_lane + 64 * (f16 & 3), (int)szraw[f16 >> 2]);
        }
    __builtin_amdgcn_sched_barrier(0);
    fetch_sz(b + 1);
    __builtin_amdgcn_sched_barrier(0);
    f32x4 accb[NB][MT];
#pragma unroll
    for (int i = 0; i < NB; ++i) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) accb[i][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        const int slot = i * TPW + t;
#pragma unroll
        for (int gi = 0; gi < GPT; ++gi) {
          const uint32_t szw = szq[slot][gi];
          const uint32_t z = (szw >> 16) & 15u;
          const float s = O::scale_to_float(szw);
          f32x4 P[MT];
          if constexpr (kRowSums) {
            // sum_k a (bias_k + u) starts from -sum_k a bias_k - z sum_k a, both sums known since the prologue
            const float zf = (float)z;
#pragma unroll
            for (int e = 0; e < 4; ++e) P[0][e] = __builtin_fmaf(-zf, asum[t][gi][e], abias[t][gi][e]);
#pragma unroll
            for (int dd = 0; dd < DPG; ++dd) {
              const int d = gi * DPG + dd;
              const u32x4 bw = O::unpack(wq[slot][d], m_lo, m_hi, c_lo, c_hi);
              P[0] = O::mfma(af[0][t][d], bw, P[0]);
            }
          } else {
            const u32x4 corr = O::correction(z | (z << 16));
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) P[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int dd = 0; dd < DPG; ++dd) {
              const int d = gi * DPG + dd;
              const u32x4 bw = O::unpack(wq[slot][d], m_lo, m_hi, c_lo, c_hi);
#pragma unroll
              for (int mt = 0; mt < MT; ++mt) {
                P[mt] = O::mfma(af[mt][t][d], corr, P[mt]);
                P[mt] = O::mfma(af[mt][t][d], bw, P[mt]);
              }
            }
          }
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int e = 0; e < 4; ++e) accb[i][mt][e] += s * P[mt][e];
        }
        fetch(slot, (b + 1) * NB + i, t);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // ---- sum the k slices of every tile of the batch (fixed order: deterministic).  Two reduction buffers used in
    // turn and one barrier per batch: whoever writes a buffer again (two batches later) has passed the barrier of
    // the batch in between, which the readers of this batch reach only after their reads.  One (column tile, row
    // tile) per wave, and the reading waves rotate, so the trips to memory of one batch's epilogue overlap with the
    // next batches.
    f32x4* rb = red + (b & 1) * (NB * MT * NW * 64);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) rb[((i * MT + mt) * NW + wave) * 64 + lane] = accb[i][mt];
    __syncthreads();
    const int first = (b * NB * MT) & (NW - 1);  // NB * MT divides NW
    if (wave >= first && wave < first + NB * MT) {
      const int q = wave - first, i = q / MT, mt = q - i * MT;
      const int nt = nt_begin + b * NB + i;
      const bool valid = b * NB + i < count && 16 * mt < p.M;
      // The slices are added in wave order (deterministic), kRB reads in flight at a time: the weight ring is live in
      // registers here, so all NW at once do not fit, but every group of reads is one LDS round trip on the path to
      // the store, and for the last batch nothing else hides it.
      constexpr int kRB = (MT == 1 && TPW <= 2 && D <= 4 && NW >= 8) ? 8 : 4;
      f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w0 = 0; w0 < NW; w0 += kRB) {
        f32x4 part[kRB];
#pragma unroll
        for (int ww = 0; ww < kRB; ++ww) part[ww] = rb[(q * NW + w0 + ww) * 64 + lane];
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
      if (store) epi_store_acc<T>(p.epi, out, sum, 16 * mt + 4 * j, nt * 16 + c, p.M, p.N, true);
    }
  }
}

// The same k-stationary decomposition for a K too long for one pass (more k tiles than 16 waves hold as activation
// fragments) at one to eight rows: instead of splitting K over workgroups -- partial tiles through memory, arrival
// counters, and a workgroup that covers a fraction of K for many column tiles -- the workgroup walks K in phases of
// 16 x TPW k tiles.  Every wave keeps its own fp32 partial tile of each of the workgroup's NB column tiles across
// the phases; per phase it swaps in the activation fragments of its next TPW k tiles (requested a phase ahead in
// the compact form they are loaded in: few rows, so few registers) and streams the NB x TPW weight tiles through the
// same register ring.  Nothing is shared between waves until the one reduction through LDS at the end: no barrier
// and no hand-over in the loop.  With few rows the activations are a small part of what a compute unit loads
// (one or two instructions per k tile against NB of weights); with sixteen rows they would be four per k tile, which
// is why this form stops at eight.
template <typename T, int GPT, int TPW, int NB, int PPI>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4))) void w4a16_kphase_kernel(KstatArgs p) {
  static_assert(PPI == 8 || PPI == 16, "up to eight rows");
  constexpr int NW = 16, API = 16 / PPI, DPG = 4 / GPT, D = NB * TPW, KP = NW * TPW;
  constexpr int GW = TPW * GPT, SZR = (NB * GW * 16 + 63) / 64;
  using O = Ops<T>;
  __shared__ f32x4 red[NB * NW * 64];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, j = lane >> 4;
  const int nt_begin = blockIdx.x * NB;
  int count = p.ntiles - nt_begin;
  count = count < NB ? count : NB;
  const int nphases = (p.KT + KP - 1) / KP;
  const int kt0 = wave * TPW;  // first k tile of this wave in phase 0; phase ph adds ph * KP

  // Resources start at (nt_begin, kt0) and end with the last k tile of the workgroup's last column tile: a column tile
  // past `count` starts KT tiles further on and is out of range whatever the phase.  k tiles past K (the last phase
  // of the last waves) are parked out of range explicitly.
  const size_t kt0c = kt0 < p.KT ? (size_t)kt0 : (size_t)p.KT - 1;
  const bool any = count > 0 && kt0 < p.KT;
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(p.weight) + ((size_t)nt_begin * p.KT + kt0c) * 1024), 0,
      any ? ((count - 1) * p.KT + (p.KT - kt0)) * 1024 : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_sz = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(p.sz) + ((size_t)nt_begin * p.G + kt0c * GPT) * 64), 0,
      any ? ((count - 1) * p.G + (p.KT - kt0) * GPT) * 64 : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.act), 0, (int)((size_t)p.M * p.K * 2), 0x00020000);
  const unsigned w_stride = (unsigned)p.KT * 1024u, sz_stride = (unsigned)p.G * 64u;

  u32x4 araw[TPW][API];  // the next phase's activations as loaded: lane l = row l / PPI, piece i * PPI + l % PPI
  auto load_a = [&](int ph) {
    const int lr = lane / PPI, lp = lane % PPI;
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int i = 0; i < API; ++i) {
        const int kt = kt0 + ph * KP + t;
        const bool ok = lr < p.M && kt < p.KT;
        const unsigned ao = ok ? ((unsigned)lr * p.K + kt * kTileK + 8 * (i * PPI + lp)) * 2u : 0x80000000u;
        araw[t][i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_a, ao, 0, 0));
      }
  };
  u32x4 wq[D];
  uint32_t szraw[SZR];
  auto fetch = [&](int slot, int i, int t, int ph) {
    const bool ok = kt0 + ph * KP + t < p.KT;
    const unsigned off = ok ? (unsigned)(ph * KP + t) * 1024u + lane * 16u + i * w_stride : 0x80000000u;
    wq[slot] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w, off, 0, 2));
  };
  auto fetch_sz = [&](int ph) {
#pragma unroll
    for (int r = 0; r < SZR; ++r) {
      const int f = 64 * r + lane, i = f / (16 * GW), gq = (f >> 4) % GW;
      const bool ok = i < NB && kt0 + ph * KP + gq / GPT < p.KT;
      const unsigned off = ok ? (unsigned)i * sz_stride + (unsigned)(ph * KP * GPT + gq) * 64u + (unsigned)c * 4u : 0x80000000u;
      szraw[r] = __builtin_amdgcn_raw_buffer_load_b32(rs_sz, off, 0, 0);
    }
  };

  uint32_t m_lo = O::kMaskLo, m_hi = O::kMaskHi, c_lo = O::kMagicLo, c_hi = O::kMagicHi;
  KSQ_PIN_SGPR(m_lo);
  KSQ_PIN_VGPR(c_lo);
  KSQ_PIN_VGPR(c_hi);
  KSQ_PIN_VGPR(m_hi);

  load_a(0);
  __builtin_amdgcn_sched_barrier(0);
  fetch_sz(0);
#pragma unroll
  for (int q = 0; q < D; ++q) {
    fetch(q, q / TPW, q % TPW, 0);
    __builtin_amdgcn_sched_barrier(0);
  }

  f32x4 acc[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int sz_lane = c * 4;
  for (int ph = 0; ph < nphases; ++ph) {
    // this phase's activation fragments: lane 16 j + c takes piece 4 d + j of row c, loaded by instruction
    // (4 d + j) / PPI, lane c * PPI + (4 d + j) % PPI; rows that were not loaded are zero
    u32x4 af[TPW][4];
#pragma unroll
    for (int t = 0; t < TPW; ++t)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const int piece = 4 * d + j;
        const int from = (c * PPI + piece % PPI) * 4;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          uint32_t v;
          if constexpr (PPI == 8) v = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)araw[t][d >> 1][q]);
          else v = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)araw[t][0][q]);
          af[t][d][q] = c < 64 / PPI ? v : 0u;
        }
      }
    uint32_t szq[D][GPT];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int t = 0; t < TPW; ++t)
#pragma unroll
        for (int gi = 0; gi < GPT; ++gi) {
          const int f16 = (i * TPW + t) * GPT + gi;
          szq[i * TPW + t][gi] = (uint32_t)__builtin_amdgcn_ds_bpermute(sz_lane + 64 * (f16 & 3), (int)szraw[f16 >> 2]);
        }
    __builtin_amdgcn_sched_barrier(0);
    load_a(ph + 1);  // a phase past the end is parked: nothing is read
    fetch_sz(ph + 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int t = 0; t < TPW; ++t) {
        const int slot = i * TPW + t;
#pragma unroll
        for (int gi = 0; gi < GPT; ++gi) {
          const uint32_t szw = szq[slot][gi];
          const uint32_t z = (szw >> 16) & 15u;
          const float s = O::scale_to_float(szw);
          const u32x4 corr = O::correction(z | (z << 16));
          f32x4 P = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int dd = 0; dd < DPG; ++dd) {
            const int d = gi * DPG + dd;
            const u32x4 bw = O::unpack(wq[slot][d], m_lo, m_hi, c_lo, c_hi);
            P = O::mfma(af[t][d], corr, P);
            P = O::mfma(af[t][d], bw, P);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[i][e] += s * P[e];
        }
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
    // every lane makes the call (the epilogue may exchange lanes); a column tile past the range stores nothing
    epi_store_acc<T>(p.epi, static_cast<uint16_t*>(p.out), sum, 4 * j, (nt_begin + wave) * 16 + c, p.M, p.N, wave < count);
  }
}

#define KSQ_GO4(MT, TPW, NB, NW) \
  hipLaunchKernelGGL((w4a16_kstat_kernel<T, GPT, MT, TPW, NB, NW, 4>), grid, dim3(64 * NW), 0, s, a)
// one row tile: the activation loads widen as the rows get fewer
#define KSQ_GO(MT, TPW, NB, NW)                                                                                  \
  do {                                                                                                           \
    if (MT == 1 && a.M <= 4)                                                                                     \
      hipLaunchKernelGGL((w4a16_kstat_kernel<T, GPT, 1, TPW, NB, NW, 16>), grid, dim3(64 * NW), 0, s, a);         \
    else if (MT == 1 && a.M <= 8)                                                                                \
      hipLaunchKernelGGL((w4a16_kstat_kernel<T, GPT, 1, TPW, NB, NW, 8>), grid, dim3(64 * NW), 0, s, a);          \
    else                                                                                                         \
      KSQ_GO4(MT, TPW, NB, NW);                                                                                  \
  } while (0)
template <typename T, int GPT>
void launch(const KstatPlan& pl, const KstatArgs& a, dim3 grid, hipStream_t s) {
  const int tpw = pl.tpw, nb = pl.nb;
  if (pl.mt == 1) {
    if (tpw <= 1) {
      if (nb >= 4) KSQ_GO(1, 1, 4, 16);
      else if (nb >= 2) KSQ_GO(1, 1, 2, 16);
      else KSQ_GO(1, 1, 1, 16);
    } else if (tpw == 2) {
      if (nb >= 4) KSQ_GO(1, 2, 4, 16);
      else if (nb >= 2) KSQ_GO(1, 2, 2, 16);
      else KSQ_GO(1, 2, 1, 16);
    } else if (tpw == 3) {
      if (nb >= 2) KSQ_GO(1, 3, 2, 16);
      else KSQ_GO(1, 3, 1, 16);
    } else {
      KSQ_GO(1, 4, 1, 16);  // 64 registers of activations: room for a ring of one column tile only
    }
  } else if (pl.mt == 2) {
    if (tpw <= 2) {
      if (nb >= 2) KSQ_GO4(2, 2, 2, 8);
      else KSQ_GO4(2, 2, 1, 8);
    } else {
      if (nb >= 2) KSQ_GO4(2, 4, 2, 8);
      else KSQ_GO4(2, 4, 1, 8);
    }
  } else {
    if (tpw <= 1) {
      if (nb >= 2) KSQ_GO4(4, 1, 2, 8);
      else KSQ_GO4(4, 1, 1, 8);
    } else {
      if (nb >= 2) KSQ_GO4(4, 2, 2, 8);
      else KSQ_GO4(4, 2, 1, 8);
    }
  }
}
#undef KSQ_GO
#undef KSQ_GO4

template <typename T, int GPT>
bool launch_kphase(int nb, int ppi, const KstatArgs& a, dim3 grid, hipStream_t s) {
#define KSQ_PH(NB, PPI) hipLaunchKernelGGL((w4a16_kphase_kernel<T, GPT, 2, NB, PPI>), grid, dim3(1024), 0, s, a)
  if (ppi == 16) {
    if (nb == 1) KSQ_PH(1, 16);
    else if (nb == 2) KSQ_PH(2, 16);
    else if (nb == 3) KSQ_PH(3, 16);
    else if (nb == 4) KSQ_PH(4, 16);
    else return false;
  } else {
    if (nb == 1) KSQ_PH(1, 8);
    else if (nb == 2) KSQ_PH(2, 8);
    else if (nb == 3) KSQ_PH(3, 8);
    else if (nb == 4) KSQ_PH(4, 8);
    else return false;
  }
#undef KSQ_PH
  return true;
}

}  // namespace

// Plan of the k-stationary kernel: row tiles (1, 2 or 4), waves per workgroup (16 for one row tile, else 8), k
// tiles per wave (the activations of waves x tpw k tiles live in registers: at most 64, 32 or 16 k tiles per
// workgroup for 1, 2 or 4 row tiles), split count, column tiles per workgroup and batch size.
// One row tile: three k tiles per wave (48 per workgroup) leave registers for a weight ring of two column tiles.
// Four (64: K = 8192 without a split across workgroups) leave room for a ring of one, which pays only where N is
// large (measured at the Llama-2-70B shapes: qkv -13 %, gate_up -6 %, o +10 %; beyond 64 k tiles the split wins).
static int kstat_tpw_max_one_row_tile(size_t ktiles, size_t ntiles, int cus) {
  if (const char* e = tuning_env("KSQ_W4_KSTAT_TPW_MAX")) {  // tuning / test override
    const int v = atoi(e);
    if (v >= 1 && v <= 4) return v;
  }
  return (ktiles > 48 && ktiles <= 64 && 2 * ntiles >= 5 * (size_t)cus) ? 4 : 3;
}

static bool env_round4() {
  const char* e = tuning_env("KSQ_W4_KSTAT_ROUND4");  // tuning / test switch
  return !(e && atoi(e) == 0);
}

KstatPlan w4a16_kstat_plan(size_t m, size_t n, size_t k, int cus, size_t workspace_bytes, size_t g) {
  KstatPlan p{};
  const size_t ntiles = n / kTileN, ktiles = k / kTileK;
  p.ok = m >= 1 && m <= 64 && ntiles * 4 <= (size_t)kCountersPerSlot;
  if (!p.ok) return p;
  p.mt = m <= 16 ? 1 : (m <= 32 ? 2 : 4);
  p.nw = p.mt == 1 ? 16 : 8;
  const size_t tpw_max = p.mt == 1 ? (size_t)kstat_tpw_max_one_row_tile(ktiles, ntiles, cus) : (p.mt == 2 ? 4 : 2);
  const size_t cap = (size_t)p.nw * tpw_max;
  size_t ksplit = (ktiles + cap - 1) / cap;
  if (const char* e = tuning_env("KSQ_W4_KSPLIT")) {  // tuning / test override; never below what the registers need
    const size_t v = (size_t)atoi(e);
    if (v > ksplit && v <= ktiles) ksplit = v;
  }
  // One to eight rows and a K that one pass does not cover: phases inside the workgroup instead of a split across
  // workgroups, where the column tiles alone give every CU one to four of them (see w4a16_kphase_kernel).  Measured
  // against the split: Llama-3-70B down (K = 28672) at one token 36.6 us, Llama-2-7B down 9.5 us.
  bool phases = p.mt == 1 && m <= 8 && ksplit >= 2 && ntiles * 4 >= 3 * (size_t)cus && ntiles <= 4 * (size_t)cus;
  if (const char* e = tuning_env("KSQ_W4_KPHASE")) {  // tuning / test switch: 0 = never, 1 = whenever the kernel can
    phases = atoi(e) != 0 && p.mt == 1 && m <= 8 && ntiles <= 4 * (size_t)cus && ktiles >= 2;
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
  auto need = [&](size_t ks) { return ks <= 1 ? (size_t)0 : ks * ntiles * p.mt * 64 * 16; };
  if (need(ksplit) > workspace_bytes) {
    p.ok = false;
    return p;
  }
  const size_t per_split = (ktiles + ksplit - 1) / ksplit;
  size_t tpw = (per_split + p.nw - 1) / p.nw;
  if (p.mt == 2) tpw = tpw <= 2 ? 2 : 4;  // instantiated widths
  p.ksplit = (int)ksplit;
  p.tpw = (int)tpw;
  size_t wgs = (size_t)cus / ksplit;
  if (wgs < 1) wgs = 1;
  if (wgs > ntiles) wgs = ntiles;
  p.nt_per_wg = (int)((ntiles + wgs - 1) / wgs);
  // One row tile: whole batches of four column tiles.  Fewer, fatter workgroups than CUs still win (measured at the
  // Llama-2-7B shapes: 3 -> 4 and 6 -> 8 column tiles per workgroup): every workgroup reads its whole k range of the
  // activations from the L2, and a short last batch costs a barrier and a reduction like a full one.
  // (beyond four with at most two k tiles per wave, where the batches are two tiles each, whole batches of two: six
  // tiles stay six -- at gate_up of Llama-2-7B 11.6 .. 11.9 us against 12.3 .. 13.0 with eight at M = 1, level at
  // M = 16; with four k tiles per wave, Llama-3-70B gate_up, sixteen tiles beat fourteen by 2 %)
  // (and three tiles stay three where a batch is one tile anyway: where the kernel takes the row-sum form, see below
  // -- a workgroup on every CU, Llama-2-7B qkv at one token 7.5 -> 7.0 us and 8.2 -> 7.9 at M = 16 -- and with four k
  // tiles per wave, Llama-3-70B qkv 11.7 -> 11.1 and 13.2 -> 12.4)
  const bool row_sums = p.mt == 1 && g == kTileK && p.tpw == 2 && ksplit == 1;
  const bool three = p.mt == 1 && (row_sums || p.tpw >= 4) && p.nt_per_wg == 3;
  if (p.mt == 1 && p.nt_per_wg >= 3 && env_round4() && !three)
    p.nt_per_wg = (p.nt_per_wg <= 4 || p.tpw >= 3) ? (p.nt_per_wg + 3) & ~3 : (p.nt_per_wg + 1) & ~1;
  if (const char* e = tuning_env("KSQ_W4_KSTAT_NT_PER_WG")) {  // tuning / test override: "v" or "ntiles:v,ntiles:v"
    for (const char* q = e; q && *q;) {
      const long a = strtol(q, const_cast<char**>(&q), 10);
      long v = a;
      bool applies = true;
      if (*q == ':') {
        v = strtol(q + 1, const_cast<char**>(&q), 10);
        applies = (size_t)a == ntiles;
      }
      if (applies && v >= 1 && (size_t)v <= ntiles) p.nt_per_wg = (int)v;
      if (*q == ',') ++q;
      else break;
    }
  }
  p.grid_x = (int)((ntiles + p.nt_per_wg - 1) / p.nt_per_wg);
  if (p.mt == 1) {
    // ring depth = nb * tpw tiles in flight per wave.  Four column tiles a batch where that is the whole workgroup;
    // with more than four the batches are two tiles each, so that the reduction of one batch overlaps the stream of
    // the next in finer steps (measured at Llama-2-7B gate_up, eight tiles per workgroup: 14.0 -> 12.3 us at M = 1,
    // 15.0 -> 13.3 at M = 16; qkv, four tiles per workgroup, is 3 % faster in one batch)
    p.nb = p.nt_per_wg >= 5 ? 2 : (p.nt_per_wg >= 3 ? 4 : (p.nt_per_wg >= 2 ? 2 : 1));
    // Two k tiles per wave and one group per k tile: batches of two keep the ring at four tiles, where the kernel
    // takes bias and zero point from the activations' row sums instead of a second matrix instruction per step
    // (Llama-2-7B qkv, three tiles per workgroup: 8.9 -> 8.3 us at M = 16, 8.1 -> 7.6 at one token).  Not with K
    // split over workgroups, where every batch ends in a hand-over (Llama-3-70B o: 10.9 -> 11.7 us in batches of two).
    if (row_sums && p.nb == 4) p.nb = 2;
    if (three && p.nt_per_wg == 3) p.nb = 1;
    if (p.tpw >= 3 && p.nb > 2) p.nb = 2;                       // register budget of 16 waves per workgroup
    if (p.tpw >= 4) p.nb = 1;
  } else {
    p.nb = p.nt_per_wg >= 2 ? 2 : 1;
  }
  if (const char* e = tuning_env("KSQ_W4_KSTAT_NB")) {  // tuning override, within what is instantiated
    const int v = atoi(e);
    if (p.mt == 1 && (v == 1 || v == 2 || (v == 4 && p.tpw <= 2)) && !(p.tpw >= 4 && v > 1) && v <= p.nt_per_wg) p.nb = v;
    if (p.mt >= 2 && (v == 1 || v == 2) && v <= p.nt_per_wg) p.nb = v;
  }
  p.partial_bytes = need(ksplit);
  return p;
}

int w4a16_launch_kstat(int dtype, const KstatPlan& plan, void* out, const void* act, const void* weight,
                       const void* sz, size_t m, size_t n, size_t k, size_t g, void* workspace, hipStream_t s,
                       const Epilogue& epi) {
  KSQ_REQUIRE(m * k * 2 < 0x7FFFFF00ull, KSQ_ERR_UNSUPPORTED, "activation tensor larger than 2 GiB");
  KSQ_REQUIRE(((size_t)plan.nt_per_wg + 8) * (k / kTileK) * 1024 < 0x3FFFFF00ull, KSQ_ERR_UNSUPPORTED,
              "column range of one workgroup larger than 1 GiB");
  KstatArgs a{};
  a.epi = epi;
  a.weight = weight;
  a.sz = sz;
  a.act = act;
  a.out = out;
  a.partial = static_cast<f32x4*>(workspace);
  a.M = (int)m;
  a.N = (int)n;
  a.K = (int)k;
  a.KT = (int)(k / kTileK);
  a.G = (int)(k / g);
  a.ntiles = (int)(n / kTileN);
  a.ksplit = plan.ksplit;
  a.nt_per_wg = plan.nt_per_wg;
  a.act_barrier = (plan.nt_per_wg + plan.nb - 1) / plan.nb >= 2 ? 1 : 0;
  a.counters = nullptr;
  if (plan.ksplit > 1) {
    KSQ_REQUIRE(workspace != nullptr, KSQ_ERR_WORKSPACE, "split-K planned without a workspace");
    a.counters = counter_slot_device_ptr(s);
    KSQ_REQUIRE(a.counters != nullptr, KSQ_ERR_HIP, "split-K planned for a stream without arrival counters");
  }
  dim3 grid((unsigned)plan.grid_x, (unsigned)plan.ksplit, 1);
  const int gpt = (int)(kTileK / g);
  if (plan.phases) {
    const int ppi = m <= 4 ? 16 : 8;
    note_launch("w4a16_kphase_kernel<tpw=2,nb=%d,gpt=%d,ppi=%d> grid=(%d)", plan.nb, gpt, ppi, plan.grid_x);
    bool ok;
    if (dtype == KSQ_F16) ok = gpt == 1 ? launch_kphase<_Float16, 1>(plan.nb, ppi, a, grid, s) : launch_kphase<_Float16, 2>(plan.nb, ppi, a, grid, s);
    else ok = gpt == 1 ? launch_kphase<__bf16, 1>(plan.nb, ppi, a, grid, s) : launch_kphase<__bf16, 2>(plan.nb, ppi, a, grid, s);
    KSQ_REQUIRE(ok, KSQ_ERR_UNSUPPORTED, "no phase kernel for %d column tiles per workgroup", plan.nb);
    KSQ_HIP_TRY(hipGetLastError());
    return KSQ_OK;
  }
  note_launch("w4a16_kstat_kernel<mt=%d,tpw=%d,nb=%d,nw=%d,gpt=%d,ppi=%d> grid=(%d,%d) nt_per_wg=%d", plan.mt, plan.tpw,
              plan.nb, plan.nw, gpt, plan.mt == 1 ? (m <= 4 ? 16 : (m <= 8 ? 8 : 4)) : 4, plan.grid_x, plan.ksplit,
              plan.nt_per_wg);
  if (dtype == KSQ_F16) {
    if (gpt == 1) launch<_Float16, 1>(plan, a, grid, s);
    else launch<_Float16, 2>(plan, a, grid, s);
  } else {
    if (gpt == 1) launch<__bf16, 1>(plan, a, grid, s);
    else launch<__bf16, 2>(plan, a, grid, s);
  }
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

}  // namespace ksq
