// W4A16 streaming kernel (decode regime, M <= 64; also the fallback for shapes the prefill kernel does not take).
//
// HBM-bound.  A workgroup is KS k-slices x 4 waves: the four waves of a slice own 4 x NT column tiles and share
// the slice's range of k tiles.  Every wave streams its 1 KiB weight tiles straight from HBM into a register ring
// D tiles deep (one 128-bit buffer load per lane is the B operand of four 16x16x32 MFMAs), while the activations
// of the slice's k range are staged once per slice into LDS in MFMA fragment order (double-buffered chunks of KCT
// tiles) and read back with conflict-free ds_read_b128.  Weights are read exactly once.
//
// Arithmetic: nibble u becomes the 16-bit pattern of bias + u with bit operations only (fp16: 1024 + u for
// nibbles at bits 0-3 of a half, 64 + u for nibbles at bits 4-7; bf16: 128 + u), which is exact.  A second MFMA per
// 32-k step multiplies the same activations with the per-column constant -(bias + z), so the accumulator holds the
// exact-integer group sum  sum_k a[m,k] * (u[k,n] - z[g,n])  (exact products, fp32 sums); the group scale is then
// applied in fp32:  acc += s[g,n] * P.  No floating-point VALU work is spent per weight.
//
// The k slices of a workgroup are reduced through LDS; a further split of k across workgroups (grid.y) is reduced
// by the last-arriving workgroup through a device-memory workspace.
//
// All global reads are range-checked buffer loads whose resource covers exactly the wave's k range of one column
// tile: tiles past the end of the range and padding column tiles read as zero without touching memory, which
// keeps the pipeline free of branches (the hardware retires loads in order, and the compiler can only leave later
// prefetches in flight across a wait when the number of loads issued after it is known statically).
#include "ksq_internal.h"
#include "ksq_epilogue.h"
#include "ksq_w4a16_ops.h"

namespace ksq {
namespace {

using namespace w4;

struct StreamArgs {
  const void* weight;  // [ntiles][KT][64] x 16 B
  const void* sz;      // [ntiles][G][16] x 4 B
  const void* act;     // [M][K] T
  void* out;           // [M][N] T
  f32x4* partial;      // [ksplit][mblocks][ntiles][MT][64]
  unsigned* counters;  // [mblocks * ngroups]
  int M, N, K, KT, G, ntiles, ngroups, ksplit;
  Epilogue epi;
};

template <typename T, int MT, int NT, int GPT, int D, int KCT, int KS>
__global__ __launch_bounds__(256 * KS)
    __attribute__((amdgpu_waves_per_eu(KS >= 4 ? 4 : (MT * NT >= 4 ? 1 : 2)))) void
w4a16_stream_kernel(StreamArgs p) {
  using O = Ops<T>;
  static_assert(D % KCT == 0 && ((D / KCT) % 2) == 0, "a ring round must span an even number of LDS chunks");
  constexpr int DPG = 4 / GPT;                       // MFMAs (32-k steps) per quantisation group inside one tile
  constexpr int NACC = (MT * NT <= 2 && DPG >= 2) ? 2 : 1;  // accumulators one group sum is spread over
  constexpr int kBuf = MT * KCT * 4 * 64;            // 16-byte elements per LDS buffer
  constexpr int kRed = (KS - 1) * 4 * MT * NT * 64;  // 16-byte elements of the slice reduction
  constexpr int kLds = KS * 2 * kBuf > kRed ? KS * 2 * kBuf : kRed;
  __shared__ u32x4 lds_a[kLds];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform, kept in a scalar register
  const int wcol = wave & 3, slice = wave >> 2;
  const int c = lane & 15, j = lane >> 4;
  const int grp = blockIdx.x * 4 + wcol;  // column-tile group of this wave
  const int nt0 = grp * NT;
  const int split = blockIdx.y, mblock = blockIdx.z;
  // k range of the workgroup, then of this wave's slice; every slice runs the same number of ring rounds
  int wg_begin, wg_end;
  split_range(p.KT, split, p.ksplit, &wg_begin, &wg_end);
  const int wg_tiles = wg_end - wg_begin;
  const int kt_begin = wg_begin + (wg_tiles * slice) / KS;
  const int kt_end = wg_begin + (wg_tiles * (slice + 1)) / KS;
  const int ntile = kt_end - kt_begin;
  const int rounds = ((wg_tiles + KS - 1) / KS + D - 1) / D;
  const int m0 = mblock * (16 * MT);

  __amdgpu_buffer_rsrc_t rs_w[NT], rs_sz[NT];
  bool tile_ok[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int nt = nt0 + t;
    tile_ok[t] = nt < p.ntiles;
    const size_t ntc = tile_ok[t] ? (size_t)nt : 0;
    const char* wb = static_cast<const char*>(p.weight) + (ntc * p.KT + kt_begin) * 1024;
    const char* sb = static_cast<const char*>(p.sz) + (ntc * p.G + (size_t)kt_begin * GPT) * 64;
    rs_w[t] = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(wb), 0, tile_ok[t] ? ntile * 1024 : 0, 0x00020000);
    rs_sz[t] =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(sb), 0, tile_ok[t] ? ntile * GPT * 64 : 0, 0x00020000);
  }
  const __amdgpu_buffer_rsrc_t rs_a =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.act), 0, (int)((size_t)p.M * p.K * 2), 0x00020000);
  // staging role of this thread inside its slice: fragment (MFMA index d = wcol, lane) of every tile of a chunk.
  // Padding rows sit at an offset that stays out of range for every k (k * 2 < 2^31); tiles past the k range read
  // real activations of the neighbouring range (or zeros past the end of the tensor), which meet zero weights and
  // a zero scale.
  unsigned a_off[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int row = m0 + 16 * mt + c;
    a_off[mt] = row < p.M ? ((unsigned)row * p.K + kt_begin * kTileK + 32 * wcol + 8 * j) * 2u : 0x80000000u;
  }
  const unsigned w_voff = lane * 16u, sz_voff = c * 4u;
  u32x4* const lds_s = lds_a + slice * (2 * kBuf);  // this slice's two activation buffers

  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 wq[D][NT];
  uint32_t szq[D][NT][GPT];
  u32x4 a_stage[2][MT][KCT];  // two chunks in flight: a chunk is fetched a full ring round before it is committed

  auto fetch = [&](int slot, int tile) {  // tile = index inside this wave's k range
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      wq[slot][t] =
          __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_w[t], w_voff + tile * 1024u, 0, 2));
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi)
        szq[slot][t][gi] = __builtin_amdgcn_raw_buffer_load_b32(rs_sz[t], sz_voff + (tile * GPT + gi) * 64u, 0, 0);
    }
  };
  auto stage_a = [&](int set, int chunk) {  // global -> registers
#pragma unroll
    for (int i = 0; i < KCT; ++i) {
      const unsigned tile = (unsigned)(chunk * KCT + i);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        a_stage[set][mt][i] =
            __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rs_a, a_off[mt] + tile * 256u, 0, 0));
    }
  };
  auto commit_a = [&](int set, int buf) {  // registers -> LDS, fragment order: [mt][tile][d][lane]
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < KCT; ++i)
        lds_s[buf * kBuf + ((mt * KCT + i) * 4 + wcol) * 64 + lane] = a_stage[set][mt][i];
  };

  // constants of the unpack kept in registers so that each output register costs one v_and_or_b32
  uint32_t m_lo = O::kMaskLo, m_hi = O::kMaskHi, c_lo = O::kMagicLo, c_hi = O::kMagicHi;
  KSQ_PIN_SGPR(m_lo);
  KSQ_PIN_VGPR(c_lo);
  KSQ_PIN_VGPR(c_hi);
  KSQ_PIN_VGPR(m_hi);

  // Software pipeline inside the wave.  A step issues the MFMAs of tile i from activation fragments that were
  // read from LDS at the end of step i - 1, and only then folds the group sums of tile i - 1 into the
  // accumulators, so neither the LDS latency nor the matrix-core latency is waited for.  Each group sum is kept in
  // two accumulators (alternating 32-k steps) to halve the dependent MFMA chain.
  u32x4 af[MT][4];
  f32x4 pend[MT][NT][GPT][NACC];
  float pend_s[NT][GPT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int gi = 0; gi < GPT; ++gi) {
      pend_s[t][gi] = 0.f;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int h = 0; h < NACC; ++h) pend[mt][t][gi][h] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  auto load_frags = [&](int buf, int il) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int d = 0; d < 4; ++d) af[mt][d] = lds_s[buf * kBuf + ((mt * KCT + il) * 4 + d) * 64 + lane];
  };
  auto flush = [&]() {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if constexpr (NACC == 2)
              acc[mt][t][i] += pend_s[t][gi] * (pend[mt][t][gi][0][i] + pend[mt][t][gi][1][i]);
            else
              acc[mt][t][i] += pend_s[t][gi] * pend[mt][t][gi][0][i];
          }
  };
  auto consume = [&](int slot) {
    f32x4 cur[MT][NT][GPT][NACC];
    float cur_s[NT][GPT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi) {
        const uint32_t szw = szq[slot][t][gi];
        const uint32_t z = (szw >> 16) & 15u;
        const u32x4 corr = O::correction(z | (z << 16));
        cur_s[t][gi] = O::scale_to_float(szw);
#pragma unroll
        for (int dd = 0; dd < DPG; ++dd) {
          const int d = gi * DPG + dd;
          const int h = dd % NACC;
          const u32x4 b = O::unpack(wq[slot][t][d], m_lo, m_hi, c_lo, c_hi);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            f32x4 pacc = dd < NACC ? f32x4{0.f, 0.f, 0.f, 0.f} : cur[mt][t][gi][h];
            pacc = O::mfma(af[mt][d], corr, pacc);
            cur[mt][t][gi][h] = O::mfma(af[mt][d], b, pacc);
          }
        }
      }
    }
    flush();  // previous tile, while this tile's MFMAs are in flight
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int gi = 0; gi < GPT; ++gi) {
        pend_s[t][gi] = cur_s[t][gi];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int h = 0; h < NACC; ++h) pend[mt][t][gi][h] = cur[mt][t][gi][h];
      }
  };

  // ---- pipeline: every wave of the workgroup runs the same number of rounds (uniform barriers)
  stage_a(0, 0);
  stage_a(1, 1);
  __builtin_amdgcn_sched_barrier(0);  // issue order = consumption order: loads retire in order
#pragma unroll
  for (int i = 0; i < D; ++i) {
    fetch(i, i);
    __builtin_amdgcn_sched_barrier(0);
  }
  commit_a(0, 0);
  stage_a(0, 2);
  __syncthreads();
  load_frags(0, 0);
  __builtin_amdgcn_sched_barrier(0);
  for (int r = 0; r < rounds; ++r) {
#pragma unroll
    for (int i = 0; i < D; ++i) {
      const int buf = (i / KCT) & 1;  // D / KCT is even, so the chunk parity is static inside a round
      const int il = i % KCT;
      consume(i);
      fetch(i, r * D + i + D);
      __builtin_amdgcn_sched_barrier(0);  // keep one tile's registers live at a time
      if (il == KCT - 1) {
        const int chunk = r * (D / KCT) + i / KCT;  // chunk just finished; its parity is that of buf
        commit_a(buf ^ 1, buf ^ 1);                 // chunk + 1, fetched a ring round ago
        stage_a(buf ^ 1, chunk + 3);
        __syncthreads();
        load_frags(buf ^ 1, 0);  // first tile of the next chunk
      } else {
        load_frags(buf, il + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  flush();

  // ---- reduce the k slices of the workgroup through LDS (the activation buffers are free now)
  if constexpr (KS > 1) {
    f32x4* red = reinterpret_cast<f32x4*>(lds_a);
    if (slice > 0) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t)
          red[((((slice - 1) * 4 + wcol) * MT + mt) * NT + t) * 64 + lane] = acc[mt][t];
    }
    __syncthreads();
    if (slice > 0) return;
#pragma unroll
    for (int sl = 1; sl < KS; ++sl)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[mt][t] += red[((((sl - 1) * 4 + wcol) * MT + mt) * NT + t) * 64 + lane];
  }

  if (grp >= p.ngroups) return;  // no barrier below this line

  // ---- epilogue: lane (c, j) holds column 16*nt + c, rows m0 + 16*mt + 4*j + i
  uint16_t* out = static_cast<uint16_t*>(p.out);
  auto store_out = [&](int mt, int t, f32x4 v) {
    if (!tile_ok[t]) return;  // uniform over the wave
    epi_store_acc<T>(p.epi, out, v, m0 + 16 * mt + 4 * j, (nt0 + t) * 16 + c, p.M, p.N, true);
  };

  if (p.ksplit == 1) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int t = 0; t < NT; ++t) store_out(mt, t, acc[mt][t]);
    return;
  }

  // split-K fix-up across workgroups: every split parks its fp32 tiles, the last one to arrive adds them in split
  // order (deterministic) and writes the result.  Counters return to zero for the next launch.
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
      if (tile_ok[t]) store_agent(p.partial + pidx(split, mt, t), acc[mt][t]);
  unsigned* ctr = p.counters + (size_t)mblock * p.ngroups + grp;
  if (!splitk_arrive_last(ctr, lane, p.ksplit)) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if (!tile_ok[t]) continue;
      f32x4 sum = {0.f, 0.f, 0.f, 0.f};
      for (int sp = 0; sp < p.ksplit; ++sp) sum += load_agent(p.partial + pidx(sp, mt, t));
      store_out(mt, t, sum);
    }
  if (lane == 0) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T, int MT, int NT, int GPT, int KS>
void launch_ks(const StreamArgs& a, dim3 grid, hipStream_t s) {
  constexpr int D = (NT == 4 || MT >= 3) ? 4 : 8;
  constexpr int KCT = (KS >= 2 || MT >= 3 || NT == 4) ? 2 : 4;
  hipLaunchKernelGGL((w4a16_stream_kernel<T, MT, NT, GPT, D, KCT, KS>), grid, dim3(256 * KS), 0, s, a);
}

template <typename T, int MT, int NT, int GPT>
void launch_one(int ks, const StreamArgs& a, dim3 grid, hipStream_t s) {
  if constexpr (MT == 1 && NT == 1) {
    if (ks == 4) return launch_ks<T, MT, NT, GPT, 4>(a, grid, s);
  }
  if constexpr (MT <= 2 && NT <= 2) {
    if (ks >= 2) return launch_ks<T, MT, NT, GPT, 2>(a, grid, s);
  }
  launch_ks<T, MT, NT, GPT, 1>(a, grid, s);
}

template <typename T, int MT, int NT>
void launch_gpt(int gpt, int ks, const StreamArgs& a, dim3 grid, hipStream_t s) {
  if (gpt == 1) launch_one<T, MT, NT, 1>(ks, a, grid, s);
  else launch_one<T, MT, NT, 2>(ks, a, grid, s);
}

template <typename T, int MT>
void launch_nt(int nt, int gpt, int ks, const StreamArgs& a, dim3 grid, hipStream_t s) {
  if (nt == 1) launch_gpt<T, MT, 1>(gpt, ks, a, grid, s);
  else if (nt == 2) launch_gpt<T, MT, 2>(gpt, ks, a, grid, s);
  else launch_gpt<T, MT, 4>(gpt, ks, a, grid, s);
}

template <typename T>
void launch_mt(int mt, int nt, int gpt, int ks, const StreamArgs& a, dim3 grid, hipStream_t s) {
  switch (mt) {
    case 1: launch_nt<T, 1>(nt, gpt, ks, a, grid, s); break;
    case 2: launch_nt<T, 2>(nt, gpt, ks, a, grid, s); break;
    case 3: launch_nt<T, 3>(nt, gpt, ks, a, grid, s); break;
    default: launch_nt<T, 4>(nt, gpt, ks, a, grid, s); break;
  }
}

}  // namespace

// in-workgroup k slices the kernel is instantiated with for a given wave tile
int w4a16_stream_max_slices(int mt, int nt) {
  if (mt == 1 && nt == 1) return 4;
  if (mt <= 2 && nt <= 2) return 2;
  return 1;
}

int w4a16_launch_stream(int dtype, const W4Plan& plan, void* out, const void* act, const void* weight,
                        const void* sz, size_t m, size_t n, size_t k, size_t g, void* workspace, hipStream_t s,
                        const Epilogue& epi) {
  // activations are addressed with 32-bit range-checked offsets
  KSQ_REQUIRE(m * k * 2 < 0x7FFFFF00ull, KSQ_ERR_UNSUPPORTED, "activation tensor larger than 2 GiB (m=%zu k=%zu)",
              m, k);
  KSQ_REQUIRE(plan.NT == 1 || plan.NT == 2 || plan.NT == 4, KSQ_ERR_INVALID_ARGUMENT, "bad plan");
  StreamArgs a{};
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
  a.ngroups = (a.ntiles + plan.NT - 1) / plan.NT;
  a.ksplit = plan.ksplit;
  a.counters = nullptr;
  if (plan.ksplit > 1) {
    KSQ_REQUIRE(workspace != nullptr, KSQ_ERR_WORKSPACE, "split-K planned without a workspace");
    KSQ_REQUIRE((size_t)a.ngroups * plan.mblocks <= (size_t)kCountersPerSlot, KSQ_ERR_UNSUPPORTED,
                "too many tiles for the split-K counters");
    a.counters = counter_slot_device_ptr(s);
    KSQ_REQUIRE(a.counters != nullptr, KSQ_ERR_HIP, "split-K planned for a stream without arrival counters");
  }
  KSQ_REQUIRE(plan.mblocks <= 65535 && plan.ksplit <= 65535, KSQ_ERR_UNSUPPORTED, "grid too large");
  dim3 grid((unsigned)((a.ngroups + 3) / 4), (unsigned)plan.ksplit, (unsigned)plan.mblocks);
  const int gpt = (int)(kTileK / g);
  note_launch("w4a16_stream_kernel<mt=%d,nt=%d,gpt=%d,slices=%d> grid=(%u,%u,%u)", plan.MT, plan.NT, gpt, plan.slices,
              grid.x, grid.y, grid.z);
  if (dtype == KSQ_F16) launch_mt<_Float16>(plan.MT, plan.NT, gpt, plan.slices, a, grid, s);
  else launch_mt<__bf16>(plan.MT, plan.NT, gpt, plan.slices, a, grid, s);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

}  // namespace ksq
