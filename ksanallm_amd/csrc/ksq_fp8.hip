// FP8 e4m3 (OCP) path: activation quantisation, rescale, on-the-fly weight conversion and the streaming GEMM.
#include <cstdlib>

#include "ksq_epilogue.h"
#include "ksq_fp8_ops.h"
#include "ksq_internal.h"

namespace ksq {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
using fp8ops::kE4m3Max;
using fp8ops::kMinScale;
using fp8ops::u32x2;
using fp8ops::u32x4;
using fp8ops::absmax8;
using fp8ops::quantize8;
using fp8ops::unpack8;

// element i of a tensor of T, as float.  The pointer is the tensor's base as the entry points take it (16-bit patterns
// for fp16 / bf16; for fp32 activations -- the reference's Fp8E4m3Quantize<float>, KS/kernels/nvidia/kernel_wrapper.cpp:1026
// -- the same pointer is a float array, and only the element-wise kernels below serve it)
template <typename T>
__device__ inline float load_as_float(const uint16_t* p, size_t i);
template <>
__device__ inline float load_as_float<_Float16>(const uint16_t* p, size_t i) {
  return (float)__builtin_bit_cast(_Float16, p[i]);
}
template <>
__device__ inline float load_as_float<__bf16>(const uint16_t* p, size_t i) {
  return __builtin_bit_cast(float, (uint32_t)p[i] << 16);
}
template <>
__device__ inline float load_as_float<float>(const uint16_t* p, size_t i) {
  return reinterpret_cast<const float*>(p)[i];
}

template <typename T>
__device__ inline uint16_t float_to_bits(float v);
template <>
__device__ inline uint16_t float_to_bits<_Float16>(float v) {
  return __builtin_bit_cast(uint16_t, (_Float16)v);
}
template <>
__device__ inline uint16_t float_to_bits<__bf16>(float v) {
  return __builtin_bit_cast(uint16_t, (__bf16)v);
}

// clamp(x / scale, +-448) -> e4m3 code (round to nearest even in hardware)
__device__ inline uint32_t quantize_pair(float a, float b, float scale) {
  float x = fminf(fmaxf(a / scale, -kE4m3Max), kE4m3Max);
  float y = fminf(fmaxf(b / scale, -kE4m3Max), kE4m3Max);
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(x, y, 0, false) & 0xFFFFu;
}

__device__ inline uint8_t quantize_one(float a, float scale) { return (uint8_t)(quantize_pair(a, 0.0f, scale) & 0xFFu); }

__device__ inline float block_max_256(float v, float* smem) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) smem[wave] = v;
  __syncthreads();
  v = fmaxf(fmaxf(smem[0], smem[1]), fmaxf(smem[2], smem[3]));
  __syncthreads();
  return v;
}

__global__ void fill_zero_kernel(float* p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0.0f;
}

// per-tensor abs-max -> scale, merged over blocks with an atomic max on the (non-negative) float bits
template <typename T>
__global__ __launch_bounds__(256) void absmax_scale_kernel(const uint16_t* x, size_t count, float* scale) {
  __shared__ float smem[4];
  float mx = 0.0f;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (size_t)gridDim.x * 256)
    mx = fmaxf(mx, fabsf(load_as_float<T>(x, i)));
  mx = block_max_256(mx, smem);
  if (threadIdx.x == 0) {
    float s = fmaxf(mx / kE4m3Max, kMinScale);
    atomicMax(reinterpret_cast<unsigned int*>(scale), __builtin_bit_cast(unsigned int, s));
  }
}

// elementwise quantisation with a given scale per channel (channel = row of length channel_size)
template <typename T>
__global__ __launch_bounds__(256) void quantize_kernel(const uint16_t* x, const float* scale, size_t num_channels,
                                                       size_t channel_size, uint8_t* q) {
  const size_t ch = blockIdx.y;
  const float s = scale[ch];
  uint8_t* qr = q + ch * channel_size;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < channel_size; i += (size_t)gridDim.x * 256)
    qr[i] = quantize_one(load_as_float<T>(x, ch * channel_size + i), s);
}

// per-token with the rows' maxima known (merged in by the GEMM that produced x): the scale, then one pass over the row.
// VEC: rows of whole 16-byte chunks (k % 8 == 0 and 16-byte aligned rows), eight elements per thread and step.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void quantize_rows_from_absmax_kernel(const uint16_t* x, size_t k, const float* row_absmax,
                                                                        uint8_t* q, float* scale) {
  const size_t row = blockIdx.x;
  const float s = fmaxf(row_absmax[row] / kE4m3Max, kMinScale);
  if (threadIdx.x == 0) scale[row] = s;
  if constexpr (VEC) {
    const u32x4* xv = reinterpret_cast<const u32x4*>(x + row * k);
    u32x2* qv = reinterpret_cast<u32x2*>(q + row * k);
    for (size_t i = threadIdx.x; i < k / 8; i += 256) {
      float f[8];
      fp8ops::unpack8<T>(xv[i], f);
      qv[i] = fp8ops::quantize8(f, s);
    }
  } else {
    for (size_t i = threadIdx.x; i < k; i += 256) q[row * k + i] = quantize_one(load_as_float<T>(x, row * k + i), s);
  }
}

// per-token: one block per row computes the row's scale and quantises the row
template <typename T>
__global__ __launch_bounds__(256) void quantize_per_token_kernel(const uint16_t* x, size_t k, uint8_t* q,
                                                                 float* scale) {
  __shared__ float smem[4];
  const size_t row = blockIdx.x;
  uint8_t* qr = q + row * k;
  float mx = 0.0f;
  for (size_t i = threadIdx.x; i < k; i += 256) mx = fmaxf(mx, fabsf(load_as_float<T>(x, row * k + i)));
  mx = block_max_256(mx, smem);
  const float s = fmaxf(mx / kE4m3Max, kMinScale);
  if (threadIdx.x == 0) scale[row] = s;
  for (size_t i = threadIdx.x; i < k; i += 256) qr[i] = quantize_one(load_as_float<T>(x, row * k + i), s);
}

// ---- vector forms (k a multiple of 8, 16-byte aligned rows): eight elements per lane and access; unpack8, absmax8 and
// quantize8 live in ksq_fp8_ops.h
template <int THREADS>
__device__ inline float block_max(float v, float* smem) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = v;
  __syncthreads();
  float m = smem[0];
#pragma unroll
  for (int w = 1; w < THREADS / 64; ++w) m = fmaxf(m, smem[w]);
  return m;
}

// One workgroup per row; the row stays in registers between the abs-max pass and the quantisation (R chunks of
// eight elements per lane), so it is read once.  Serves per-token rows and, with a single row, small whole tensors.
template <typename T, int THREADS, int R>
__global__ __launch_bounds__(THREADS) void quantize_rows_vec_kernel(const uint16_t* x, size_t k, uint8_t* q,
                                                                    float* scale) {
  __shared__ float smem[THREADS / 64];
  const size_t row = blockIdx.x;
  const u32x4* xr = reinterpret_cast<const u32x4*>(x + row * k);
  u32x2* qr = reinterpret_cast<u32x2*>(q + row * k);
  const unsigned nchunks = (unsigned)(k / 8);
  u32x4 v[R];
  float mx = 0.0f;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const unsigned c = threadIdx.x + i * THREADS;
    v[i] = c < nchunks ? xr[c] : u32x4{0u, 0u, 0u, 0u};
    float f[8];
    unpack8<T>(v[i], f);
    mx = absmax8(f, mx);
  }
  mx = block_max<THREADS>(mx, smem);
  const float s = fmaxf(mx / kE4m3Max, kMinScale);
  if (threadIdx.x == 0) scale[row] = s;
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const unsigned c = threadIdx.x + i * THREADS;
    float f[8];
    unpack8<T>(v[i], f);
    if (c < nchunks) qr[c] = quantize8(f, s);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void absmax_scale_vec_kernel(const u32x4* x, size_t nchunks, float* scale) {
  __shared__ float smem[4];
  float mx = 0.0f;
  for (size_t c = (size_t)blockIdx.x * 256 + threadIdx.x; c < nchunks; c += (size_t)gridDim.x * 256) {
    float f[8];
    unpack8<T>(x[c], f);
    mx = absmax8(f, mx);
  }
  mx = block_max<256>(mx, smem);
  if (threadIdx.x == 0) {
    float s = fmaxf(mx / kE4m3Max, kMinScale);
    atomicMax(reinterpret_cast<unsigned int*>(scale), __builtin_bit_cast(unsigned int, s));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void quantize_vec_kernel(const u32x4* x, const float* scale, size_t nchunks,
                                                           u32x2* q) {
  const float s = scale[0];
  for (size_t c = (size_t)blockIdx.x * 256 + threadIdx.x; c < nchunks; c += (size_t)gridDim.x * 256) {
    float f[8];
    unpack8<T>(x[c], f);
    q[c] = quantize8(f, s);
  }
}

template <typename T>
bool launch_rows_vec(const uint16_t* x, size_t rows, size_t k, uint8_t* q, float* scale, hipStream_t s) {
  if (k % 8 != 0 || (reinterpret_cast<uintptr_t>(x) & 15) != 0 || (reinterpret_cast<uintptr_t>(q) & 7) != 0) return false;
  const size_t nchunks = k / 8;
  dim3 grid((unsigned)rows);
  // few rows: spread a row over 1024 lanes; many rows: 256 lanes per row keep more rows in flight
  if (rows > 64 && nchunks <= 256 * 4) {
    if (nchunks <= 256) hipLaunchKernelGGL((quantize_rows_vec_kernel<T, 256, 1>), grid, dim3(256), 0, s, x, k, q, scale);
    else if (nchunks <= 512) hipLaunchKernelGGL((quantize_rows_vec_kernel<T, 256, 2>), grid, dim3(256), 0, s, x, k, q, scale);
    else hipLaunchKernelGGL((quantize_rows_vec_kernel<T, 256, 4>), grid, dim3(256), 0, s, x, k, q, scale);
    return true;
  }
  if (nchunks > 1024 * 8) return false;
  if (nchunks <= 1024) hipLaunchKernelGGL((quantize_rows_vec_kernel<T, 1024, 1>), grid, dim3(1024), 0, s, x, k, q, scale);
  else if (nchunks <= 2048) hipLaunchKernelGGL((quantize_rows_vec_kernel<T, 1024, 2>), grid, dim3(1024), 0, s, x, k, q, scale);
  else if (nchunks <= 4096) hipLaunchKernelGGL((quantize_rows_vec_kernel<T, 1024, 4>), grid, dim3(1024), 0, s, x, k, q, scale);
  else hipLaunchKernelGGL((quantize_rows_vec_kernel<T, 1024, 8>), grid, dim3(1024), 0, s, x, k, q, scale);
  return true;
}

__device__ inline float e4m3_to_float(uint8_t c) {
  return __builtin_amdgcn_cvt_f32_fp8((int)c, 0);
}

__global__ __launch_bounds__(256) void rescale_kernel(const uint8_t* in, uint8_t* out, size_t count,
                                                      const float* s_in, const float* s_out) {
  const float r = *s_in / *s_out;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < count; i += (size_t)gridDim.x * 256) {
    float v = fminf(fmaxf(e4m3_to_float(in[i]) * r, -kE4m3Max), kE4m3Max);  // the cast saturates to +-448
    out[i] = (uint8_t)((uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(v, 0.0f, 0, false) & 0xFFu);
  }
}

// [k,n] T -> [n,k] e4m3 through a 64x64 LDS tile
template <typename T>
__global__ __launch_bounds__(256) void transpose_quantize_kernel(const uint16_t* w, size_t k, size_t n,
                                                                 const float* scale, uint8_t* wq) {
  __shared__ uint8_t tile[64][65];
  const float s = *scale;
  const size_t k0 = (size_t)blockIdx.y * 64, n0 = (size_t)blockIdx.x * 64;
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    int kk = i >> 6, nn = i & 63;
    uint8_t v = 0;
    if (k0 + kk < k && n0 + nn < n) v = quantize_one(load_as_float<T>(w, (k0 + kk) * n + n0 + nn), s);
    tile[kk][nn] = v;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    int nn = i >> 6, kk = i & 63;
    if (k0 + kk < k && n0 + nn < n) wq[(n0 + nn) * k + k0 + kk] = tile[kk][nn];
  }
}

// per-column abs-max of a [k,n] tensor -> scale[n] (merged over row blocks with an atomic max on the float bits)
template <typename T>
__global__ __launch_bounds__(256) void colmax_scale_kernel(const uint16_t* w, size_t k, size_t n, float* scale) {
  const size_t col = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (col >= n) return;
  const size_t rows = (k + gridDim.y - 1) / gridDim.y, k0 = (size_t)blockIdx.y * rows;
  const size_t k1 = k0 + rows < k ? k0 + rows : k;
  float mx = 0.0f;
  for (size_t r = k0; r < k1; ++r) mx = fmaxf(mx, fabsf(load_as_float<T>(w, r * n + col)));
  const float s = fmaxf(mx / kE4m3Max, kMinScale);
  atomicMax(reinterpret_cast<unsigned int*>(scale + col), __builtin_bit_cast(unsigned int, s));
}

// [k,n] T -> [n,k] e4m3 through a 64x64 LDS tile, one scale per column of the source (= row of the result)
template <typename T>
__global__ __launch_bounds__(256) void transpose_quantize_per_channel_kernel(const uint16_t* w, size_t k, size_t n,
                                                                             const float* scale, uint8_t* wq) {
  __shared__ uint8_t tile[64][65];
  const size_t k0 = (size_t)blockIdx.y * 64, n0 = (size_t)blockIdx.x * 64;
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    int kk = i >> 6, nn = i & 63;
    uint8_t v = 0;
    if (k0 + kk < k && n0 + nn < n) v = quantize_one(load_as_float<T>(w, (k0 + kk) * n + n0 + nn), scale[n0 + nn]);
    tile[kk][nn] = v;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * 64; i += 256) {
    int nn = i >> 6, kk = i & 63;
    if (k0 + kk < k && n0 + nn < n) wq[(n0 + nn) * k + k0 + kk] = tile[kk][nn];
  }
}

__global__ void max3_kernel(const float* a, const float* b, const float* c, float* out) {
  if (threadIdx.x == 0 && blockIdx.x == 0) out[0] = fmaxf(fmaxf(a[0], b[0]), c[0]);
}

__global__ __launch_bounds__(256) void expand3_kernel(const float* a, const float* b, const float* c, size_t na,
                                                      size_t nb, size_t nc, float* out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < na + nb + nc) out[i] = i < na ? a[0] : (i < na + nb ? b[0] : c[0]);
}

// ---- streaming GEMM ------------------------------------------------------------------------------------------
struct Fp8Args {
  const uint8_t* aq;  // [M][K]
  const uint8_t* wq;  // [N][K]
  const float* a_scale;
  const float* w_scale;
  void* out;  // [M][N] T
  f32x4* partial;
  unsigned* counters;
  int M, N, K, KB /* 128-byte k blocks, rounded up */, ntiles, ksplit;
  int a_scale_per_row, w_scale_per_col;
  Epilogue epi;
};

// Wave = one 16-column tile x a range of 128-k blocks.  Each lane reads 2 x 16 B of its weight row per block (the
// B operands of four 16x16x32 fp8 MFMAs) and the matching 2 x 16 B of each activation row tile.
template <typename T, int MT, int D>
__global__ __launch_bounds__(256) void fp8_stream_kernel(Fp8Args p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, j = lane >> 4;
  const int nt = blockIdx.x * 4 + wave;
  if (nt >= p.ntiles) return;  // wave-uniform; no block-level barrier below
  const int split = blockIdx.y, mblock = blockIdx.z;
  int kb_begin, kb_end;
  split_range(p.KB, split, p.ksplit, &kb_begin, &kb_end);
  const int m0 = mblock * 16 * MT;

  int wrow = nt * 16 + c;
  wrow = wrow < p.N ? wrow : p.N - 1;
  const uint8_t* wptr = p.wq + (size_t)wrow * p.K + 16 * j;
  const uint8_t* aptr[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int row = m0 + 16 * mt + c;
    row = row < p.M ? row : p.M - 1;
    aptr[mt] = p.aq + (size_t)row * p.K + 16 * j;
  }

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 wq[D][2];
  u32x4 aq[D][MT][2];
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  auto fetch = [&](int slot, int kb) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int koff = kb * 128 + 64 * h;
      const bool ok = koff + 16 * j < p.K;  // K % 16 == 0, so a 16-byte chunk is inside or outside as a whole
      wq[slot][h] = ok ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wptr + koff)) : zero4;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        aq[slot][mt][h] = ok ? *reinterpret_cast<const u32x4*>(aptr[mt] + koff) : zero4;
    }
  };
  auto consume = [&](int slot) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        u32x2 bw = {wq[slot][h][2 * q], wq[slot][h][2 * q + 1]};
        const long b = __builtin_bit_cast(long, bw);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          u32x2 aw = {aq[slot][mt][h][2 * q], aq[slot][mt][h][2 * q + 1]};
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(__builtin_bit_cast(long, aw), b, acc[mt], 0, 0, 0);
        }
      }
  };

#pragma unroll
  for (int i = 0; i < D; ++i)
    if (kb_begin + i < kb_end) fetch(i, kb_begin + i);
  for (int kb = kb_begin; kb < kb_end; kb += D) {
#pragma unroll
    for (int i = 0; i < D; ++i) {
      if (kb + i < kb_end) {
        consume(i);
        if (kb + i + D < kb_end) fetch(i, kb + i + D);
      }
    }
  }

  epi_elem_t<T>* out = static_cast<epi_elem_t<T>*>(p.out);
  const int col = nt * 16 + c;
  const float ws = p.w_scale[p.w_scale_per_col ? (col < p.N ? col : p.N - 1) : 0];
  auto store_out = [&](int mt, f32x4 v) {
    const int row0 = m0 + 16 * mt + 4 * j;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = row0 + i;
      v[i] = (v[i] * ws) * p.a_scale[p.a_scale_per_row ? (row < p.M ? row : p.M - 1) : 0];
    }
    epi_store_acc<T>(p.epi, out, v, row0, col, p.M, p.N, col < p.N);
  };

  if (p.ksplit == 1) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) store_out(mt, acc[mt]);
    return;
  }
  const size_t split_stride = (size_t)gridDim.z * p.ntiles * MT * 64;
  auto pidx = [&](int sp, int mt) {
    return (size_t)sp * split_stride + (((size_t)mblock * p.ntiles + nt) * MT + mt) * 64 + lane;
  };
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) store_agent(p.partial + pidx(split, mt), acc[mt]);
  unsigned* ctr = p.counters + (size_t)mblock * p.ntiles + nt;
  if (!splitk_arrive_last(ctr, lane, p.ksplit)) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    for (int sp = 0; sp < p.ksplit; ++sp) sum += load_agent(p.partial + pidx(sp, mt));
    store_out(mt, sum);
  }
  if (lane == 0) __hip_atomic_store(ctr, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T>
void launch_fp8_stream(int mt, const Fp8Args& a, dim3 grid, hipStream_t s) {
  switch (mt) {
    case 1: hipLaunchKernelGGL((fp8_stream_kernel<T, 1, 4>), grid, dim3(256), 0, s, a); break;
    case 2: hipLaunchKernelGGL((fp8_stream_kernel<T, 2, 3>), grid, dim3(256), 0, s, a); break;
    case 3: hipLaunchKernelGGL((fp8_stream_kernel<T, 3, 2>), grid, dim3(256), 0, s, a); break;
    default: hipLaunchKernelGGL((fp8_stream_kernel<T, 4, 2>), grid, dim3(256), 0, s, a); break;
  }
}

unsigned blocks_for(size_t count, unsigned cap) {
  size_t b = (count + 255) / 256;
  if (b < 1) b = 1;
  return (unsigned)(b > cap ? cap : b);
}

}  // namespace
}  // namespace ksq

using namespace ksq;

extern "C" {

int ksq_fp8_quantize(int dtype, const void* act, size_t m, size_t k, int mode, void* act_q, float* act_scale,
                     void* stream) {
  KSQ_REQUIRE(dtype == KSQ_F16 || dtype == KSQ_BF16 || dtype == KSQ_F32, KSQ_ERR_INVALID_ARGUMENT, "bad dtype %d", dtype);
  KSQ_REQUIRE(mode >= KSQ_FP8_PER_TENSOR_DYNAMIC && mode <= KSQ_FP8_PER_TOKEN_DYNAMIC, KSQ_ERR_INVALID_ARGUMENT,
              "bad quantisation mode %d", mode);
  KSQ_REQUIRE(act && act_q && act_scale, KSQ_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if (m == 0 || k == 0) return KSQ_OK;
  KSQ_REQUIRE(m <= 65535u * 16u, KSQ_ERR_UNSUPPORTED, "m=%zu too large", m);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t* x = static_cast<const uint16_t*>(act);
  uint8_t* q = static_cast<uint8_t*>(act_q);
  if (dtype == KSQ_F32) {  // fp32 activations: the element-wise kernels (the vector forms read 16-bit elements)
    if (mode == KSQ_FP8_PER_TOKEN_DYNAMIC) {
      KSQ_REQUIRE(m < (1ull << 31), KSQ_ERR_UNSUPPORTED, "m too large");
      hipLaunchKernelGGL(quantize_per_token_kernel<float>, dim3((unsigned)m), dim3(256), 0, s, x, k, q, act_scale);
    } else {
      const size_t count = m * k;
      if (mode == KSQ_FP8_PER_TENSOR_DYNAMIC) {
        hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, s, act_scale, 1);
        hipLaunchKernelGGL(absmax_scale_kernel<float>, dim3(blocks_for(count, 2048)), dim3(256), 0, s, x, count, act_scale);
      }
      hipLaunchKernelGGL(quantize_kernel<float>, dim3(blocks_for(count, 4096), 1), dim3(256), 0, s, x, act_scale, (size_t)1,
                         count, q);
    }
    KSQ_HIP_TRY(hipGetLastError());
    return KSQ_OK;
  }
  const bool f16 = dtype == KSQ_F16;
  if (mode == KSQ_FP8_PER_TOKEN_DYNAMIC) {
    KSQ_REQUIRE(m < (1ull << 31), KSQ_ERR_UNSUPPORTED, "m too large");
    const bool done = f16 ? launch_rows_vec<_Float16>(x, m, k, q, act_scale, s) : launch_rows_vec<__bf16>(x, m, k, q, act_scale, s);
    if (!done) {
      if (f16) hipLaunchKernelGGL(quantize_per_token_kernel<_Float16>, dim3((unsigned)m), dim3(256), 0, s, x, k, q, act_scale);
      else hipLaunchKernelGGL(quantize_per_token_kernel<__bf16>, dim3((unsigned)m), dim3(256), 0, s, x, k, q, act_scale);
    }
  } else {
    const size_t count = m * k;
    const bool vec = count % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0;
    // a small tensor is one row of one workgroup: abs-max and quantisation in a single launch
    if (mode == KSQ_FP8_PER_TENSOR_DYNAMIC && vec && count <= 65536 &&
        (f16 ? launch_rows_vec<_Float16>(x, 1, count, q, act_scale, s) : launch_rows_vec<__bf16>(x, 1, count, q, act_scale, s))) {
      KSQ_HIP_TRY(hipGetLastError());
      return KSQ_OK;
    }
    if (mode == KSQ_FP8_PER_TENSOR_DYNAMIC) {
      // a fill kernel rather than a memset node keeps the call safe to record into a HIP graph
      hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, s, act_scale, 1);
      if (vec) {
        const unsigned nb = blocks_for(count / 8, 1024);
        const u32x4* xv = reinterpret_cast<const u32x4*>(x);
        if (f16) hipLaunchKernelGGL(absmax_scale_vec_kernel<_Float16>, dim3(nb), dim3(256), 0, s, xv, count / 8, act_scale);
        else hipLaunchKernelGGL(absmax_scale_vec_kernel<__bf16>, dim3(nb), dim3(256), 0, s, xv, count / 8, act_scale);
      } else {
        const unsigned nb = blocks_for(count, 2048);
        if (f16) hipLaunchKernelGGL(absmax_scale_kernel<_Float16>, dim3(nb), dim3(256), 0, s, x, count, act_scale);
        else hipLaunchKernelGGL(absmax_scale_kernel<__bf16>, dim3(nb), dim3(256), 0, s, x, count, act_scale);
      }
    }
    if (vec) {
      const unsigned nb = blocks_for(count / 8, 1024);
      const u32x4* xv = reinterpret_cast<const u32x4*>(x);
      u32x2* qv = reinterpret_cast<u32x2*>(q);
      if (f16) hipLaunchKernelGGL(quantize_vec_kernel<_Float16>, dim3(nb), dim3(256), 0, s, xv, act_scale, count / 8, qv);
      else hipLaunchKernelGGL(quantize_vec_kernel<__bf16>, dim3(nb), dim3(256), 0, s, xv, act_scale, count / 8, qv);
    } else {
      const unsigned nb = blocks_for(count, 4096);
      if (f16) hipLaunchKernelGGL(quantize_kernel<_Float16>, dim3(nb, 1), dim3(256), 0, s, x, act_scale, (size_t)1, count, q);
      else hipLaunchKernelGGL(quantize_kernel<__bf16>, dim3(nb, 1), dim3(256), 0, s, x, act_scale, (size_t)1, count, q);
    }
  }
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

int ksq_fp8_rescale(const void* in, void* out, size_t count, const float* scale_in, const float* scale_out,
                    void* stream) {
  KSQ_REQUIRE(in && out && scale_in && scale_out, KSQ_ERR_INVALID_ARGUMENT, "null pointer");
  if (count == 0) return KSQ_OK;
  hipLaunchKernelGGL(rescale_kernel, dim3(blocks_for(count, 4096)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), count, scale_in, scale_out);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

int ksq_fp8_convert_weight(int dtype, const void* w, size_t k, size_t n, void* w_q, float* w_scale, void* stream) {
  KSQ_REQUIRE(dtype == KSQ_F16 || dtype == KSQ_BF16, KSQ_ERR_INVALID_ARGUMENT, "bad dtype %d", dtype);
  KSQ_REQUIRE(w && w_q && w_scale, KSQ_ERR_INVALID_ARGUMENT, "null tensor pointer");
  KSQ_REQUIRE(k > 0 && n > 0, KSQ_ERR_INVALID_ARGUMENT, "k and n must be positive");
  KSQ_REQUIRE((k + 63) / 64 <= 65535, KSQ_ERR_UNSUPPORTED, "k too large");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t* x = static_cast<const uint16_t*>(w);
  const size_t count = k * n;
  hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(64), 0, s, w_scale, 1);
  const unsigned nb = blocks_for(count, 2048);
  dim3 grid((unsigned)((n + 63) / 64), (unsigned)((k + 63) / 64));
  if (dtype == KSQ_F16) {
    hipLaunchKernelGGL(absmax_scale_kernel<_Float16>, dim3(nb), dim3(256), 0, s, x, count, w_scale);
    hipLaunchKernelGGL(transpose_quantize_kernel<_Float16>, grid, dim3(256), 0, s, x, k, n, w_scale,
                       static_cast<uint8_t*>(w_q));
  } else {
    hipLaunchKernelGGL(absmax_scale_kernel<__bf16>, dim3(nb), dim3(256), 0, s, x, count, w_scale);
    hipLaunchKernelGGL(transpose_quantize_kernel<__bf16>, grid, dim3(256), 0, s, x, k, n, w_scale,
                       static_cast<uint8_t*>(w_q));
  }
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

int ksq_fp8_convert_weight_per_channel(int dtype, const void* w, size_t k, size_t n, void* w_q, float* w_scale,
                                       void* stream) {
  KSQ_REQUIRE(dtype == KSQ_F16 || dtype == KSQ_BF16, KSQ_ERR_INVALID_ARGUMENT, "bad dtype %d", dtype);
  KSQ_REQUIRE(w && w_q && w_scale, KSQ_ERR_INVALID_ARGUMENT, "null tensor pointer");
  KSQ_REQUIRE(k > 0 && n > 0, KSQ_ERR_INVALID_ARGUMENT, "k and n must be positive");
  KSQ_REQUIRE((k + 63) / 64 <= 65535 && n < (1ull << 31), KSQ_ERR_UNSUPPORTED, "k or n too large");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t* x = static_cast<const uint16_t*>(w);
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, w_scale, (int)n);
  size_t kblocks = (k + 511) / 512;
  if (kblocks > 64) kblocks = 64;
  dim3 cgrid((unsigned)((n + 255) / 256), (unsigned)kblocks);
  dim3 grid((unsigned)((n + 63) / 64), (unsigned)((k + 63) / 64));
  if (dtype == KSQ_F16) {
    hipLaunchKernelGGL(colmax_scale_kernel<_Float16>, cgrid, dim3(256), 0, s, x, k, n, w_scale);
    hipLaunchKernelGGL(transpose_quantize_per_channel_kernel<_Float16>, grid, dim3(256), 0, s, x, k, n, w_scale,
                       static_cast<uint8_t*>(w_q));
  } else {
    hipLaunchKernelGGL(colmax_scale_kernel<__bf16>, cgrid, dim3(256), 0, s, x, k, n, w_scale);
    hipLaunchKernelGGL(transpose_quantize_per_channel_kernel<__bf16>, grid, dim3(256), 0, s, x, k, n, w_scale,
                       static_cast<uint8_t*>(w_q));
  }
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

int ksq_fp8_merge_qkv_scales(int mode, const float* q_scale, const float* k_scale, const float* v_scale, size_t nq,
                             size_t nk, size_t nv, void* w_q, size_t k, float* w_scale, void* stream) {
  KSQ_REQUIRE(mode == KSQ_FP8_MERGE_MAX || mode == KSQ_FP8_MERGE_PER_CHANNEL, KSQ_ERR_INVALID_ARGUMENT,
              "bad merge mode %d", mode);
  KSQ_REQUIRE(q_scale && k_scale && v_scale && w_scale, KSQ_ERR_INVALID_ARGUMENT, "null scale pointer");
  KSQ_REQUIRE(nq > 0 && nk > 0 && nv > 0 && k > 0, KSQ_ERR_INVALID_ARGUMENT, "row counts and k must be positive");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (mode == KSQ_FP8_MERGE_PER_CHANNEL) {
    const size_t n = nq + nk + nv;
    KSQ_REQUIRE(n < (1ull << 31), KSQ_ERR_UNSUPPORTED, "too many rows");
    hipLaunchKernelGGL(expand3_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, q_scale, k_scale, v_scale, nq,
                       nk, nv, w_scale);
  } else {
    KSQ_REQUIRE(w_q != nullptr, KSQ_ERR_INVALID_ARGUMENT, "the max merge rescales the weight: w_q is null");
    hipLaunchKernelGGL(max3_kernel, dim3(1), dim3(64), 0, s, q_scale, k_scale, v_scale, w_scale);
    uint8_t* base = static_cast<uint8_t*>(w_q);
    const float* part_scale[3] = {q_scale, k_scale, v_scale};
    const size_t part_rows[3] = {nq, nk, nv};
    size_t row0 = 0;
    for (int i = 0; i < 3; ++i) {
      const size_t count = part_rows[i] * k;
      hipLaunchKernelGGL(rescale_kernel, dim3(blocks_for(count, 4096)), dim3(256), 0, s, base + row0 * k, base + row0 * k,
                         count, part_scale[i], w_scale);
      row0 += part_rows[i];
    }
  }
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

static int check_fp8_shape(size_t n, size_t k) {
  KSQ_REQUIRE(k > 0 && n > 0, KSQ_ERR_INVALID_ARGUMENT, "k and n must be positive (k=%zu n=%zu)", k, n);
  KSQ_REQUIRE(k % 16 == 0, KSQ_ERR_UNSUPPORTED, "k=%zu must be a multiple of 16", k);
  KSQ_REQUIRE(k < (1u << 30) && n < (1u << 30), KSQ_ERR_UNSUPPORTED, "k or n too large");
  return KSQ_OK;
}

int ksq_fp8_workspace_bytes(size_t max_m, size_t n, size_t k, size_t* bytes) {
  KSQ_REQUIRE(bytes, KSQ_ERR_INVALID_ARGUMENT, "null output pointer");
  KSQ_REQUIRE(max_m > 0, KSQ_ERR_INVALID_ARGUMENT, "max_m must be positive");
  int rc = check_fp8_shape(n, k);
  if (rc != KSQ_OK) return rc;
  const DeviceInfo* di = device_info();
  const int cus = di ? di->cus : 256;
  size_t best = 0;
  const size_t ms[4] = {16, 32, 48, 64};
  for (size_t mm : ms) {
    if (mm - 15 > max_m) break;
    Fp8Plan p = fp8_plan(mm, n, k, cus, (size_t)-1);
    if (p.partial_bytes > best) best = p.partial_bytes;
    const Fp8KstatPlan kp = fp8_kstat_plan(mm < max_m ? mm : max_m, n, k, cus, (size_t)-1);
    if (kp.ok && kp.partial_bytes > best) best = kp.partial_bytes;
  }
  // large m: the partial tiles of a split (last) round of 256 x 256 tiles; the plan depends on the number of 256-row
  // blocks only
  for (size_t mb = 1; mb <= (max_m + 255) / 256 && mb <= 64; ++mb) {
    const size_t mm = mb * 256 < max_m ? mb * 256 : max_m;
    if (fp8_prefill_supported(mm, n, k, cus)) {
      const size_t need = fp8_prefill_workspace_bytes(mm, n, k, cus);
      if (need > best) best = need;
    }
  }
  *bytes = best;
  return KSQ_OK;
}

// front part of the workspace of ksq_fp8_gemm_dynamic: e4m3 activations and one scale per row, each rounded up to 256
static size_t dynamic_front_bytes(size_t m, size_t k) { return (m * k + 255) / 256 * 256 + (m * 4 + 255) / 256 * 256; }

int ksq_fp8_gemm_dynamic_workspace_bytes(size_t max_m, size_t n, size_t k, size_t* bytes) {
  int rc = ksq_fp8_workspace_bytes(max_m, n, k, bytes);
  if (rc != KSQ_OK) return rc;
  *bytes = (*bytes + 255) / 256 * 256 + dynamic_front_bytes(max_m, k);
  return KSQ_OK;
}

int ksq_fp8_gemm_dynamic(int dtype, void* out, const void* act, const void* w_q, const float* w_scale,
                         size_t w_scale_count, size_t m, size_t n, size_t k, int epilogue, const void* bias,
                         void* workspace, size_t workspace_bytes, void* stream) {
  KSQ_REQUIRE(dtype == KSQ_F16 || dtype == KSQ_BF16 || dtype == KSQ_F32, KSQ_ERR_INVALID_ARGUMENT, "bad dtype %d", dtype);
  KSQ_REQUIRE(out && act && w_q && w_scale, KSQ_ERR_INVALID_ARGUMENT, "null tensor pointer");
  KSQ_REQUIRE(epilogue >= KSQ_EPILOGUE_NONE && epilogue <= KSQ_EPILOGUE_SILU_MUL, KSQ_ERR_INVALID_ARGUMENT,
              "bad epilogue %d", epilogue);
  KSQ_REQUIRE(epilogue != KSQ_EPILOGUE_BIAS || (bias && (reinterpret_cast<uintptr_t>(bias) & 15) == 0),
              KSQ_ERR_INVALID_ARGUMENT, "the bias epilogue needs a 16-byte aligned bias");
  KSQ_REQUIRE(epilogue != KSQ_EPILOGUE_SILU_MUL || n % 16 == 0, KSQ_ERR_UNSUPPORTED,
              "the SiLU-mul epilogue needs n %% 16 == 0 (got %zu)", n);
  int rc = check_fp8_shape(n, k);
  if (rc != KSQ_OK) return rc;
  if (m == 0) return KSQ_OK;
  KSQ_REQUIRE(w_scale_count == 1 || w_scale_count == n, KSQ_ERR_INVALID_ARGUMENT,
              "w_scale_count must be 1 or n (got %zu)", w_scale_count);
  KSQ_REQUIRE((reinterpret_cast<uintptr_t>(act) & 15) == 0 && (reinterpret_cast<uintptr_t>(w_q) & 15) == 0,
              KSQ_ERR_INVALID_ARGUMENT, "act and w_q must be 16-byte aligned");
  const DeviceInfo* di = device_info();
  if (!di) return KSQ_ERR_HIP;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255) != 0) workspace = nullptr;
  if (!workspace) workspace_bytes = 0;
  const size_t front = dynamic_front_bytes(m, k);
  char* gemm_ws = workspace_bytes > front ? static_cast<char*>(workspace) + front : nullptr;
  size_t gemm_ws_bytes = gemm_ws ? workspace_bytes - front : 0;
  // One launch instead of two: the kernel that takes the row maxima and quantises its share of the activations itself.
  // Every one of its workgroups repeats that work, so it only ties with the two launches at a single row without a
  // split of K (Qwen-72B qkv: 22.2 us against 3.0 + 19.3) and loses beyond (two rows 23.5 against 22.5, eight rows
  // 29.9 against 23.6; K = 29568, split four ways: 65.9 against 59.3): it serves m = 1, and up to eight rows on request.
  const char* sw = tuning_env("KSQ_FP8_FUSED_QUANT");  // tuning / test switch: 0 = never, 1 = up to eight rows
  const size_t fused_rows = sw ? (atoi(sw) == 0 ? 0 : 8) : 1;
  if (m <= fused_rows && dtype != KSQ_F32 && k % 128 == 0 && m * k * 2 < 0x7FFFFF00ull) {
    if (gemm_ws && !counter_slot_available(s)) gemm_ws = nullptr, gemm_ws_bytes = 0;
    const Fp8KstatPlan kp = fp8_kstat_plan(m, n, k, di->cus, gemm_ws_bytes, true);
    if (kp.ok && kp.nb <= 2 && kp.tpw <= 4 && (kp.ksplit == 1 || sw)) {
      Epilogue epi;
      epi.kind = epilogue;
      epi.bias = bias;
      return fp8_launch_kstat(dtype, kp, out, nullptr, nullptr, m, w_q, w_scale, w_scale_count, m, n, k, gemm_ws, s, epi,
                              act);
    }
  }
  // Otherwise: quantise into the front of the workspace, then the GEMM.
  KSQ_REQUIRE(workspace_bytes >= front, KSQ_ERR_WORKSPACE,
              "m=%zu k=%zu needs %zu bytes of 256-byte aligned workspace for the quantised activations", m, k, front);
  void* act_q = workspace;
  float* act_scale = reinterpret_cast<float*>(static_cast<char*>(workspace) + (m * k + 255) / 256 * 256);
  rc = ksq_fp8_quantize(dtype, act, m, k, KSQ_FP8_PER_TOKEN_DYNAMIC, act_q, act_scale, stream);
  if (rc != KSQ_OK) return rc;
  return ksq_fp8_gemm_ex(dtype, out, act_q, act_scale, m, w_q, w_scale, w_scale_count, m, n, k, epilogue, bias, gemm_ws,
                         gemm_ws_bytes, stream);
}

int ksq_fp8_gemm(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                 const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                 void* workspace, size_t workspace_bytes, void* stream) {
  return ksq_fp8_gemm_ex(out_dtype, out, act_q, act_scale, act_scale_count, w_q, w_scale, w_scale_count, m, n, k,
                         KSQ_EPILOGUE_NONE, nullptr, workspace, workspace_bytes, stream);
}

static int fp8_gemm_impl(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                         const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                         int epilogue, const void* bias, float* row_absmax, void* workspace, size_t workspace_bytes,
                         void* stream) {
  reset_launch_note();
  KSQ_REQUIRE(epilogue >= KSQ_EPILOGUE_NONE && epilogue <= KSQ_EPILOGUE_SILU_MUL, KSQ_ERR_INVALID_ARGUMENT,
              "bad epilogue %d", epilogue);
  KSQ_REQUIRE(epilogue != KSQ_EPILOGUE_BIAS || (bias && (reinterpret_cast<uintptr_t>(bias) & 15) == 0),
              KSQ_ERR_INVALID_ARGUMENT, "the bias epilogue needs a 16-byte aligned bias");
  KSQ_REQUIRE(epilogue != KSQ_EPILOGUE_SILU_MUL || n % 16 == 0, KSQ_ERR_UNSUPPORTED,
              "the SiLU-mul epilogue needs n %% 16 == 0 (got %zu)", n);
  Epilogue epi;
  epi.kind = epilogue;
  epi.bias = bias;
  epi.row_absmax = row_absmax;
  KSQ_REQUIRE(out_dtype == KSQ_F16 || out_dtype == KSQ_BF16 || out_dtype == KSQ_F32, KSQ_ERR_INVALID_ARGUMENT,
              "bad dtype %d", out_dtype);
  KSQ_REQUIRE(out && act_q && w_q, KSQ_ERR_INVALID_ARGUMENT, "null tensor pointer");
  // the reference layer refuses a missing weight scale (KS/layers/nvidia/fp8_matmul_layer.cpp:49-51)
  KSQ_REQUIRE(w_scale != nullptr, KSQ_ERR_INVALID_ARGUMENT, "weight scale is null");
  KSQ_REQUIRE(act_scale != nullptr, KSQ_ERR_INVALID_ARGUMENT, "activation scale is null");
  int rc = check_fp8_shape(n, k);
  if (rc != KSQ_OK) return rc;
  if (m == 0) return KSQ_OK;
  KSQ_REQUIRE(act_scale_count == 1 || act_scale_count == m, KSQ_ERR_INVALID_ARGUMENT,
              "act_scale_count must be 1 or m (got %zu)", act_scale_count);
  KSQ_REQUIRE(w_scale_count == 1 || w_scale_count == n, KSQ_ERR_INVALID_ARGUMENT,
              "w_scale_count must be 1 or n (got %zu)", w_scale_count);
  KSQ_REQUIRE((reinterpret_cast<uintptr_t>(act_q) & 15) == 0 && (reinterpret_cast<uintptr_t>(w_q) & 15) == 0,
              KSQ_ERR_INVALID_ARGUMENT, "act_q and w_q must be 16-byte aligned");
  const DeviceInfo* di = device_info();
  if (!di) return KSQ_ERR_HIP;
  if (fp8_prefill_supported(m, n, k, di->cus) && (reinterpret_cast<uintptr_t>(out) & 15) == 0)
    return fp8_launch_prefill(out_dtype, out, act_q, act_scale, act_scale_count, w_q, w_scale, w_scale_count, m, n, k,
                              workspace, workspace ? workspace_bytes : 0, static_cast<hipStream_t>(stream), epi);
  if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 15) != 0) workspace = nullptr;
  // split-K needs the stream's arrival counters; a stream that got none is planned as if it had no workspace
  if (workspace && !counter_slot_available(static_cast<hipStream_t>(stream))) workspace = nullptr;
  if (m <= 64) {
    const char* e = tuning_env("KSQ_FP8_KSTAT");  // tuning / test switch: 0 sends small m to the streaming kernel
    if (!(e && atoi(e) == 0)) {
      const Fp8KstatPlan kp = fp8_kstat_plan(m, n, k, di->cus, workspace ? workspace_bytes : 0);
      if (kp.ok)
        return fp8_launch_kstat(out_dtype, kp, out, act_q, act_scale, act_scale_count, w_q, w_scale, w_scale_count, m,
                                n, k, workspace, static_cast<hipStream_t>(stream), epi);
    }
  }
  Fp8Plan plan = fp8_plan(m, n, k, di->cus, workspace ? workspace_bytes : 0);
  Fp8Args a{};
  a.epi = epi;
  a.aq = static_cast<const uint8_t*>(act_q);
  a.wq = static_cast<const uint8_t*>(w_q);
  a.a_scale = act_scale;
  a.w_scale = w_scale;
  a.out = out;
  a.partial = static_cast<f32x4*>(workspace);
  a.M = (int)m;
  a.N = (int)n;
  a.K = (int)k;
  a.KB = (int)((k + 127) / 128);
  a.ntiles = (int)((n + 15) / 16);
  a.ksplit = plan.ksplit;
  a.a_scale_per_row = act_scale_count > 1 || (m == 1 && false);
  a.w_scale_per_col = w_scale_count > 1;
  if (act_scale_count == m && m == 1) a.a_scale_per_row = 0;  // one row: index 0 either way
  if (w_scale_count == n && n == 1) a.w_scale_per_col = 0;
  a.counters = nullptr;
  if (plan.ksplit > 1) {
    a.counters = counter_slot_device_ptr(static_cast<hipStream_t>(stream));
    KSQ_REQUIRE(a.counters != nullptr, KSQ_ERR_HIP, "split-K planned for a stream without arrival counters");
  }
  KSQ_REQUIRE(plan.mblocks <= 65535, KSQ_ERR_UNSUPPORTED, "m too large");
  dim3 grid((unsigned)((a.ntiles + 3) / 4), (unsigned)plan.ksplit, (unsigned)plan.mblocks);
  hipStream_t s = static_cast<hipStream_t>(stream);
  note_launch("fp8_stream_kernel<mt=%d> grid=(%u,%u,%u)", plan.MT, grid.x, grid.y, grid.z);
  if (out_dtype == KSQ_F16) launch_fp8_stream<_Float16>(plan.MT, a, grid, s);
  else if (out_dtype == KSQ_F32) launch_fp8_stream<float>(plan.MT, a, grid, s);
  else launch_fp8_stream<__bf16>(plan.MT, a, grid, s);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

int ksq_fp8_gemm_ex(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                    const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                    int epilogue, const void* bias, void* workspace, size_t workspace_bytes, void* stream) {
  return fp8_gemm_impl(out_dtype, out, act_q, act_scale, act_scale_count, w_q, w_scale, w_scale_count, m, n, k, epilogue,
                       bias, nullptr, workspace, workspace_bytes, stream);
}

int ksq_fp8_gemm_rowmax(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                        const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                        int epilogue, const void* bias, float* row_absmax, void* workspace, size_t workspace_bytes,
                        void* stream) {
  KSQ_REQUIRE(row_absmax != nullptr && (reinterpret_cast<uintptr_t>(row_absmax) & 3) == 0, KSQ_ERR_INVALID_ARGUMENT,
              "row_absmax is null or misaligned");
  return fp8_gemm_impl(out_dtype, out, act_q, act_scale, act_scale_count, w_q, w_scale, w_scale_count, m, n, k, epilogue,
                       bias, row_absmax, workspace, workspace_bytes, stream);
}

int ksq_fill_zero_f32(float* p, size_t count, void* stream) {
  KSQ_REQUIRE(p != nullptr || count == 0, KSQ_ERR_INVALID_ARGUMENT, "null pointer");
  if (count == 0) return KSQ_OK;
  KSQ_REQUIRE(count < (1ull << 31), KSQ_ERR_UNSUPPORTED, "count too large");
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     p, (int)count);
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

// scale[r] = max(row_absmax[r] / 448, floor), then the quantisation pass of the per-token mode on its own
int ksq_fp8_quantize_rows_from_absmax(int dtype, const void* act, size_t m, size_t k, const float* row_absmax,
                                      void* act_q, float* act_scale, void* stream) {
  KSQ_REQUIRE(dtype == KSQ_F16 || dtype == KSQ_BF16, KSQ_ERR_INVALID_ARGUMENT, "bad dtype %d", dtype);
  KSQ_REQUIRE(act && act_q && act_scale && row_absmax, KSQ_ERR_INVALID_ARGUMENT, "null tensor pointer");
  if (m == 0 || k == 0) return KSQ_OK;
  KSQ_REQUIRE(m < (1ull << 31), KSQ_ERR_UNSUPPORTED, "m=%zu too large", m);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t* x = static_cast<const uint16_t*>(act);
  uint8_t* q = static_cast<uint8_t*>(act_q);
  const bool vec = k % 8 == 0 && (reinterpret_cast<uintptr_t>(act) & 15) == 0 && (reinterpret_cast<uintptr_t>(act_q) & 7) == 0;
  const dim3 grid((unsigned)m), block(256);
  if (dtype == KSQ_F16) {
    if (vec) hipLaunchKernelGGL((quantize_rows_from_absmax_kernel<_Float16, true>), grid, block, 0, s, x, k, row_absmax, q, act_scale);
    else hipLaunchKernelGGL((quantize_rows_from_absmax_kernel<_Float16, false>), grid, block, 0, s, x, k, row_absmax, q, act_scale);
  } else {
    if (vec) hipLaunchKernelGGL((quantize_rows_from_absmax_kernel<__bf16, true>), grid, block, 0, s, x, k, row_absmax, q, act_scale);
    else hipLaunchKernelGGL((quantize_rows_from_absmax_kernel<__bf16, false>), grid, block, 0, s, x, k, row_absmax, q, act_scale);
  }
  KSQ_HIP_TRY(hipGetLastError());
  return KSQ_OK;
}

}  // extern "C"
