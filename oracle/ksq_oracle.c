/*
 * ksq_oracle.c -- CPU restatement of KsanaLLM's quantized linear-layer path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls this file: it is
 * the checker that the parity tests, the smoke test and the bench's host-core baseline leg use.
 *
 * Every function cites the reference code it restates (paths relative to the KsanaLLM tree;
 * KS = src/ksana_llm, LK = 3rdparty/LLM_kernels/csrc/kernels/nvidia, LU = 3rdparty/LLM_kernels/csrc/utils/nvidia).
 * The reference path is CUDA on CUTLASS/cuBLASLt and cannot be compiled here, so nothing below was
 * checked by running it.  What pins each function instead:
 *   - layout unpackers: brute-force bit extraction written independently in the tests, pack/unpack
 *     identities, the AutoAWQ order / reverse-order composition being the identity;
 *   - dequantize-then-GEMM: integer special cases that are exact in fp32, one-hot activations that
 *     return dequantized rows exactly, an fp64-accumulated GEMM on small shapes, numpy matmul;
 *   - e4m3 codec: all 256 codes against the OCP closed form and against torch.float8_e4m3fn casts;
 *   - fp8 scale / quantize / rescale: the closed forms the reference's own unit test asserts
 *     (LU/utils_test.cu:49-56, 93-99, 136-141).
 * Parity unpinned (no reference-side vector exists and none can be produced here): the fp16
 * two-rounding dequantisation order inside the CUTLASS warp dequantizer, the fp16 accumulation order of
 * the batched GEMV, and the accumulation mode of cuBLASLt's FP8 matmul.  The tolerances of the parity
 * tests (max relative error 1e-2, mean absolute error <= 2e-3 x RMS) are what stand in for them.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { ORC_F16 = 0, ORC_BF16 = 1, ORC_F32 = 2 };

/* ---------------------------------------------------------------- scalar formats */

static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static float half_to_float(uint16_t h) {
  uint32_t s = (uint32_t)(h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1Fu;
  uint32_t m = h & 0x3FFu;
  if (e == 0) {
    if (m == 0) return u2f(s);
    float v = ldexpf((float)m, -24); /* subnormal: m * 2^-24 */
    return (s ? -v : v);
  }
  if (e == 31) return u2f(s | 0x7F800000u | (m << 13));
  return u2f(s | ((e + 112u) << 23) | (m << 13));
}

/* round-to-nearest-even float -> half, IEEE semantics (overflow -> inf) */
static uint16_t float_to_half(float f) {
  uint32_t x = f2u(f);
  uint16_t s = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7FFFFFFFu;
  if (ax >= 0x7F800000u) return (uint16_t)(s | 0x7C00u | (ax > 0x7F800000u ? 0x200u : 0u));
  if (ax >= 0x477FF000u) return (uint16_t)(s | 0x7C00u); /* >= 65520 rounds to inf */
  if (ax < 0x33000001u) return s;                       /* <= 2^-25 rounds to zero */
  int e = (int)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7FFFFFu) | 0x800000u;
  int shift = (e < -14) ? (13 + (-14 - e)) : 13; /* bits dropped from the 24-bit significand */
  uint32_t keep = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (keep & 1u))) keep++;
  if (e < -14) return (uint16_t)(s | keep); /* subnormal (carry into exponent is natural) */
  uint32_t he = (uint32_t)(e + 15);
  uint32_t out = (he << 10) + (keep - 0x400u); /* keep in [0x400,0x800]; 0x800 carries */
  return (uint16_t)(s | out);
}

static float bf16_to_float(uint16_t b) { return u2f((uint32_t)b << 16); }

static uint16_t float_to_bf16(float f) {
  uint32_t x = f2u(f);
  if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x40u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7FFFu + lsb;
  return (uint16_t)(x >> 16);
}

static inline float load_elem(const void* p, size_t i, int dtype) {
  switch (dtype) {
    case ORC_F16: return half_to_float(((const uint16_t*)p)[i]);
    case ORC_BF16: return bf16_to_float(((const uint16_t*)p)[i]);
    default: return ((const float*)p)[i];
  }
}

static inline void store_elem(void* p, size_t i, int dtype, float v) {
  switch (dtype) {
    case ORC_F16: ((uint16_t*)p)[i] = float_to_half(v); break;
    case ORC_BF16: ((uint16_t*)p)[i] = float_to_bf16(v); break;
    default: ((float*)p)[i] = v; break;
  }
}

void orc_to_f32(const void* src, int dtype, size_t n, float* dst) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) dst[i] = load_elem(src, i, dtype);
}

void orc_from_f32(const float* src, int dtype, size_t n, void* dst) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) store_elem(dst, i, dtype, src[i]);
}

/* ---------------------------------------------------------------- checkpoint layouts */

/* GPTQ qweight int32 [K/8, N] -> unsigned nibbles u[K, N] in [0,15].
 * KS/models/quant/quant_weight.cpp:291-300 (CutlassUnpackGPTQ): transposes, views the int32 as bytes,
 * takes byte%16 then byte/16, transposes back; i.e. element k = 8r + j sits in bits 4j..4j+3 of row r. */
void orc_gptq_unpack(const int32_t* qweight, size_t K, size_t N, uint8_t* u) {
#pragma omp parallel for schedule(static)
  for (size_t k = 0; k < K; ++k)
    for (size_t n = 0; n < N; ++n)
      u[k * N + n] = (uint8_t)(((uint32_t)qweight[(k >> 3) * N + n] >> (4 * (k & 7))) & 0xFu);
}

void orc_gptq_pack(const uint8_t* u, size_t K, size_t N, int32_t* qweight) {
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < K / 8; ++r)
    for (size_t n = 0; n < N; ++n) {
      uint32_t w = 0;
      for (size_t j = 0; j < 8; ++j) w |= (uint32_t)(u[(8 * r + j) * N + n] & 0xFu) << (4 * j);
      qweight[r * N + n] = (int32_t)w;
    }
}

/* AWQ int32 [R, N/8] -> unsigned nibbles [R, N]; serves qweight (R = K) and qzeros (R = K/g).
 * KS/models/quant/quant_weight.cpp:262-287: CutlassUnpackQWeight shifts each word by 0,4,..,28 (slot j =
 * bits 4j..4j+3), CutlassGetReverseOrder then gathers slots in the order [0,4,1,5,2,6,3,7], so logical
 * column 8c + i is read from slot REV[i]. */
static const int AWQ_REV[8] = {0, 4, 1, 5, 2, 6, 3, 7};

void orc_awq_unpack(const int32_t* q, size_t R, size_t N, uint8_t* u) {
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < R; ++r)
    for (size_t c = 0; c < N / 8; ++c) {
      uint32_t w = (uint32_t)q[r * (N / 8) + c];
      for (int i = 0; i < 8; ++i) u[r * N + 8 * c + i] = (uint8_t)((w >> (4 * AWQ_REV[i])) & 0xFu);
    }
}

/* AutoAWQ's packing order (awq/utils/packing_utils.py, AWQ_ORDER = [0,2,4,6,1,3,5,7]; the reference cites
 * it at quant_weight.cpp:260): slot j of a word holds logical column 8c + ORDER[j]. */
static const int AWQ_ORDER[8] = {0, 2, 4, 6, 1, 3, 5, 7};

void orc_awq_pack(const uint8_t* u, size_t R, size_t N, int32_t* q) {
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < R; ++r)
    for (size_t c = 0; c < N / 8; ++c) {
      uint32_t w = 0;
      for (int j = 0; j < 8; ++j) w |= (uint32_t)(u[r * N + 8 * c + AWQ_ORDER[j]] & 0xFu) << (4 * j);
      q[r * (N / 8) + c] = (int32_t)w;
    }
}

/* ksana canonical row-major int4: int8 [K, N/2], byte = (q[k,2b] & 0xF) | (q[k,2b+1] << 4), q = u - 8.
 * KS/models/quant/quant_weight.cpp:249-251 (subtract 2^(bits-1)) and :304-328 (CutlassPackInt8ToPackedInt4). */
void orc_rowmajor_pack(const uint8_t* u, size_t K, size_t N, uint8_t* packed) {
#pragma omp parallel for schedule(static)
  for (size_t k = 0; k < K; ++k)
    for (size_t b = 0; b < N / 2; ++b) {
      int q0 = (int)u[k * N + 2 * b] - 8, q1 = (int)u[k * N + 2 * b + 1] - 8;
      packed[k * (N / 2) + b] = (uint8_t)((q0 & 0xF) | ((q1 & 0xF) << 4));
    }
}

void orc_rowmajor_unpack(const uint8_t* packed, size_t K, size_t N, uint8_t* u) {
#pragma omp parallel for schedule(static)
  for (size_t k = 0; k < K; ++k)
    for (size_t b = 0; b < N / 2; ++b) {
      uint8_t byte = packed[k * (N / 2) + b];
      int q0 = (int)(byte & 0xF), q1 = (int)(byte >> 4);
      if (q0 >= 8) q0 -= 16; /* two's-complement nibble */
      if (q1 >= 8) q1 -= 16;
      u[k * N + 2 * b] = (uint8_t)(q0 + 8);
      u[k * N + 2 * b + 1] = (uint8_t)(q1 + 8);
    }
}

/* AWQ zero points at the layer boundary: zeros = scales * (8 - qzeros), evaluated in the scale dtype.
 * KS/models/quant/quant_weight.cpp:530-536 (qzeros were cast to half at :253-256, so (8 - z) is exact and
 * the product is rounded once). */
void orc_awq_additive_zeros(const void* scales, int dtype, const uint8_t* z, size_t G, size_t N, void* zeros) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < G * N; ++i) store_elem(zeros, i, dtype, load_elem(scales, i, dtype) * (8.0f - (float)z[i]));
}

/* ---------------------------------------------------------------- dequantize-then-GEMM */

/* w[k,n] = s[k/g,n] * (u[k,n] - z[k/g,n]) in fp32; z == NULL means the symmetric zero 8 (GPTQ: qzeros are
 * dropped, quant_weight.cpp:73-75).  AWQ semantics: quant_weight.cpp:530-531.  Group row = k / g:
 * LK/cutlass_extensions/transform/threadblock/fine_grained_scale_zero_iterator.h:152-153. */
void orc_dequant(const uint8_t* u, const void* scales, int sdtype, const uint8_t* z, size_t K, size_t N, size_t g,
                 float* w) {
#pragma omp parallel for schedule(static)
  for (size_t k = 0; k < K; ++k) {
    size_t gr = k / g;
    for (size_t n = 0; n < N; ++n) {
      float s = load_elem(scales, gr * N + n, sdtype);
      float zz = z ? (float)z[gr * N + n] : 8.0f;
      w[k * N + n] = s * ((float)u[k * N + n] - zz);
    }
  }
}

/* The form the reference kernels evaluate: w = (u - 8) * s + zeros', zeros' additive in the scale dtype
 * (NULL for GPTQ).  LK/cutlass_extensions/interleaved_numeric_conversion.h:198-265,301-354 (nibble -> q = u - 8)
 * and gemm/warp/mma_tensorop_dequantizer.h:206-245,368-394 (scale, then add zero).  Evaluated here in fp32. */
void orc_dequant_additive(const uint8_t* u, const void* scales, int sdtype, const void* zeros_additive, size_t K,
                          size_t N, size_t g, float* w) {
#pragma omp parallel for schedule(static)
  for (size_t k = 0; k < K; ++k) {
    size_t gr = k / g;
    for (size_t n = 0; n < N; ++n) {
      float s = load_elem(scales, gr * N + n, sdtype);
      float za = zeros_additive ? load_elem(zeros_additive, gr * N + n, sdtype) : 0.0f;
      w[k * N + n] = ((float)u[k * N + n] - 8.0f) * s + za;
    }
  }
}

/* out[m,n] = sum_k a[m,k] * w[k,n], fp32 accumulation in ascending k, cache-blocked, OpenMP over N blocks.
 * The GEMM contract of LK/asymmetric_gemm/asymmetric_gemm_wrapper.cu:53-77 (alpha = 1, no bias, fp32
 * accumulators per LK/cutlass_extensions/gemm/kernel/default_fpA_intB_traits.h:121-128). */
void orc_gemm_f32(const float* a, const float* w, size_t M, size_t N, size_t K, float* out) {
  const size_t NB = 256, KB = 256, MB = 16;
  size_t nblocks = (N + NB - 1) / NB;
#pragma omp parallel for schedule(dynamic, 1)
  for (size_t nb = 0; nb < nblocks; ++nb) {
    size_t n0 = nb * NB, n1 = n0 + NB < N ? n0 + NB : N;
    size_t nw = n1 - n0;
    float acc[16 * 256];
    for (size_t m0 = 0; m0 < M; m0 += MB) {
      size_t m1 = m0 + MB < M ? m0 + MB : M;
      for (size_t i = 0; i < (m1 - m0) * NB; ++i) acc[i] = 0.0f;
      for (size_t k0 = 0; k0 < K; k0 += KB) {
        size_t k1 = k0 + KB < K ? k0 + KB : K;
        for (size_t m = m0; m < m1; ++m) {
          float* accrow = acc + (m - m0) * NB;
          for (size_t k = k0; k < k1; ++k) {
            float av = a[m * K + k];
            const float* wrow = w + k * N + n0;
            for (size_t j = 0; j < nw; ++j) accrow[j] += av * wrow[j];
          }
        }
      }
      for (size_t m = m0; m < m1; ++m)
        for (size_t j = 0; j < nw; ++j) out[m * N + n0 + j] = acc[(m - m0) * NB + j];
    }
  }
}

/* Same product with fp64 accumulation; bounds the fp32 oracle's own rounding on small shapes. */
void orc_gemm_f64acc(const float* a, const float* w, size_t M, size_t N, size_t K, double* out) {
#pragma omp parallel for schedule(static)
  for (size_t m = 0; m < M; ++m) {
    double* row = out + m * N;
    for (size_t n = 0; n < N; ++n) row[n] = 0.0;
    for (size_t k = 0; k < K; ++k) {
      double av = (double)a[m * K + k];
      const float* wrow = w + k * N;
      for (size_t n = 0; n < N; ++n) row[n] += av * (double)wrow[n];
    }
  }
}

/* Whole W4A16 layer forward in one call: unpacked nibbles in, fp32 result out.  This is also the host-core
 * baseline the bench times (dequantize to fp32 + blocked GEMM).  `w_scratch` must hold K*N floats,
 * `a_scratch` M*K floats. */
void orc_w4a16_forward(const void* act, int adtype, const uint8_t* u, const void* scales, int sdtype,
                       const uint8_t* z, size_t M, size_t N, size_t K, size_t g, float* w_scratch, float* a_scratch,
                       float* out) {
  orc_dequant(u, scales, sdtype, z, K, N, g, w_scratch);
  orc_to_f32(act, adtype, M * K, a_scratch);
  orc_gemm_f32(a_scratch, w_scratch, M, N, K, out);
}

/* ---------------------------------------------------------------- FP8 e4m3 (OCP "fn": bias 7, max 448, no inf) */

float orc_e4m3_decode(uint8_t c) {
  int s = c >> 7, e = (c >> 3) & 0xF, m = c & 7;
  float v;
  if (e == 15 && m == 7) return u2f(0x7FC00000u | ((uint32_t)s << 31));
  if (e == 0) v = ldexpf((float)m, -9);
  else v = ldexpf((float)(8 + m), e - 10);
  return s ? -v : v;
}

/* Round-to-nearest-even, saturating to +-448 (what a CUDA __nv_fp8_e4m3 construction from float does,
 * used at LU/cuda_fp8_utils.cu:27-35).  NaN -> 0x7F | sign. */
uint8_t orc_e4m3_encode(float x) {
  uint32_t bits = f2u(x);
  uint8_t s = (uint8_t)((bits >> 24) & 0x80u);
  float ax = fabsf(x);
  if (ax != ax) return (uint8_t)(s | 0x7Fu);
  if (ax >= 448.0f) return (uint8_t)(s | 0x7Eu); /* 448 <= ax: saturate (values in (448,464) would round to 448 anyway) */
  if (ax < 0.015625f) {                           /* below 2^-6: subnormal grid of 2^-9 */
    float q = nearbyintf(ax * 512.0f);            /* exact scaling, RNE; q == 8 lands on code 0x08 = 2^-6 */
    return (uint8_t)(s | (uint8_t)q);
  }
  int e;
  float fr = frexpf(ax, &e);            /* ax = fr * 2^e, fr in [0.5,1) */
  float q = nearbyintf(fr * 16.0f);     /* 4 significant bits: q in [8,16] */
  int ee = e - 1;                       /* ax = (q/8) * 2^ee */
  if (q >= 16.0f) { q = 8.0f; ee += 1; }
  int code = ((ee + 7) << 3) | ((int)q - 8);
  if (code > 0x7E) code = 0x7E;
  return (uint8_t)(s | code);
}

/* scale[c] = max(absmax(x[c,:]) / 448, 1/(448*512)).  LU/cuda_fp8_utils.cu:85-116, constants
 * LU/cuda_fp8_utils.h:42-43 (FP8_E4M3_MIN_SCALE = 1.0f / 448 / 512). */
void orc_fp8_compute_scale(const void* x, int dtype, size_t num_channels, size_t channel_size, float* scale) {
  const float min_scale = 1.0f / 448.0f / 512.0f;
#pragma omp parallel for schedule(static)
  for (size_t c = 0; c < num_channels; ++c) {
    float mx = 0.0f;
    for (size_t i = 0; i < channel_size; ++i) mx = fmaxf(mx, fabsf(load_elem(x, c * channel_size + i, dtype)));
    scale[c] = fmaxf(mx / 448.0f, min_scale);
  }
}

/* q = e4m3(min(max(x / scale[c], -448), 448)), true division.  LU/cuda_fp8_utils.cu:27-35. */
void orc_fp8_quantize(const void* x, int dtype, const float* scale, size_t num_channels, size_t channel_size,
                      uint8_t* q) {
#pragma omp parallel for schedule(static)
  for (size_t c = 0; c < num_channels; ++c)
    for (size_t i = 0; i < channel_size; ++i) {
      float v = load_elem(x, c * channel_size + i, dtype) / scale[c];
      v = fminf(fmaxf(v, -448.0f), 448.0f);
      q[c * channel_size + i] = orc_e4m3_encode(v);
    }
}

/* q' = e4m3(float(q) * (s_in / s_out)).  LU/cuda_fp8_utils.cu:140-147 (the ratio is formed first). */
void orc_fp8_rescale(const uint8_t* q, size_t n, float s_in, float s_out, uint8_t* out) {
  float r = s_in / s_out;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) out[i] = orc_e4m3_encode(orc_e4m3_decode(q[i]) * r);
}

/* out[m,n] = (acc * w_scale[n or 0]) * a_scale[m or 0], acc = sum_k aq[m,k] * wq[n,k] in fp32 (products of two
 * e4m3 values are exact in fp32).  Weight is [N,K], K contiguous: KS/layers/nvidia/fp8_matmul_layer.cpp:37-39.
 * Per-tensor scalar scales are what the reference layer passes (kernel_wrapper.cpp:1033-1041); the per-row x
 * per-column order follows LK/asymmetric_gemm/fp8_rowwise_gemm/fp8_rowwise_gemm_kernel_template_sm90.h:119-131. */
void orc_fp8_gemm(const uint8_t* aq, const float* a_scale, size_t a_scale_count, const uint8_t* wq,
                  const float* w_scale, size_t w_scale_count, size_t M, size_t N, size_t K, float* out) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = orc_e4m3_decode((uint8_t)i);
  float* af = (float*)malloc(sizeof(float) * M * K);
  for (size_t i = 0; i < M * K; ++i) af[i] = lut[aq[i]];
#pragma omp parallel
  {
    float* wrow = (float*)malloc(sizeof(float) * K);
#pragma omp for schedule(static)
    for (size_t n = 0; n < N; ++n) {
      for (size_t k = 0; k < K; ++k) wrow[k] = lut[wq[n * K + k]];
      float ws = w_scale[w_scale_count > 1 ? n : 0];
      for (size_t m = 0; m < M; ++m) {
        const float* arow = af + m * K;
        float acc = 0.0f;
        for (size_t k = 0; k < K; ++k) acc += arow[k] * wrow[k];
        out[m * N + n] = (acc * ws) * a_scale[a_scale_count > 1 ? m : 0];
      }
    }
    free(wrow);
  }
  free(af);
}

/* On-the-fly FP8 weight conversion: [K,N] T -> [N,K] e4m3 with one scale for the whole tensor.
 * KS/models/quant/quant_weight.cpp:685-726 (transpose :701-708, scale + quantize :716-718). */
void orc_fp8_convert_weight(const void* w_kn, int dtype, size_t K, size_t N, uint8_t* wq_nk, float* scale) {
  float* t = (float*)malloc(sizeof(float) * K * N);
  for (size_t k = 0; k < K; ++k)
    for (size_t n = 0; n < N; ++n) t[n * K + k] = load_elem(w_kn, k * N + n, dtype);
  /* the reference quantizes the T-typed transposed tensor; values are unchanged by the transpose */
  orc_fp8_compute_scale(t, ORC_F32, 1, K * N, scale);
  orc_fp8_quantize(t, ORC_F32, scale, 1, K * N, wq_nk);
  free(t);
}

/* The same with one scale per output channel (column of the [K,N] source): the per-channel extension of
 * KS/models/quant/quant_weight.cpp:685-726 that the row-wise FP8 GEMM
 * (LK/asymmetric_gemm/fp8_rowwise_gemm/fp8_rowwise_gemm_kernel_template_sm90.h:119-131) consumes. */
void orc_fp8_convert_weight_per_channel(const void* w_kn, int dtype, size_t K, size_t N, uint8_t* wq_nk, float* scale) {
  float* t = (float*)malloc(sizeof(float) * K * N);
  for (size_t k = 0; k < K; ++k)
    for (size_t n = 0; n < N; ++n) t[n * K + k] = load_elem(w_kn, k * N + n, dtype);
  orc_fp8_compute_scale(t, ORC_F32, N, K, scale);
  orc_fp8_quantize(t, ORC_F32, scale, N, K, wq_nk);
  free(t);
}

/* ---------------------------------------------------------------- CUTLASS weight preprocessor (F1 input layout)
 *
 * preprocess_weights_for_mixed_gemm for QuantType::W4_A16, shape {K, N}
 * (LK/asymmetric_gemm/cutlass_preprocessors.cpp:466-508).  On sm80..sm89 the layout details are
 * ColumnMajorTileInterleave<64, 4> with the LDSM row permutation
 * (LK/cutlass_extensions/gemm/kernel/mixed_gemm_B_layout.h:106-120: ThreadblockK = 128*8/16 = 64,
 * ColumnsInterleaved = (128*8/4)/64 = 4, OpMultiplyAddDequantizeInterleavedBToA), so all four steps run; on sm90
 * (:130-136: ColumnMajor, OpMultiplyAdd) only the transpose runs and the bias step is skipped (:497-499).
 * Each step below is a separate pass over a whole buffer, as in the reference, on nibble arrays for clarity:
 * in[k][n] signed nibble as stored (two's complement), row-major bytes [K][N/2], low nibble = even n.
 *
 * Pinned by: every step being a bijection on nibble positions (the tests check that the multiset of values
 * survives and that distinct inputs give distinct outputs), by the product's repack, which reads this layout
 * through a closed-form inverse written independently of these loops, reproducing the repack of the
 * row-major source bit for bit, and by bit-plane probes (a tensor with a single marked nibble lands where the
 * closed form says).  The reference itself cannot be run here (CUTLASS headers and the CUDA runtime are absent).
 */
static inline uint8_t get_nib(const uint8_t* b, size_t i) { return (i & 1) ? (uint8_t)(b[i >> 1] >> 4) : (uint8_t)(b[i >> 1] & 0xF); }
static inline void set_nib(uint8_t* b, size_t i, uint8_t v) {
  if (i & 1) b[i >> 1] = (uint8_t)((b[i >> 1] & 0x0F) | (v << 4));
  else b[i >> 1] = (uint8_t)((b[i >> 1] & 0xF0) | (v & 0xF));
}

/* :129-141 the map, :143-197 the pass: inside every group of 32 rows, row r of the output is row map[r] of the
 * input (whole rows move; the reference moves them 32 bits at a time) */
void orc_cutlass_permute_rows(const uint8_t* in, size_t K, size_t N, uint8_t* out) {
  static const int map[32] = {0, 1, 8,  9,  16, 17, 24, 25, 2, 3, 10, 11, 18, 19, 26, 27,
                              4, 5, 12, 13, 20, 21, 28, 29, 6, 7, 14, 15, 22, 23, 30, 31};
  const size_t row_bytes = N / 2;
  for (size_t base = 0; base < K; base += 32)
    for (size_t r = 0; r < 32; ++r) memcpy(out + (base + r) * row_bytes, in + (base + (size_t)map[r]) * row_bytes, row_bytes);
}

/* :203-323 sub-byte transpose: out is [N][K/2] bytes, nibble k of row n = in nibble n of row k */
void orc_cutlass_transpose(const uint8_t* in, size_t K, size_t N, uint8_t* out) {
  for (size_t k = 0; k < K; ++k)
    for (size_t n = 0; n < N; ++n) set_nib(out, n * K + k, get_nib(in, k * N + n));
}

/* :426-464 on 32-bit registers of the column-major tensor ([N][K/8] registers): rows_per_tile = 64 ->
 * 8 registers per tile, interleave = 4 columns */
void orc_cutlass_interleave_columns(const uint32_t* in, size_t K, size_t N, uint32_t* out) {
  const size_t vec_rows = K / 8, per_tile = 64 / 8, il = 4;
  for (size_t col = 0; col < N; ++col) {
    const size_t wcol = col / il;
    for (size_t base = 0; base < vec_rows; base += per_tile)
      for (size_t v = base; v < base + per_tile && v < vec_rows; ++v) {
        const size_t wv = il * base + per_tile * (col % il) + v % per_tile;
        out[wcol * vec_rows * il + wv] = in[col * vec_rows + v];
      }
  }
}

/* :352-401 every nibble + 8 (signed -> unsigned), then inside every 32-bit register destination slot d takes
 * source slot 2d (d < 4) or 2(d - 4) + 1 */
void orc_cutlass_bias_and_interleave(uint32_t* regs, size_t count) {
  for (size_t i = 0; i < count; ++i) {
    const uint32_t r = regs[i];
    uint32_t biased = 0, t = 0;
    for (int e = 0; e < 8; ++e) {
      int v = (int)((r >> (4 * e)) & 0xF);
      if (v >= 8) v -= 16; /* sign extension of the stored nibble */
      biased |= (uint32_t)(v + 8) << (4 * e);
    }
    for (int d = 0; d < 8; ++d) {
      const int src = d < 4 ? 2 * d : 2 * (d - 4) + 1;
      t |= ((biased >> (4 * src)) & 0xFu) << (4 * d);
    }
    regs[i] = t;
  }
}

/* rowmajor: [K][N/2] bytes; out: K*N/2 bytes.  arch 80: all four steps; arch 90: the transpose only. */
void orc_cutlass_preprocess(const uint8_t* rowmajor, size_t K, size_t N, int arch, uint8_t* out) {
  const size_t bytes = K * N / 2;
  uint8_t* a = (uint8_t*)malloc(bytes);
  uint8_t* b = (uint8_t*)malloc(bytes);
  memcpy(a, rowmajor, bytes);
  if (arch < 90) {
    orc_cutlass_permute_rows(a, K, N, b);
    uint8_t* t = a; a = b; b = t;
  }
  memset(b, 0, bytes);
  orc_cutlass_transpose(a, K, N, b);
  { uint8_t* t = a; a = b; b = t; }
  if (arch < 90) {
    orc_cutlass_interleave_columns((const uint32_t*)a, K, N, (uint32_t*)b);
    uint8_t* t = a; a = b; b = t;
    orc_cutlass_bias_and_interleave((uint32_t*)a, bytes / 4);
  }
  memcpy(out, a, bytes);
  free(a);
  free(b);
}

/* ---------------------------------------------------------------- Marlin weight layout (F1 input layout)
 *
 * gptq_marlin_repack_kernel<256, 4, false> (LK/gptq_marlin/gptq_marlin_repack.cu:31-233) and
 * awq_marlin_repack_kernel<256, 4> (LK/gptq_marlin/awq_marlin_repack.cu:30-170) with the CUDA launch geometry
 * written out as loops: tiles of tile_k_size = 16 by tile_n_size = 64 (marlin_params.h:44-45), four warps of 32
 * threads per tile, one output word per thread.  Pinned by the formulation published with the format
 * (vLLM's marlin_permute_weights / get_weight_perm, which the reference cites at quant_weight.cpp:348), written
 * out in the tests with numpy, and by the library's closed-form inverse reproducing the plain repack.
 */
static const int MARLIN_TC_OFFSETS[4] = {0, 1, 8, 9};
static const int MARLIN_PACK_IDX[8] = {0, 2, 4, 6, 1, 3, 5, 7};

static void marlin_store(const uint32_t vals[8], size_t k_tile, size_t n_tile, size_t n_tiles, int th_id, int warp_id,
                         uint32_t* out) {
  uint32_t res = 0;
  for (int i = 0; i < 8; ++i) res |= vals[MARLIN_PACK_IDX[i]] << (i * 4);
  out[(k_tile * n_tiles + n_tile) * 128 + (size_t)th_id * 4 + (size_t)warp_id] = res; /* :199-206 */
}

/* qweight: GPTQ int32 [K/8][N] */
void orc_marlin_repack_gptq(const uint32_t* qweight, size_t K, size_t N, uint32_t* out) {
  const size_t k_tiles = K / 16, n_tiles = N / 64;
  for (size_t k_tile = 0; k_tile < k_tiles; ++k_tile)
    for (size_t n_tile = 0; n_tile < n_tiles; ++n_tile)
      for (int warp_id = 0; warp_id < 4; ++warp_id)
        for (int th_id = 0; th_id < 32; ++th_id) {
          const int tc_col = th_id / 4, tc_row = (th_id % 4) * 2; /* :142-143 */
          const size_t cur_n = n_tile * 64 + (size_t)warp_id * 16 + (size_t)tc_col;
          uint32_t vals[8];
          for (int i = 0; i < 4; ++i) { /* :185-193: the tile's two packed rows, element cur_elem of the tile */
            const size_t k = k_tile * 16 + (size_t)(tc_row + MARLIN_TC_OFFSETS[i]);
            vals[i] = (qweight[(k / 8) * N + cur_n] >> (4 * (k % 8))) & 0xF;
            vals[4 + i] = (qweight[(k / 8) * N + cur_n + 8] >> (4 * (k % 8))) & 0xF;
          }
          marlin_store(vals, k_tile, n_tile, n_tiles, th_id, warp_id, out);
        }
}

/* qweight: AWQ int32 [K][N/8], AutoAWQ nibble order */
void orc_marlin_repack_awq(const uint32_t* qweight, size_t K, size_t N, uint32_t* out) {
  static const int undo_pack[8] = {0, 4, 1, 5, 2, 6, 3, 7}; /* awq_marlin_repack.cu:119-121 */
  const size_t k_tiles = K / 16, n_tiles = N / 64;
  for (size_t k_tile = 0; k_tile < k_tiles; ++k_tile)
    for (size_t n_tile = 0; n_tile < n_tiles; ++n_tile)
      for (int warp_id = 0; warp_id < 4; ++warp_id)
        for (int th_id = 0; th_id < 32; ++th_id) {
          const int tc_col = th_id / 4, tc_row = (th_id % 4) * 2;
          const int cur_n = warp_id * 16 + tc_col; /* inside the tile */
          const size_t packed = (n_tile * 64 + (size_t)cur_n) / 8;
          const int pos = undo_pack[cur_n % 8];
          uint32_t vals[8];
          for (int i = 0; i < 4; ++i) { /* :129-138 */
            const size_t k = k_tile * 16 + (size_t)(tc_row + MARLIN_TC_OFFSETS[i]);
            vals[i] = (qweight[k * (N / 8) + packed] >> (4 * pos)) & 0xF;
            vals[4 + i] = (qweight[k * (N / 8) + packed + 1] >> (4 * pos)) & 0xF;
          }
          marlin_store(vals, k_tile, n_tile, n_tiles, th_id, warp_id, out);
        }
}

/* ---------------------------------------------------------------- desc_act (F3)
 * perm = stable argsort of g_idx (MarlinSortGIdx, KS/models/quant/quant_weight.cpp:455-460: torch::argsort with
 * stable = true); the activations' columns are gathered through it (permute_cols_kernel,
 * LK/gptq_marlin/gptq_marlin.cu:380-384) and the weight rows stored in the same order.  Insertion sort: stable
 * by construction, written independently of the product's counting sort. */
void orc_act_order_perm(const int32_t* g_idx, size_t K, int32_t* perm) {
  for (size_t i = 0; i < K; ++i) {
    size_t j = i;
    while (j > 0 && g_idx[perm[j - 1]] > g_idx[i]) {
      perm[j] = perm[j - 1];
      --j;
    }
    perm[j] = (int32_t)i;
  }
}

/* ---------------------------------------------------------------- epilogues (F2), on the fp32 GEMM result
 * SiLU-mul: KS/models/common/common_model.cpp:540-547 runs gate and up GEMMs and then silu(gate) * up
 * (LK/activation: silu(x) = x / (1 + exp(-x))); here gate = acc[:, :H], up = acc[:, H:] of one [M, 2H] result.
 * Bias: out + bias[n] (common_model.cpp:456-459). */
void orc_silu_mul(const float* acc, size_t M, size_t H, float* out) {
  for (size_t m = 0; m < M; ++m)
    for (size_t h = 0; h < H; ++h) {
      const double g = acc[m * 2 * H + h], u = acc[m * 2 * H + H + h];
      out[m * H + h] = (float)(g / (1.0 + exp(-g)) * u);
    }
}

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
