/*
 * ksq.h -- C ABI of the MI355X (gfx950) quantized linear-layer path.
 *
 * One shared library, libksq.so, exports everything below with C linkage.  All pointers are device pointers
 * unless the parameter name ends in `_host`; `stream` is a hipStream_t passed as void* (NULL = the default
 * stream).  Every function returns KSQ_OK (0) or a negative ksq_status; no exception crosses this boundary and
 * ksq_last_error_string() gives the reason for the last failure on the calling thread.  Nothing here allocates
 * device memory, synchronises the stream, or branches on device data, so the GEMM entry points are safe to call
 * from a serving loop and under HIP graph capture.
 *
 * Citations name the interface of KsanaLLM that each entry point replaces
 * (KS = src/ksana_llm, LK = 3rdparty/LLM_kernels/csrc/kernels/nvidia, LU = 3rdparty/LLM_kernels/csrc/utils/nvidia).
 */
#ifndef KSQ_H_
#define KSQ_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum ksq_status {
  KSQ_OK = 0,
  KSQ_ERR_INVALID_ARGUMENT = -1, /* null pointer, zero size, bad enum */
  KSQ_ERR_UNSUPPORTED = -2,      /* shape / group size / layout the kernels do not cover */
  KSQ_ERR_WORKSPACE = -3,        /* workspace missing or too small where it is mandatory */
  KSQ_ERR_HIP = -4               /* a HIP runtime call or kernel launch failed */
} ksq_status;

/* Activation / output element type (the reference instantiates its layers for float, half and __nv_bfloat16:
 * KS/layers/nvidia/group_matmul_layer.cpp:171-175, fp8_matmul_layer.cpp:69-73).
 * KSQ_F32 is accepted by the FP8 entry points that take activations or produce results -- ksq_fp8_quantize,
 * ksq_fp8_gemm / _ex / _rowmax (out_dtype), ksq_fp8_gemm_dynamic (both) -- which is where the reference has an fp32
 * path (Fp8E4m3Quantize<float>, Fp8QuantizedMatMul<float>: KS/kernels/nvidia/kernel_wrapper.cpp:1026, 1043); a
 * bias row is then fp32 too.  The W4A16 entry points take KSQ_F16 and KSQ_BF16: the reference's float instantiation
 * of that GEMM is empty (LK/asymmetric_gemm/asymmetric_gemm_wrapper.cu:44-85). */
typedef enum ksq_dtype { KSQ_F16 = 0, KSQ_BF16 = 1, KSQ_F32 = 2 } ksq_dtype;

/* Source layouts the repack step reads. */
typedef enum ksq_w4_layout {
  /* GPTQ checkpoint: qweight int32 [K/8, N], element k = 8r + j in bits 4j..4j+3 of row r; symmetric, the
   * zero point is 8 and qzeros are ignored (KS/models/quant/quant_weight.cpp:291-300, :73-75). */
  KSQ_W4_GPTQ_INT32_KPACK = 0,
  /* AWQ checkpoint: qweight int32 [K, N/8], slot j of a word holds column 8c + [0,2,4,6,1,3,5,7][j];
   * qzeros int32 [K/g, N/8] packed the same way (KS/models/quant/quant_weight.cpp:262-287). */
  KSQ_W4_AWQ_INT32_NPACK = 1,
  /* ksana's canonical form after CutlassAutoUnpack: int8 [K, N/2], low nibble = even column, signed q = u - 8
   * (KS/models/quant/quant_weight.cpp:249-251, :304-328) -- the input of the CUTLASS preprocessor that this
   * repack replaces (LK/asymmetric_gemm/cutlass_preprocessors.cpp:466-508). */
  KSQ_W4_ROWMAJOR_INT4_SIGNED = 2,
  /* What the loader's CUTLASS back end leaves in the weight tensor on sm80..sm89: the output of
   * preprocess_weights_for_mixed_gemm for W4_A16 (LK/asymmetric_gemm/cutlass_preprocessors.cpp:466-508):
   * rows permuted inside groups of 32 (:129-197), transposed to column major with eight k per 32-bit register
   * (:203-323), four columns interleaved per 64 rows (:426-464; ColumnMajorTileInterleave<64, 4>,
   * LK/cutlass_extensions/gemm/kernel/mixed_gemm_B_layout.h:106-120), nibbles biased to unsigned and
   * re-ordered [e0 e2 e4 e6 e1 e3 e5 e7] inside every register (:352-401).  Same byte count as the row-major
   * form; needs K % 64 == 0 and N % 4 == 0. */
  KSQ_W4_CUTLASS_SM80_INTERLEAVED = 3,
  /* The same preprocessor's output on sm90 (only the transpose runs: :487-490; the bias step is skipped,
   * :497-499): int8 [N, K/2], low nibble = even k, signed q = u - 8. */
  KSQ_W4_CUTLASS_SM90_COLMAJOR = 4,
  /* What the loader's Marlin back end leaves behind (gptq_marlin_repack / awq_marlin_repack,
   * LK/gptq_marlin/gptq_marlin_repack.cu:31-233, awq_marlin_repack.cu:30-170; both write the same format):
   * int32 [K/16, N*16/8], tiles of 16 k x 64 n = 128 words; word th*4 + w of a tile (th 0..31, w 0..3) holds, in
   * nibble slots [0,2,4,6,1,3,5,7] -> values 0..7, the elements k = 2*(th%4) + {0,1,8,9}, n = 16*w + th/4 (values
   * 0..3) and n + 8 (values 4..7), unsigned.  With this layout the scales are read in the Marlin order too
   * (MarlinPermuteScales, KS/models/quant/quant_weight.cpp:350-375) and AWQ zero points must be given as
   * KSQ_ZERO_MARLIN_INT32.  Needs N % 64 == 0.  A desc_act Marlin weight already has its rows in sorted order:
   * pass row_perm = NULL to the repack and the loader's perm as act_perm to the GEMM. */
  KSQ_W4_MARLIN = 5
} ksq_w4_layout;

/* Order of the columns in the repacked weight (and in its scale / zero words). */
typedef enum ksq_column_order {
  KSQ_COLS_NATURAL = 0,
  /* The source tensor is two halves side by side, [gate | up] along N (N/2 columns each); destination column
   * 2i is gate column i and 2i + 1 is up column i, which puts each pair into neighbouring lanes of one MFMA tile
   * for KSQ_EPILOGUE_SILU_MUL. */
  KSQ_COLS_HALVES_INTERLEAVED = 1
} ksq_column_order;

/* What the GEMMs do with the fp32 result before it is stored. */
typedef enum ksq_epilogue {
  KSQ_EPILOGUE_NONE = 0,
  /* out[m,n] = T(acc[m,n] + bias[n]), bias is T [n] (qkv bias: KS/models/common/common_model.cpp:456-459) */
  KSQ_EPILOGUE_BIAS = 1,
  /* weight columns interleaved as KSQ_COLS_HALVES_INTERLEAVED; out is [m, n/2]:
   * out[m,i] = T(silu(acc[m,2i]) * acc[m,2i+1]), silu(x) = x / (1 + exp(-x)), in fp32.  One GEMM instead of the
   * reference's two plus its SiLU-mul layer (common_model.cpp:540-547). */
  KSQ_EPILOGUE_SILU_MUL = 2
} ksq_epilogue;

/* How zero points are handed to the repack step. */
typedef enum ksq_zero_kind {
  KSQ_ZERO_NONE = 0,          /* symmetric: z = 8 for every group (GPTQ) */
  KSQ_ZERO_AWQ_INT32 = 1,     /* AWQ qzeros int32 [K/g, N/8], as in the checkpoint */
  KSQ_ZERO_UINT8 = 2,         /* unpacked z in [0,15], uint8 [K/g, N] */
  KSQ_ZERO_ADDITIVE = 3,      /* ksana's layer-boundary form: T [K/g, N] holding scales * (8 - z)
                                 (KS/models/quant/quant_weight.cpp:530-536); z is recovered exactly */
  KSQ_ZERO_MARLIN_INT32 = 4   /* Marlin zero points int32 [K/g, N/8] (MarlinZeroPoints, quant_weight.cpp:397-426):
                                 the scale permutation on blocks of 64, [0,2,4,6,1,3,5,7] on blocks of 8, packed
                                 eight columns per word in order */
} ksq_zero_kind;

typedef enum ksq_fp8_merge_mode {
  KSQ_FP8_MERGE_MAX = 0,         /* one scale = max of the three; the three row ranges are requantised in place */
  KSQ_FP8_MERGE_PER_CHANNEL = 1  /* one scale per row of the fused weight; the weight bytes are left alone (exact) */
} ksq_fp8_merge_mode;

typedef enum ksq_fp8_quant_mode {
  KSQ_FP8_PER_TENSOR_DYNAMIC = 0, /* one scale from the abs-max of the whole [m,k] tensor (is_static = false) */
  KSQ_FP8_PER_TENSOR_STATIC = 1,  /* caller-supplied scalar scale (checkpoint input_scale, is_static = true) */
  KSQ_FP8_PER_TOKEN_DYNAMIC = 2   /* one scale per row (num_channels = m) */
} ksq_fp8_quant_mode;

/* Library / error plumbing. */
int ksq_version(void);
const char* ksq_last_error_string(void);
/* Number of the compute units of the current device that the launch heuristics use (0 on failure). */
int ksq_device_compute_units(void);

/* Diagnostics (no counterpart in the reference): with the log switched on, every GEMM entry point records what it
 * launched -- kernel, template arguments, grid -- and ksq_last_launch_string() returns that of the calling thread's last
 * GEMM call ("" before the first).  Off by default: the launch path then formats nothing. */
void ksq_set_launch_log(int enabled);
const char* ksq_last_launch_string(void);

/* Split-K arrival counters in the caller's memory (no counterpart in the reference; its split-K semaphores live in the
 * workspace of every call, LK/asymmetric_gemm/fpA_intB_gemm/fpA_intB_gemm_template.h:498-504).
 * The kernels that split K across workgroups count arrivals in device memory that has to be zero between launches;
 * they return it to zero themselves.  By default that memory is the library's, one region per stream.  A caller can
 * bind KSQ_SPLITK_COUNTER_BYTES of its own device memory (256-byte aligned, zero-filled once by the caller) to a
 * stream: every later GEMM call on that stream -- and every graph captured from it while the binding holds -- uses it.
 * That is how two graphs captured from one stream can be replayed at the same time (bind different memory before each
 * capture), how more streams than the library has regions keep their split-K plans, and how a process recovers after
 * a kernel was aborted mid-flight (bind freshly zeroed memory).  counters == NULL removes the binding.  The memory
 * must stay valid while a launch or a captured graph that uses it can still run. */
#define KSQ_SPLITK_COUNTER_BYTES 65536
int ksq_bind_splitk_counters(void* stream, void* counters, size_t bytes);

/* ------------------------------------------------------------------ W4A16: load-time repack
 *
 * Replaces CutlassPreprocessWeightsForMixedGemmWarpper / preprocess_weights_for_mixed_gemm
 * (KS/models/quant/quant_weight.cpp:331-346, 577-579; LK/asymmetric_gemm/cutlass_preprocessors.cpp:466-508)
 * and the scale / zero binding of ConvertGroupTensor (quant_weight.cpp:530-536, 632-636).
 *
 * Output "fragment order" (N % 16 == 0, g in {64,128}, K a whole number of groups -- with g = 64 that includes the odd
 * multiples of 64 that the reference's kernels take, LK/asymmetric_gemm/fpA_intB_gemm/fpA_intB_gemm_template.h:168-171;
 * such a K is padded to whole 128-row tiles here: the rows past K hold u = z = 8 under a zero scale, the sizes below
 * count them, and the GEMM pads the activation rows to match in its workspace, so such a K needs a workspace):
 *   weight : K*N/2 bytes = tiles [N/16][K/128] of 1024 B.  Tile (nt,kt) is 64 lanes x 16 B; lane l = 16*j + c
 *            owns column n = 16*nt + c; 32-bit word d (0..3) of the lane covers k = 128*kt + 32*d + 8*j + e,
 *            e = 0..7, with element e in nibble e/2 when e is even and nibble 4 + e/2 when e is odd; nibbles are
 *            the unsigned u in [0,15].  One 128-bit load per lane is the B operand of four 16x16x32 MFMAs.
 *   sz     : (K/g)*N 32-bit words = [N/16][K/g][16]; word = scale bits (T) | z << 16 with z in [0,15]
 *            | E << 24, E (int8) = the largest binary exponent among the column's scales when they are bf16, else 0. */
/* Column tiles are contiguous in both buffers: tensors that share K (q_proj / k_proj / v_proj, gate_proj / up_proj)
 * are fused along N by repacking each, in order, to dst_weight + ksq_w4a16_repack_sizes(k, n_before).weight_bytes and
 * dst_sz + ...sz_bytes, n_before = the columns already placed (a multiple of 16); no concatenated copy is needed
 * (replaces the concat of KS/models/quant/quant_weight.cpp:471-513). */
int ksq_w4a16_repack_sizes(size_t k, size_t n, size_t group_size, size_t* weight_bytes, size_t* sz_bytes);

int ksq_w4a16_repack(int src_layout, const void* qweight, int zero_kind, const void* zeros, const void* scales,
                     int scale_dtype, size_t k, size_t n, size_t group_size, void* dst_weight, void* dst_sz,
                     void* stream);

/* Same transform on host memory (no GPU needed); used when weights are prepared before upload. */
int ksq_w4a16_repack_host(int src_layout, const void* qweight_host, int zero_kind, const void* zeros_host,
                          const void* scales_host, int scale_dtype, size_t k, size_t n, size_t group_size,
                          void* dst_weight_host, void* dst_sz_host);

/* The repack with a row permutation and a column order.  row_perm (int32 [k], device memory for the device
 * call; NULL = identity) makes destination row i hold source row row_perm[i]: with the permutation of
 * ksq_gptq_act_order_perm the rows of a desc_act GPTQ checkpoint end up grouped, so that scales[i / g] is the
 * scale of row i and the ordinary kernels apply; the activations' columns are permuted to match at run time
 * (the scheme of the reference's Marlin back end: LK/gptq_marlin/gptq_marlin.cu:380-392).  Scales and zeros are
 * indexed by group and are not permuted. */
int ksq_w4a16_repack_ex(int src_layout, const void* qweight, int zero_kind, const void* zeros, const void* scales,
                        int scale_dtype, size_t k, size_t n, size_t group_size, const int32_t* row_perm,
                        int column_order, void* dst_weight, void* dst_sz, void* stream);
int ksq_w4a16_repack_ex_host(int src_layout, const void* qweight_host, int zero_kind, const void* zeros_host,
                             const void* scales_host, int scale_dtype, size_t k, size_t n, size_t group_size,
                             const int32_t* row_perm_host, int column_order, void* dst_weight_host,
                             void* dst_sz_host);

/* perm = stable argsort of g_idx (MarlinSortGIdx, KS/models/quant/quant_weight.cpp:455-460), on the host.
 * Fails with KSQ_ERR_UNSUPPORTED unless every group 0 .. k/g - 1 has exactly g rows, which is what lets the
 * permuted tensor run on the kernels for grouped rows (the reference's is_k_full case, gptq_marlin.cu:386-392). */
int ksq_gptq_act_order_perm(const int32_t* g_idx_host, size_t k, size_t group_size, int32_t* perm_host);

/* out[m, i] = in[m, perm[i]] for a row-major [m, k] tensor of 16-bit elements (permute_cols_kernel,
 * LK/gptq_marlin/gptq_marlin.cu:380-384). */
int ksq_permute_columns(void* out, const void* in, const int32_t* perm, size_t m, size_t k, void* stream);

/* ------------------------------------------------------------------ W4A16: GEMM
 *
 * Replaces InvokeFpAIntBGroupCudaGemm / InvokeFpAIntBGroupCutlassGemm and
 * GetFpAIntBGroupCutlassGemmWorkspaceSize (KS/kernels/nvidia/kernel_wrapper.cpp:209-302), i.e.
 * FpAIntBGroupCudaGemmWrapper::Gemm (LK/weight_only_batched_gemv/weight_only_gemv_wrapper.cu:27-46) and
 * FpAIntBGroupCutlassGemmWrapper::Gemm (LK/asymmetric_gemm/asymmetric_gemm_wrapper.cu:53-77):
 *   out[m,n] = T( sum_k act[m,k] * s[k/g,n] * (u[k,n] - z[k/g,n]) ),  fp32 accumulation.
 * act is [m,k] row-major T, out is [m,n] row-major T, weight / sz come from ksq_w4a16_repack.
 * The workspace (256-byte aligned, ksq_w4a16_workspace_bytes) holds split-K partial sums and, for bf16
 * activations at m >= 65, the fp16 re-encoding of the activations.  With workspace == NULL, misaligned or too
 * small the call still succeeds on a slower route that needs none.  The workspace is scratch for the duration
 * of one call and holds no state between calls; calls that may overlap in time on one device need a workspace
 * each.  The arrival counters of the split-K kernels are library-owned device memory, one region per stream (the
 * first 64 streams per device that launch a split-K kernel; later streams get the same results without split-K):
 * launches on one stream never overlap, so no launch shares counters with one in flight -- with one exception:
 * two HIP graphs captured from the same stream and replayed at the same time on different streams would, unless the
 * caller binds counters of its own before each capture (ksq_bind_splitk_counters above). */
int ksq_w4a16_workspace_bytes(size_t max_m, size_t n, size_t k, size_t* bytes);

int ksq_w4a16_gemm(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m, size_t n,
                   size_t k, size_t group_size, void* workspace, size_t workspace_bytes, void* stream);

/* The same GEMM with the steps either side of it fused in:
 *   act_perm (int32 [k] or NULL): the activations' columns are gathered through it first (desc_act weights
 *     repacked with the same permutation); needs a workspace from ksq_w4a16_workspace_bytes_ex(.., 1, ..),
 *     whose first m*k*2 bytes (rounded up to 256) hold the permuted copy -- without one the call fails with
 *     KSQ_ERR_WORKSPACE;
 *   epilogue / bias: see ksq_epilogue.  n is the width of the weight; out has n/2 columns for SILU_MUL. */
int ksq_w4a16_workspace_bytes_ex(size_t max_m, size_t n, size_t k, int act_order, size_t* bytes);
int ksq_w4a16_gemm_ex(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m,
                      size_t n, size_t k, size_t group_size, const int32_t* act_perm, int epilogue,
                      const void* bias, void* workspace, size_t workspace_bytes, void* stream);

/* ksq_w4a16_gemm for callers that cannot allocate device memory (code under HIP graph capture that owns no
 * buffer, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference, whose
 * layers always receive a workspace from their factory.  The split-K partial tiles and, for bf16 activations at
 * m >= 65, the re-encoded activations go to a file-scope device array of KSQ_STATIC_SCRATCH_BYTES inside the library
 * (every GPU the library runs on holds its own copy until the process ends); the call allocates and frees nothing.
 * A shape whose ksq_w4a16_workspace_bytes(m, n, k) exceeds KSQ_STATIC_SCRATCH_BYTES fails with KSQ_ERR_WORKSPACE
 * (every shape of Llama-2-7B / Llama-3-70B width fits up to m = 64).  All calls on one GPU share the one array:
 * calls that may overlap in time on one GPU (different streams, different threads) race; serialise them or use
 * ksq_w4a16_gemm with a workspace each.  The result is bit-identical to ksq_w4a16_gemm given a workspace of
 * ksq_w4a16_workspace_bytes(m, n, k) bytes.  The first call of the library on a device resolves the array's
 * address: make one call (ksq_device_compute_units() will do) on every device before capturing a graph. */
#define KSQ_STATIC_SCRATCH_BYTES (64u << 20)
int ksq_w4a16_gemm_static_scratch(int dtype, void* out, const void* act, const void* weight, const void* sz,
                                  size_t m, size_t n, size_t k, size_t group_size, void* stream);

/* ------------------------------------------------------------------ FP8 e4m3 (OCP: bias 7, max 448, no inf)
 *
 * ksq_fp8_quantize replaces Fp8E4m3Quantize (KS/kernels/nvidia/kernel_wrapper.cpp:1015-1027) =
 * InvokeComputeFP8QuantizeScale + InvokeQuantizeMatrix (LU/cuda_fp8_utils.cu:27-44, 85-127):
 *   scale[c] = max(absmax(x[c,:]) / 448, 1/(448*512));  q = e4m3(clamp(x / scale[c], +-448)).
 * act is [m,k] T; act_q is [m,k] bytes; act_scale holds 1 float (per-tensor) or m floats (per-token). */
int ksq_fp8_quantize(int dtype, const void* act, size_t m, size_t k, int mode, void* act_q, float* act_scale,
                     void* stream);

/* Replaces RescaleFp8E4m3 (KS/kernels/nvidia/kernel_wrapper.cpp:1043-1046, LU/cuda_fp8_utils.cu:140-155):
 * out[i] = e4m3(float(in[i]) * (*scale_in / *scale_out)); in-place allowed. */
int ksq_fp8_rescale(const void* in, void* out, size_t count, const float* scale_in, const float* scale_out,
                    void* stream);

/* On-the-fly weight conversion, replaces the device work of ConvertFp8E4m3Tensor
 * (KS/models/quant/quant_weight.cpp:685-726): w is [k,n] T; w_q becomes [n,k] e4m3 (k contiguous) with a single
 * scale written to w_scale[0]. */
int ksq_fp8_convert_weight(int dtype, const void* w, size_t k, size_t n, void* w_q, float* w_scale, void* stream);

/* The same with one scale per output channel (the per-channel x per-token form of ksq_fp8_gemm):
 * w_scale[c] = max(absmax(w[:,c]) / 448, 1/(448*512)), w_q[c,:] = e4m3(clamp(w[:,c] / w_scale[c], +-448)). */
int ksq_fp8_convert_weight_per_channel(int dtype, const void* w, size_t k, size_t n, void* w_q, float* w_scale,
                                       void* stream);

/* Fused q/k/v weight [nq+nk+nv, k] e4m3 whose three row ranges were quantised with their own scalar scales.
 * KSQ_FP8_MERGE_MAX replaces BindFp8E4m3ScaleOfQkvWeight + GetMaxScaleOfQkv
 * (KS/models/quant/quant_weight.cpp:816-897): w_scale[0] = max of the three and every range is requantised in place,
 * w_q = e4m3(float(w_q) * (part_scale / w_scale[0])).  KSQ_FP8_MERGE_PER_CHANNEL writes nq+nk+nv scales instead and
 * leaves w_q untouched (may be NULL): the per-channel GEMM then reproduces the three separate GEMMs exactly. */
int ksq_fp8_merge_qkv_scales(int mode, const float* q_scale, const float* k_scale, const float* v_scale, size_t nq,
                             size_t nk, size_t nv, void* w_q, size_t k, float* w_scale, void* stream);

/* Replaces Fp8QuantizedMatMul (KS/kernels/nvidia/kernel_wrapper.cpp:1033-1041, cuBLASLt FP8 matmul through
 * LK/gemm_wrapper/gemm_wrapper.cc:39-107), extended to the per-token x per-channel scales of
 * LK/asymmetric_gemm/fp8_rowwise_gemm/fp8_rowwise_gemm_kernel_template_sm90.h:119-131:
 *   out[m,n] = T( (sum_k a[m,k] * w[n,k]) * w_scale[n or 0] * act_scale[m or 0] ),  fp32 accumulation.
 * act_q is [m,k] e4m3, w_q is [n,k] e4m3 (k contiguous), scale counts are 1 or m / 1 or n. */
int ksq_fp8_workspace_bytes(size_t max_m, size_t n, size_t k, size_t* bytes);

int ksq_fp8_gemm(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                 const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                 void* workspace, size_t workspace_bytes, void* stream);

/* The same GEMM with an epilogue (see ksq_epilogue).  For KSQ_EPILOGUE_SILU_MUL the rows of w_q (and, when there
 * are n of them, its scales) are interleaved gate / up: row 2i = gate row i, row 2i + 1 = up row i
 * (ksq_interleave_halves builds that from [gate ; up]); out is [m, n/2]. */
int ksq_fp8_gemm_ex(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                    const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                    int epilogue, const void* bias, void* workspace, size_t workspace_bytes, void* stream);

/* Per-token dynamic quantisation and the GEMM as one call: act is [m,k] T (not yet quantised), out is T,
 *   scale[r] = max(absmax(act[r,:]) / 448, 1/(448*512)),  a_q = e4m3(clamp(act / scale[r], +-448)),
 *   out[m,n] = T( (sum_k a_q[m,k] * w[n,k]) * w_scale[n or 0] * scale[m] ),
 * i.e. ksq_fp8_quantize(KSQ_FP8_PER_TOKEN_DYNAMIC) followed by ksq_fp8_gemm_ex, which is what it runs for m > 1: one
 * call for the reference's Fp8E4m3Quantize + Fp8QuantizedMatMul pair (KS/kernels/nvidia/kernel_wrapper.cpp:1015-1041,
 * KS/layers/nvidia/fp8_matmul_layer.cpp:56-63).  A single token (k a multiple of 128, at most 8192) is one launch:
 * every workgroup takes the row maximum and quantises the activations itself, with the same arithmetic, so the
 * quantised bytes are those of ksq_fp8_quantize.  (Measured, that form only ties with the two launches at one row and
 * loses from two rows on, since every workgroup repeats the quantisation; it can do up to eight rows.)  The workspace
 * (ksq_fp8_gemm_dynamic_workspace_bytes, 256-byte aligned) holds the quantised activations and scales of the two-launch
 * route and the split-K partial sums; without one only the single-launch case works, anything else fails with
 * KSQ_ERR_WORKSPACE. */
int ksq_fp8_gemm_dynamic_workspace_bytes(size_t max_m, size_t n, size_t k, size_t* bytes);
int ksq_fp8_gemm_dynamic(int dtype, void* out, const void* act, const void* w_q, const float* w_scale,
                         size_t w_scale_count, size_t m, size_t n, size_t k, int epilogue, const void* bias,
                         void* workspace, size_t workspace_bytes, void* stream);

/* out row 2i = in row i, out row 2i + 1 = in row rows/2 + i, for rows of row_bytes bytes (rows even, row_bytes a
 * multiple of 4; in and out must not overlap).  Load-time helper for the interleaved gate / up weight and its
 * per-channel scales (row_bytes = 4). */
int ksq_interleave_halves(void* out, const void* in, size_t rows, size_t row_bytes, void* stream);

/* ------------------------------------------------------------------ row maxima from the producing GEMM
 *
 * The producer's half of folding the per-token FP8 quantisation into its neighbour (no counterpart in the reference,
 * whose quantiser makes a max pass of its own over the tensor: LU/cuda_fp8_utils.cu:85-127, merging blocks by atomic
 * maximum on the float bits, :111-115 -- the same merge is used here, from the GEMM's epilogue).
 *
 * ksq_w4a16_gemm_rowmax / ksq_fp8_gemm_rowmax are ksq_w4a16_gemm_ex (without act_perm) / ksq_fp8_gemm_ex; in
 * addition the largest |out[row, :]| of every row -- of the values as stored, after the epilogue -- is merged into
 * row_absmax[row] (fp32 [m]) by atomic maximum.  row_absmax must hold zeros on entry (ksq_fill_zero_f32, which is
 * safe to record into a HIP graph), or the maxima of columns that another call contributed.
 * ksq_fp8_quantize_rows_from_absmax is then ksq_fp8_quantize(KSQ_FP8_PER_TOKEN_DYNAMIC) without its max pass:
 * act_scale[r] = max(row_absmax[r] / 448, 1 / (448 * 512)), one read of act; bit-identical bytes and scales when
 * row_absmax holds the rows' maxima. */
int ksq_fill_zero_f32(float* p, size_t count, void* stream);
int ksq_w4a16_gemm_rowmax(int dtype, void* out, const void* act, const void* weight, const void* sz, size_t m, size_t n,
                          size_t k, size_t group_size, int epilogue, const void* bias, float* row_absmax,
                          void* workspace, size_t workspace_bytes, void* stream);
int ksq_fp8_gemm_rowmax(int out_dtype, void* out, const void* act_q, const float* act_scale, size_t act_scale_count,
                        const void* w_q, const float* w_scale, size_t w_scale_count, size_t m, size_t n, size_t k,
                        int epilogue, const void* bias, float* row_absmax, void* workspace, size_t workspace_bytes,
                        void* stream);
int ksq_fp8_quantize_rows_from_absmax(int dtype, const void* act, size_t m, size_t k, const float* row_absmax,
                                      void* act_q, float* act_scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KSQ_H_ */
