// Implementation of the layer shims over the C ABI (ksq.h).  Error conventions follow the reference: success is
// Status(); misuse and device errors raise std::runtime_error through KLLM_THROW (KS/utils/logger.h:123), the way
// KS/layers/nvidia/{group_matmul,fp8_matmul}_layer.cpp and the kernel library do.
#include <hip/hip_runtime_api.h>

#include <mutex>
#include <sstream>
#include <unordered_map>

#include "fp8_matmul_layer.h"
#include "group_matmul_layer.h"
#include "ksq.h"

namespace ksana_llm {

namespace {

void ThrowOnKsqError(int code, const char* what) {
  if (code == KSQ_OK) return;
  std::ostringstream os;
  os << what << " failed (" << code << "): " << ksq_last_error_string();
  KLLM_THROW(os.str());
}

template <typename T>
int KsqDtype() {
  return TypeTraits<T>::kDataType == TYPE_FP16 ? KSQ_F16 : (TypeTraits<T>::kDataType == TYPE_FP32 ? KSQ_F32 : KSQ_BF16);
}

constexpr size_t kFp8GemmWorkspaceBytes = 32ull << 20;  // the reference reserves 32 MiB for cuBLASLt here

}  // namespace

Status CreateTensor(Tensor& tensor, const std::vector<size_t>& shape, DataType dtype, int rank, MemoryDevice device) {
  (void)rank;
  tensor.device = device;
  tensor.dtype = dtype;
  tensor.shape = shape;
  const size_t bytes = tensor.GetTotalBytes();
  void* ptr = nullptr;
  if (bytes > 0) {
    hipError_t e = device == MEMORY_DEVICE ? hipMalloc(&ptr, bytes) : hipHostMalloc(&ptr, bytes, 0);
    if (e != hipSuccess) KLLM_THROW(std::string("CreateTensor: ") + hipGetErrorString(e));
  }
  tensor.refer_ptr = ptr;
  return Status();
}

Status DestroyTensor(Tensor& tensor, int rank) {
  (void)rank;
  if (tensor.refer_ptr) {
    if (tensor.device == MEMORY_DEVICE) (void)hipFree(tensor.refer_ptr);
    else (void)hipHostFree(tensor.refer_ptr);
  }
  tensor.refer_ptr = nullptr;
  return Status();
}

// ---------------------------------------------------------------------------------------------- GroupMatMulLayer
namespace {

// Weights that reached Forward as the reference's own loader leaves them (QuantWeight::ConvertGroupTensor,
// KS/models/quant/quant_weight.cpp:463-660: "*.weight" preprocessed for its CUTLASS or Marlin back end, `.scales` in
// T, `.zeros` additive in T) and were converted on their first use: the bytes of the loader's tensor now hold the
// fragment order (same size), the scale/zero words live here.  Keyed by the loader's device pointer and shared by
// all layers of the process, since one layer object serves the same projection of every decoder layer.
struct AdoptedWeight {
  void* weight = nullptr;  // what the GEMM reads: the loader's own tensor, or `padded` when K had to be padded
  Tensor sz;
  Tensor padded;
};
std::mutex g_adopted_mutex;
std::unordered_map<const void*, AdoptedWeight> g_adopted;

}  // namespace

void ForgetAdoptedGroupQuantWeights(int rank) {
  std::lock_guard<std::mutex> lock(g_adopted_mutex);
  for (auto& kv : g_adopted) {
    DestroyTensor(kv.second.sz, rank);
    DestroyTensor(kv.second.padded, rank);
  }
  g_adopted.clear();
}

template <typename T, DataType WT>
void GroupMatMulLayer<T, WT>::AdoptLoaderWeight(const Tensor& weight_tensor, void** weight, void** sz) {
  std::lock_guard<std::mutex> lock(g_adopted_mutex);
  auto it = g_adopted.find(weight_tensor.refer_ptr);
  if (it == g_adopted.end()) {
    // First use: not safe under graph capture (it allocates and synchronises); the warm-up step that every serving
    // engine runs before it captures takes care of that.
    const GroupWeightLayout layout = backend_ == MARLIN_BACKEND ? GROUP_WEIGHT_MARLIN : loader_layout_;
    Stream& stream = context_->GetComputeStreams()[rank_];
    Tensor fresh, fresh_sz;
    RepackGroupQuantWeight(layout, weight_tensor, weight_tensor.zeros, /*zeros_additive=*/true, *weight_tensor.scales,
                           max_k_, max_n_, groupsize_, fresh, fresh_sz, rank_, stream);
    AdoptedWeight ad;
    ad.sz = fresh_sz;
    const size_t loader_bytes = max_k_ * max_n_ / 2;
    if (fresh.GetTotalBytes() == loader_bytes) {
      hipError_t e = hipMemcpyAsync(weight_tensor.refer_ptr, fresh.refer_ptr, loader_bytes, hipMemcpyDeviceToDevice,
                                    static_cast<hipStream_t>(stream.Get()));
      if (e == hipSuccess) e = hipStreamSynchronize(static_cast<hipStream_t>(stream.Get()));
      if (e != hipSuccess) KLLM_THROW(std::string("GroupMatMulLayer: adopting a loader-format weight: ") + hipGetErrorString(e));
      DestroyTensor(fresh, rank_);
      ad.weight = weight_tensor.refer_ptr;
    } else {  // K = 64 x odd: the fragment order pads the last k tile and no longer fits the loader's tensor
      ad.padded = fresh;
      ad.weight = fresh.refer_ptr;
    }
    it = g_adopted.emplace(weight_tensor.refer_ptr, ad).first;
  }
  *weight = it->second.weight;
  *sz = it->second.sz.refer_ptr;
}

template <typename T, DataType WT>
Status GroupMatMulLayer<T, WT>::Init(const std::vector<std::any>& parameters, std::shared_ptr<Context> context,
                                     int rank) {
  context_ = context;
  rank_ = rank;

  int parameter_index = 0;
  is_awq_ = std::any_cast<const bool>(parameters[parameter_index++]);
  is_gptq_desc_ = std::any_cast<const bool>(parameters[parameter_index++]);
  is_k_full_ = std::any_cast<const bool>(parameters[parameter_index++]);
  backend_ = std::any_cast<const GroupQuantBackend>(parameters[parameter_index++]);
  max_m_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  max_n_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  max_k_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  groupsize_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  cutlass_use_gemv_cuda_core_ = std::any_cast<const bool>(parameters[parameter_index++]);

  is_k_full_ = is_gptq_desc_ ? is_k_full_ : true;
  return Status();
}

template <typename T, DataType WT>
size_t GroupMatMulLayer<T, WT>::GetWorkSpaceSize() {
  if constexpr (WT == TYPE_I4_GROUP) {
    size_t bytes = 0;
    // the kernels take whole groups (and the reference k % 64 == 0: fpA_intB_gemm_template.h:168-171)
    if (groupsize_ == 0 || max_k_ % groupsize_ != 0) KLLM_THROW("GroupMatMulLayer: k is not a multiple of the group size.");
    ThrowOnKsqError(ksq_w4a16_workspace_bytes_ex(max_m_, max_n_, max_k_, is_gptq_desc_ ? 1 : 0, &bytes),
                    "ksq_w4a16_workspace_bytes_ex");
    return bytes;
  } else {
    KLLM_THROW("Not supported weight data type. GroupMatMul only supports TYPE_I4_GROUP.");
  }
}

template <typename T, DataType WT>
Status GroupMatMulLayer<T, WT>::Preprocess(const ModelConfig& model_config_) {
  (void)model_config_;
  if constexpr (WT != TYPE_I4_GROUP) {
    KLLM_THROW("Not supported weight data type. GroupMatMul only supports TYPE_I4_GROUP.");
  }
  return Status();
}

template <typename T, DataType WT>
Status GroupMatMulLayer<T, WT>::Forward(const std::vector<Tensor>& input_tensors,
                                        std::vector<Tensor>& output_tensors) {
  if constexpr (WT == TYPE_I4_GROUP) {
    const Tensor& weight_tensor = input_tensors[1];
    if (weight_tensor.scales == nullptr) {
      KLLM_THROW("GroupMatMulLayer: weight tensor has no scales bound.");
    }
    const int32_t* act_perm = nullptr;
    if (is_gptq_desc_) {
      // the reference serves desc_act through its Marlin back end only (KS/utils/environment.cpp:105-106); here the
      // rows were grouped at load time and the activations follow them
      if (!is_k_full_) KLLM_THROW("GroupMatMulLayer: desc_act with a partial K (is_k_full = false) is not supported.");
      if (weight_tensor.perm == nullptr) KLLM_THROW("GroupMatMulLayer: desc_act weight tensor has no perm bound.");
      act_perm = weight_tensor.perm->GetPtr<int32_t>();
    }
    void* p_qweight_tensor = weight_tensor.GetPtr<void>();
    void* p_sz_tensor = weight_tensor.scales->GetPtr<void>();
    if (weight_tensor.scales->dtype == TYPE_FP16 || weight_tensor.scales->dtype == TYPE_BF16) {
      // not repacked by RepackGroupQuantWeight: the reference loader's own output, converted on first use
      if (is_gptq_desc_) KLLM_THROW("GroupMatMulLayer: a desc_act weight must be repacked with its perm at load time.");
      AdoptLoaderWeight(weight_tensor, &p_qweight_tensor, &p_sz_tensor);
    }

    const size_t m = input_tensors[0].shape[0];
    const size_t n = max_n_;
    const size_t k = max_k_;

    void* ws = workspace_buffer_ ? workspace_buffer_->GetPtr<void>() : nullptr;
    const size_t ws_bytes = workspace_buffer_ ? workspace_buffer_->GetTotalBytes() : 0;
    ThrowOnKsqError(
        ksq_w4a16_gemm_ex(KsqDtype<T>(), output_tensors[0].GetPtr<void>(), input_tensors[0].GetPtr<void>(),
                          p_qweight_tensor, p_sz_tensor, m, n, k, groupsize_, act_perm, epilogue_,
                          bias_ ? bias_->GetPtr<void>() : nullptr, ws, ws_bytes,
                          context_->GetComputeStreams()[rank_].Get()),
        "ksq_w4a16_gemm_ex");

    output_tensors[0].shape = {m, epilogue_ == KSQ_EPILOGUE_SILU_MUL ? n / 2 : n};
    output_tensors[0].dtype = input_tensors[0].dtype;
    return Status();
  } else {
    KLLM_THROW("Not supported weight data type. GroupMatMul only supports TYPE_I4_GROUP.");
  }
}

template <typename T, DataType WT>
void GroupMatMulLayer<T, WT>::SetEpilogue(int kind, const Tensor* bias) {
  if (kind < KSQ_EPILOGUE_NONE || kind > KSQ_EPILOGUE_SILU_MUL) KLLM_THROW("GroupMatMulLayer: unknown epilogue.");
  if (kind == KSQ_EPILOGUE_BIAS && bias == nullptr) KLLM_THROW("GroupMatMulLayer: the bias epilogue needs a bias.");
  epilogue_ = kind;
  bias_ = kind == KSQ_EPILOGUE_BIAS ? bias : nullptr;
}

template class GroupMatMulLayer<float16, TYPE_I4_GROUP>;
template class GroupMatMulLayer<bfloat16, TYPE_I4_GROUP>;

namespace {

int KsqLayout(GroupWeightLayout layout) {
  return layout == GROUP_WEIGHT_GPTQ_INT32     ? KSQ_W4_GPTQ_INT32_KPACK
         : layout == GROUP_WEIGHT_AWQ_INT32    ? KSQ_W4_AWQ_INT32_NPACK
         : layout == GROUP_WEIGHT_CUTLASS_SM80 ? KSQ_W4_CUTLASS_SM80_INTERLEAVED
         : layout == GROUP_WEIGHT_CUTLASS_SM90 ? KSQ_W4_CUTLASS_SM90_COLMAJOR
         : layout == GROUP_WEIGHT_MARLIN       ? KSQ_W4_MARLIN
                                               : KSQ_W4_ROWMAJOR_INT4_SIGNED;
}

int KsqZeroKind(GroupWeightLayout layout, const Tensor* qzeros, bool zeros_additive) {
  if (qzeros == nullptr) return KSQ_ZERO_NONE;
  if (layout == GROUP_WEIGHT_MARLIN) return KSQ_ZERO_MARLIN_INT32;
  if (zeros_additive) return KSQ_ZERO_ADDITIVE;
  return (qzeros->dtype == TYPE_INT32 || qzeros->dtype == TYPE_UINT32) ? KSQ_ZERO_AWQ_INT32 : KSQ_ZERO_UINT8;
}

}  // namespace

Status RepackGroupQuantWeight(GroupWeightLayout layout, const Tensor& qweight, const Tensor* qzeros,
                              bool zeros_additive, const Tensor& scales, size_t k, size_t n, size_t groupsize,
                              Tensor& weight, Tensor& weight_sz, int rank, Stream& stream, Tensor* perm,
                              bool interleave_gate_up) {
  size_t weight_bytes = 0, sz_bytes = 0;
  ThrowOnKsqError(ksq_w4a16_repack_sizes(k, n, groupsize, &weight_bytes, &sz_bytes), "ksq_w4a16_repack_sizes");
  if (scales.dtype != TYPE_FP16 && scales.dtype != TYPE_BF16) KLLM_THROW("RepackGroupQuantWeight: scales must be fp16 or bf16.");
  // ksana's "*.weight" shape, with K rounded up to whole k tiles of 128 as the repack writes it (K = 64 x odd under
  // group size 64 gains half a tile of padding: the sizes are the library's, never k * n / 2 computed here)
  const size_t kp = weight_bytes / (n / 2);
  CreateTensor(weight, {kp, n / 2}, TYPE_UINT8, rank, MEMORY_DEVICE);
  CreateTensor(weight_sz, {sz_bytes / (4 * n), n}, TYPE_UINT32, rank, MEMORY_DEVICE);
  const int src = KsqLayout(layout);
  if (perm != nullptr && (perm->dtype != TYPE_INT32 || perm->GetElementNumber() != k))
    KLLM_THROW("RepackGroupQuantWeight: perm must be int32 [k].");
  const int zero_kind = KsqZeroKind(layout, qzeros, zeros_additive);
  ThrowOnKsqError(
      ksq_w4a16_repack_ex(src, qweight.GetPtr<void>(), zero_kind, qzeros ? qzeros->GetPtr<void>() : nullptr,
                          scales.GetPtr<void>(), scales.dtype == TYPE_FP16 ? KSQ_F16 : KSQ_BF16, k, n, groupsize,
                          perm ? perm->GetPtr<int32_t>() : nullptr,
                          interleave_gate_up ? KSQ_COLS_HALVES_INTERLEAVED : KSQ_COLS_NATURAL, weight.GetPtr<void>(),
                          weight_sz.GetPtr<void>(), stream.Get()),
      "ksq_w4a16_repack_ex");
  weight.dtype = TYPE_I4_GROUP;
  weight.scales = &weight_sz;
  weight.perm = perm;
  return Status();
}

Status RepackFusedGroupQuantWeight(GroupWeightLayout layout, const std::vector<GroupWeightPart>& parts,
                                   bool zeros_additive, size_t k, size_t groupsize, Tensor& weight, Tensor& weight_sz,
                                   int rank, Stream& stream) {
  size_t n = 0;
  for (const GroupWeightPart& part : parts) {
    if (part.qweight == nullptr || part.scales == nullptr || part.n == 0 || part.n % 16 != 0)
      KLLM_THROW("RepackFusedGroupQuantWeight: every part needs a weight, scales and a width that is a multiple of 16.");
    if (part.scales->dtype != parts[0].scales->dtype || (part.qzeros == nullptr) != (parts[0].qzeros == nullptr))
      KLLM_THROW("RepackFusedGroupQuantWeight: the parts must agree in scale type and in having zero points.");
    n += part.n;
  }
  if (parts.empty()) KLLM_THROW("RepackFusedGroupQuantWeight: no parts.");
  const DataType st = parts[0].scales->dtype;
  if (st != TYPE_FP16 && st != TYPE_BF16) KLLM_THROW("RepackFusedGroupQuantWeight: scales must be fp16 or bf16.");
  size_t weight_bytes = 0, sz_bytes = 0;
  ThrowOnKsqError(ksq_w4a16_repack_sizes(k, n, groupsize, &weight_bytes, &sz_bytes), "ksq_w4a16_repack_sizes");
  CreateTensor(weight, {weight_bytes / (n / 2), n / 2}, TYPE_UINT8, rank, MEMORY_DEVICE);  // K in whole k tiles
  CreateTensor(weight_sz, {sz_bytes / (4 * n), n}, TYPE_UINT32, rank, MEMORY_DEVICE);
  size_t n0 = 0;
  for (const GroupWeightPart& part : parts) {
    // columns n0 .. n0 + part.n - 1 are the column tiles n0 / 16 .. of the fused buffers: a contiguous range of each
    size_t part_w = 0, part_sz = 0;
    ThrowOnKsqError(ksq_w4a16_repack_sizes(k, n0 == 0 ? part.n : n0, groupsize, &part_w, &part_sz), "ksq_w4a16_repack_sizes");
    const size_t w_off = n0 == 0 ? 0 : part_w, sz_off = n0 == 0 ? 0 : part_sz;  // bytes taken by the columns before n0
    ThrowOnKsqError(
        ksq_w4a16_repack(KsqLayout(layout), part.qweight->GetPtr<void>(), KsqZeroKind(layout, part.qzeros, zeros_additive),
                         part.qzeros ? part.qzeros->GetPtr<void>() : nullptr, part.scales->GetPtr<void>(),
                         st == TYPE_FP16 ? KSQ_F16 : KSQ_BF16, k, part.n, groupsize, weight.GetPtr<char>() + w_off,
                         weight_sz.GetPtr<char>() + sz_off, stream.Get()),
        "ksq_w4a16_repack");
    n0 += part.n;
  }
  weight.dtype = TYPE_I4_GROUP;
  weight.scales = &weight_sz;
  return Status();
}

Status SortGptqGIdx(const std::vector<int32_t>& g_idx, size_t groupsize, std::vector<int32_t>& perm) {
  perm.assign(g_idx.size(), 0);
  ThrowOnKsqError(ksq_gptq_act_order_perm(g_idx.data(), g_idx.size(), groupsize, perm.data()),
                  "ksq_gptq_act_order_perm");
  return Status();
}

// ------------------------------------------------------------------------------------------------ Fp8MatMulLayer
template <typename T>
Status Fp8MatMulLayer<T>::Init(const std::vector<std::any>& parameters, std::shared_ptr<Context> context, int rank) {
  STATUS_CHECK_FAILURE(BaseLayer::Init(parameters, context, rank));
  int parameter_index = 0;
  max_m_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  max_k_ = std::any_cast<const size_t>(parameters[parameter_index++]);
  return Status();
}

template <typename T>
size_t Fp8MatMulLayer<T>::GetWorkSpaceSize(const int m, const int k) {
  // [ GEMM split-K workspace | m*k e4m3 activations | m float scales ]; the reference's layout with one scale
  // slot per token instead of one in total (KS/layers/nvidia/fp8_matmul_layer.cpp:22-28, 45-46, 60)
  size_t input_size = (size_t)m * k * GetTypeSize(TYPE_FP8_E4M3);
  input_size = (input_size + 15) / 16 * 16;
  size_t scale_size = (size_t)m * GetTypeSize(TYPE_FP32);
  return input_size + scale_size + kFp8GemmWorkspaceBytes + 512;  // + the slack of two 256-byte roundings
}

template <typename T>
size_t Fp8MatMulLayer<T>::GetWorkSpaceSize() {
  return GetWorkSpaceSize(max_m_, max_k_);
}

template <typename T>
Status Fp8MatMulLayer<T>::Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) {
  int m = input_tensors[0].shape[0];
  int k = input_tensors[0].shape[1];
  int n = input_tensors[1].shape[0];
  const void* input = input_tensors[0].GetPtr<const void>();
  size_t workspace_size = GetWorkSpaceSize(m, k);
  if (!workspace_buffer_ || workspace_size > workspace_buffer_->GetTotalBytes()) {
    std::ostringstream os;
    os << "workspace size " << workspace_size << " > buffer size "
       << (workspace_buffer_ ? workspace_buffer_->GetTotalBytes() : 0);
    KLLM_THROW(os.str());
  }
  char* gemm_workspace = workspace_buffer_->GetPtr<char>();
  char* input_quant = gemm_workspace + kFp8GemmWorkspaceBytes;
  const void* weight_quant = input_tensors[1].GetPtr<const void>();
  const float* weight_scale =
      input_tensors[1].weight_scales ? input_tensors[1].weight_scales->GetPtr<const float>() : nullptr;
  if (weight_scale == nullptr) {
    KLLM_THROW("Cannot load weight_scale. Weight_scale is nullptr.");
  }
  const size_t weight_scale_count = input_tensors[1].weight_scales->GetElementNumber() == (size_t)n && n > 1 ? n : 1;
  void* output = output_tensors[0].GetPtr<void>();
  output_tensors[0].shape = {static_cast<size_t>(m),
                             static_cast<size_t>(epilogue_ == KSQ_EPILOGUE_SILU_MUL ? n / 2 : n)};
  output_tensors[0].dtype = input_tensors[0].dtype;
  void* stream = context_->GetComputeStreams()[rank_].Get();
  float* input_scale = nullptr;
  size_t input_scale_count = 1;
  size_t quant_bytes = ((size_t)m * k + 15) / 16 * 16;
  if (input_tensors[1].input_scales) {
    input_scale = input_tensors[1].input_scales->GetPtr<float>();
    ThrowOnKsqError(ksq_fp8_quantize(KsqDtype<T>(), input, m, k, KSQ_FP8_PER_TENSOR_STATIC, input_quant, input_scale,
                                     stream), "ksq_fp8_quantize");
  } else if (weight_scale_count > 1) {
    // per-channel weight scales go with per-token activation scales: quantisation and GEMM as one call (a single
    // launch for decode batches of up to eight tokens); the call carves the same buffer up itself
    ThrowOnKsqError(ksq_fp8_gemm_dynamic(KsqDtype<T>(), output, input, weight_quant, weight_scale, weight_scale_count, m,
                                         n, k, epilogue_, bias_ ? bias_->GetPtr<void>() : nullptr, gemm_workspace,
                                         workspace_buffer_->GetTotalBytes(), stream), "ksq_fp8_gemm_dynamic");
    return Status();
  } else {
    input_scale = reinterpret_cast<float*>(input_quant + quant_bytes);
    const bool per_token = false;
    input_scale_count = per_token ? m : 1;
    ThrowOnKsqError(ksq_fp8_quantize(KsqDtype<T>(), input, m, k,
                                     per_token ? KSQ_FP8_PER_TOKEN_DYNAMIC : KSQ_FP8_PER_TENSOR_DYNAMIC, input_quant,
                                     input_scale, stream), "ksq_fp8_quantize");
  }
  ThrowOnKsqError(ksq_fp8_gemm_ex(KsqDtype<T>(), output, input_quant, input_scale, input_scale_count, weight_quant,
                                  weight_scale, weight_scale_count, m, n, k, epilogue_,
                                  bias_ ? bias_->GetPtr<void>() : nullptr, gemm_workspace, kFp8GemmWorkspaceBytes,
                                  stream), "ksq_fp8_gemm_ex");
  return Status();
}

template <typename T>
void Fp8MatMulLayer<T>::SetEpilogue(int kind, const Tensor* bias) {
  if (kind < KSQ_EPILOGUE_NONE || kind > KSQ_EPILOGUE_SILU_MUL) KLLM_THROW("Fp8MatMulLayer: unknown epilogue.");
  if (kind == KSQ_EPILOGUE_BIAS && bias == nullptr) KLLM_THROW("Fp8MatMulLayer: the bias epilogue needs a bias.");
  epilogue_ = kind;
  bias_ = kind == KSQ_EPILOGUE_BIAS ? bias : nullptr;
}

Status ConvertFp8Weight(const Tensor& weight, bool per_channel, Tensor& weight_fp8, Tensor& weight_scale, int rank,
                        Stream& stream) {
  if (weight.shape.size() != 2) KLLM_THROW("ConvertFp8Weight: weight must be [k, n].");
  if (weight.dtype != TYPE_FP16 && weight.dtype != TYPE_BF16) KLLM_THROW("ConvertFp8Weight: weight must be fp16 or bf16.");
  const size_t k = weight.shape[0], n = weight.shape[1];
  CreateTensor(weight_fp8, {n, k}, TYPE_FP8_E4M3, rank, MEMORY_DEVICE);
  CreateTensor(weight_scale, {per_channel ? n : 1}, TYPE_FP32, rank, MEMORY_DEVICE);
  const int dt = weight.dtype == TYPE_FP16 ? KSQ_F16 : KSQ_BF16;
  if (per_channel)
    ThrowOnKsqError(ksq_fp8_convert_weight_per_channel(dt, weight.GetPtr<void>(), k, n, weight_fp8.GetPtr<void>(),
                                                       weight_scale.GetPtr<float>(), stream.Get()),
                    "ksq_fp8_convert_weight_per_channel");
  else
    ThrowOnKsqError(ksq_fp8_convert_weight(dt, weight.GetPtr<void>(), k, n, weight_fp8.GetPtr<void>(),
                                           weight_scale.GetPtr<float>(), stream.Get()),
                    "ksq_fp8_convert_weight");
  weight_fp8.weight_scales = &weight_scale;
  return Status();
}

Status MergeFp8QkvScales(Tensor& qkv_weight, const Tensor& q_scale, const Tensor& k_scale, const Tensor& v_scale,
                         size_t nq, size_t nk, size_t nv, bool per_channel, Tensor& merged_scale, int rank,
                         Stream& stream) {
  if (qkv_weight.shape.size() != 2 || qkv_weight.shape[0] != nq + nk + nv)
    KLLM_THROW("MergeFp8QkvScales: weight must be [nq + nk + nv, k].");
  CreateTensor(merged_scale, {per_channel ? nq + nk + nv : 1}, TYPE_FP32, rank, MEMORY_DEVICE);
  ThrowOnKsqError(
      ksq_fp8_merge_qkv_scales(per_channel ? KSQ_FP8_MERGE_PER_CHANNEL : KSQ_FP8_MERGE_MAX, q_scale.GetPtr<float>(),
                               k_scale.GetPtr<float>(), v_scale.GetPtr<float>(), nq, nk, nv, qkv_weight.GetPtr<void>(),
                               qkv_weight.shape[1], merged_scale.GetPtr<float>(), stream.Get()),
      "ksq_fp8_merge_qkv_scales");
  qkv_weight.weight_scales = &merged_scale;
  return Status();
}

template class Fp8MatMulLayer<float>;  // fp32 activations and results (KS/layers/nvidia/fp8_matmul_layer.cpp:69)
template class Fp8MatMulLayer<float16>;
template class Fp8MatMulLayer<bfloat16>;


}  // namespace ksana_llm
