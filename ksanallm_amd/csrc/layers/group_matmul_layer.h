// GroupMatMulLayer: the weight-only int4 group-quantized MatMul layer (GPTQ / AWQ), MI355X implementation.
// Interface and parameter pack of KS/layers/group_matmul_layer.h and KS/layers/nvidia/group_matmul_layer.cpp:13-169
// (KS = src/ksana_llm of the KsanaLLM tree); the arithmetic is behind the C ABI of ksq.h.
#pragma once

#include "base_layer.h"

namespace ksana_llm {

// layouts a 4-bit group-quantized weight can arrive in (see RepackGroupQuantWeight below)
enum GroupWeightLayout {
  GROUP_WEIGHT_GPTQ_INT32,
  GROUP_WEIGHT_AWQ_INT32,
  GROUP_WEIGHT_ROWMAJOR_INT4,
  GROUP_WEIGHT_CUTLASS_SM80,
  GROUP_WEIGHT_CUTLASS_SM90,
  GROUP_WEIGHT_MARLIN  // Marlin tiles; scales in Marlin order; qzeros (AWQ) as Marlin zero points
};

template <typename T, DataType WT>
class GroupMatMulLayer : public BaseLayer {
 public:
  // parameters, in this order: bool is_awq, bool is_gptq_desc, bool is_k_full, GroupQuantBackend backend,
  // size_t max_m, size_t max_n, size_t max_k, size_t groupsize, bool cutlass_use_gemv_cuda_core
  Status Init(const std::vector<std::any>& parameters, std::shared_ptr<Context> context, int rank) override;

  size_t GetWorkSpaceSize() override;

  // The reference times up to 105 tactics for every m here; the launch plan of this path is a closed-form function
  // of (m, n, k), so there is nothing to measure.
  Status Preprocess(const ModelConfig& model_config_) override;

  // input_tensors[0]: activations [m, k] T.  input_tensors[1]: weight in fragment order (ksq_w4a16_repack) whose
  // .scales points at the repacked scale/zero words; for a desc_act layer its .perm is the int32 [k] row order the
  // weight was repacked with (the activations' columns are gathered through it, as the reference's Marlin back end
  // does: LK/gptq_marlin/gptq_marlin.cu:380-392).  output_tensors[0]: [m, n] T (n/2 columns with the SiLU-mul
  // epilogue); shape and dtype are set here.
  Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) override;

  // Not in the reference, which runs these as layers of their own (KS/models/common/common_model.cpp:456-459,
  // 540-547): fold a bias row (kind = KSQ_EPILOGUE_BIAS, bias = T [n]) or SiLU(gate) * up of a fused, column
  // interleaved gate/up weight (KSQ_EPILOGUE_SILU_MUL) into the GEMM.  The bias tensor must outlive the layer.
  void SetEpilogue(int kind, const Tensor* bias = nullptr);

  // Which of the reference loader's CUTLASS layouts a weight is in when it reaches Forward without having been
  // repacked (its `.scales` still T [k/g, n], `.zeros` additive T or null): the loader's preprocess is architecture
  // dependent (LK/asymmetric_gemm/cutlass_preprocessors.cpp:504), so a loader carried over unchanged states which
  // one it ran.  GROUP_WEIGHT_CUTLASS_SM80 by default; a Marlin back end (Init) overrides this.  Such a weight is
  // converted once, at its first Forward: its bytes are rewritten in place into the fragment order and the combined
  // scale/zero words are kept by the library (ForgetAdoptedGroupQuantWeights frees them).
  void SetLoaderLayout(int group_weight_layout) { loader_layout_ = static_cast<GroupWeightLayout>(group_weight_layout); }

 private:
  void AdoptLoaderWeight(const Tensor& weight_tensor, void** weight, void** sz);
  GroupWeightLayout loader_layout_ = GROUP_WEIGHT_CUTLASS_SM80;
  bool is_awq_ = false;
  bool is_gptq_desc_ = false;
  bool is_k_full_ = true;
  GroupQuantBackend backend_ = CUTLASS_BACKEND;
  size_t max_m_ = 0, max_n_ = 0, max_k_ = 0;
  size_t groupsize_ = 128;
  bool cutlass_use_gemv_cuda_core_ = true;
  int epilogue_ = 0;
  const Tensor* bias_ = nullptr;
};

// Load-time half (replaces the CPU layout preprocess + scale / zero binding of QuantWeight::ConvertGroupTensor,
// KS/models/quant/quant_weight.cpp:530-536, 577-579, 632-636): repacks one checkpoint weight that is already on
// the device into fragment order and binds `weight.scales`.  `qzeros` may be null (GPTQ).  The tensors that
// `weight` and `weight_sz` end up owning are allocated here.
// GROUP_WEIGHT_CUTLASS_SM80 / _SM90: what the reference's own loader leaves in "*.weight" after
// CutlassPreprocessWeightsForMixedGemmWarpper (quant_weight.cpp:331-346) on those architectures, so an untouched
// loader can be followed by this call.  `perm` (int32 [k] on the device, from SortGptqGIdx) repacks a desc_act
// checkpoint with its rows grouped and is bound to weight.perm; `interleave_gate_up` repacks a fused [gate | up]
// weight with its column pairs interleaved for the SiLU-mul epilogue.
Status RepackGroupQuantWeight(GroupWeightLayout layout, const Tensor& qweight, const Tensor* qzeros, bool zeros_additive,
                              const Tensor& scales, size_t k, size_t n, size_t groupsize, Tensor& weight,
                              Tensor& weight_sz, int rank, Stream& stream, Tensor* perm = nullptr,
                              bool interleave_gate_up = false);

// Several checkpoint tensors that share K, side by side along N in one repacked weight: what the loader's concat of
// q_proj / k_proj / v_proj into query_key_value (and of gate_proj / up_proj) does before its repack
// (KS/models/quant/quant_weight.cpp:471-513), without the concatenated copy: column tiles are contiguous in the
// fragment order, so every part is repacked straight into its own range of the fused buffers.  Every part's width
// must be a multiple of 16.
struct GroupWeightPart {
  const Tensor* qweight;
  const Tensor* qzeros;  // nullptr = symmetric
  const Tensor* scales;
  size_t n;
};
Status RepackFusedGroupQuantWeight(GroupWeightLayout layout, const std::vector<GroupWeightPart>& parts,
                                   bool zeros_additive, size_t k, size_t groupsize, Tensor& weight, Tensor& weight_sz,
                                   int rank, Stream& stream);

// perm = stable argsort of a desc_act checkpoint's g_idx (MarlinSortGIdx, quant_weight.cpp:455-460), on the host.
// Throws unless every group has exactly `groupsize` rows.
Status SortGptqGIdx(const std::vector<int32_t>& g_idx, size_t groupsize, std::vector<int32_t>& perm);

// Frees the scale/zero words (and padded weights) of every loader-format weight that a GroupMatMulLayer converted at
// its first Forward; call it when the model's weights are released.
void ForgetAdoptedGroupQuantWeights(int rank);

}  // namespace ksana_llm
