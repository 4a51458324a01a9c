// GroupMatMulLayer: the weight-only int4 group-quantized MatMul layer (GPTQ / AWQ), MI355X implementation.
// Interface and parameter pack of KS/layers/group_matmul_layer.h and KS/layers/nvidia/group_matmul_layer.cpp:13-169
// (KS = src/ksana_llm of the KsanaLLM tree); the arithmetic is behind the C ABI of ksq.h.
#pragma once

#include "base_layer.h"

namespace ksana_llm {

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
  // .scales points at the repacked scale/zero words.  output_tensors[0]: [m, n] T; shape and dtype are set here.
  Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) override;

 private:
  bool is_awq_ = false;
  bool is_gptq_desc_ = false;
  bool is_k_full_ = true;
  GroupQuantBackend backend_ = CUTLASS_BACKEND;
  size_t max_m_ = 0, max_n_ = 0, max_k_ = 0;
  size_t groupsize_ = 128;
  bool cutlass_use_gemv_cuda_core_ = true;
};

// Load-time half (replaces the CPU layout preprocess + scale / zero binding of QuantWeight::ConvertGroupTensor,
// KS/models/quant/quant_weight.cpp:530-536, 577-579, 632-636): repacks one checkpoint weight that is already on
// the device into fragment order and binds `weight.scales`.  `qzeros` may be null (GPTQ).  The tensors that
// `weight` and `weight_sz` end up owning are allocated here.
enum GroupWeightLayout { GROUP_WEIGHT_GPTQ_INT32, GROUP_WEIGHT_AWQ_INT32, GROUP_WEIGHT_ROWMAJOR_INT4 };
Status RepackGroupQuantWeight(GroupWeightLayout layout, const Tensor& qweight, const Tensor* qzeros, bool zeros_additive,
                              const Tensor& scales, size_t k, size_t n, size_t groupsize, Tensor& weight,
                              Tensor& weight_sz, int rank, Stream& stream);

}  // namespace ksana_llm
