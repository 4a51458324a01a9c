// Fp8MatMulLayer: FP8 e4m3 MatMul layer, MI355X implementation.  Interface of KS/layers/fp8_matmul_layer.h and
// KS/layers/nvidia/fp8_matmul_layer.cpp:13-67 (KS = src/ksana_llm of the KsanaLLM tree).
#pragma once

#include "base_layer.h"

namespace ksana_llm {

template <typename T>
class Fp8MatMulLayer : public BaseLayer {
 public:
  // parameters: size_t max_m, size_t max_k
  Status Init(const std::vector<std::any>& parameters, std::shared_ptr<Context> context, int rank) override;

  // input_tensors[0]: activations [m, k] T.  input_tensors[1]: weight [n, k] e4m3 with .weight_scales (1 or n
  // floats; required) and optional .input_scales (static activation scale).  With one weight scale the activations
  // are quantized per tensor, as in the reference; with n weight scales they are quantized per token and the GEMM
  // applies per-token x per-channel scales.
  Status Forward(const std::vector<Tensor>& input_tensors, std::vector<Tensor>& output_tensors) override;

  size_t GetWorkSpaceSize(const int m, const int k);

  size_t GetWorkSpaceSize() override;

 private:
  int max_m_ = 0;
  int max_k_ = 0;
  size_t max_n_hint_ = 0;
};

}  // namespace ksana_llm
