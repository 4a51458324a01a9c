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

  // Not in the reference: fold a bias row (KSQ_EPILOGUE_BIAS, bias = T [n]) or SiLU(gate) * up of a row-interleaved
  // gate/up weight (KSQ_EPILOGUE_SILU_MUL; output [m, n/2]) into the GEMM.  The bias tensor must outlive the layer.
  void SetEpilogue(int kind, const Tensor* bias = nullptr);

  size_t GetWorkSpaceSize() override;

 private:
  int max_m_ = 0;
  int max_k_ = 0;
  size_t max_n_hint_ = 0;
  int epilogue_ = 0;
  const Tensor* bias_ = nullptr;
};

// Load-time half (replaces the device work of QuantWeight::ConvertFp8E4m3Tensor and BindFp8E4m3ScaleOfQkvWeight,
// KS/models/quant/quant_weight.cpp:685-726, 816-897).
//
// ConvertFp8Weight: weight [k, n] T on the device -> weight_fp8 [n, k] e4m3 + weight_scale (1 float, or n floats
// with per_channel), both allocated here; weight_fp8.weight_scales is bound.
Status ConvertFp8Weight(const Tensor& weight, bool per_channel, Tensor& weight_fp8, Tensor& weight_scale, int rank,
                        Stream& stream);
// MergeFp8QkvScales: qkv_weight [nq + nk + nv, k] e4m3 whose three row ranges carry the scalar scales q/k/v_scale.
// per_channel = false is the reference: one scale = their maximum and the ranges are requantised in place;
// per_channel = true writes one scale per row and leaves the bytes alone.  merged_scale is allocated here and bound
// to qkv_weight.weight_scales.
Status MergeFp8QkvScales(Tensor& qkv_weight, const Tensor& q_scale, const Tensor& k_scale, const Tensor& v_scale,
                         size_t nq, size_t nk, size_t nv, bool per_channel, Tensor& merged_scale, int rank,
                         Stream& stream);

}  // namespace ksana_llm
