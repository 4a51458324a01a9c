// Test-side stand-in for the caller of the quantized MatMul layers.
//
// In KsanaLLM the layers are created by MatMulLayerFactory<T> (src/ksana_llm/layers/matmul_layer_factory.h), which
// stays in KsanaLLM unchanged when this library is wired in; nothing of it is product code here.  The tests only need
// something that plays its part towards a layer, and this harness is that, written for the tests:
//   * it turns (weight name, model config) into the layer's parameter pack -- the order of the pack is the layers'
//     contract (GroupMatMulLayer::Init: is_awq, is_gptq_desc, is_k_full, backend, max_m, max_n, max_k, groupsize,
//     cutlass_use_gemv_cuda_core; Fp8MatMulLayer::Init: max_m, max_k) and is what the tests want to exercise;
//   * it drives a new layer through Init, GetWorkSpaceSize, SetWorkSpaceBuffer and Preprocess, in that order;
//   * it owns the one workspace tensor that every layer it made shares, grown to the largest request.
#pragma once

#include <any>
#include <memory>
#include <sstream>
#include <string>
#include <type_traits>
#include <vector>

#include "base_layer.h"
#include "fp8_matmul_layer.h"
#include "group_matmul_layer.h"

namespace ksana_llm {

template <typename T>
class LayerHarness {
 public:
  LayerHarness(const ModelConfig& config, std::shared_ptr<Context> context, int rank = 0)
      : config_(config), context_(std::move(context)), rank_(rank) {}

  ~LayerHarness() {
    if (workspace_) DestroyTensor(*workspace_, rank_);
  }

  // A layer for the named weight, as a model would ask for it.  Group-quantized checkpoints (GPTQ / AWQ) get a
  // GroupMatMulLayer whose K and N come from the model dimensions by projection name (a repacked weight tensor no
  // longer has a meaningful shape); an e4m3 weight tensor gets an Fp8MatMulLayer sized by its own [n, k] shape.
  std::shared_ptr<BaseLayer> ForWeight(BaseWeight& weights, const std::string& weight_name, DataType io_type) {
    const QuantMode method = config_.quant_config.method;
    if (config_.is_quant && (method == QUANT_GPTQ || method == QUANT_AWQ)) {
      size_t k = 0, n = 0;
      bool whole_k = true;
      if (ProjectionShape(weight_name, &k, &n, &whole_k)) {
        const std::vector<std::any> pack = {method == QUANT_AWQ,
                                            config_.quant_config.desc_act,
                                            whole_k,
                                            config_.quant_config.backend,
                                            config_.max_scheduler_token_num,
                                            n,
                                            k,
                                            config_.quant_config.group_size,
                                            true};
        return Make(TYPE_I4_GROUP, io_type, pack);
      }
    }
    const Tensor w = weights.GetModelWeights(weight_name);
    if (w.dtype == TYPE_FP8_E4M3) {
      const std::vector<std::any> pack = {config_.max_scheduler_token_num, w.shape[1]};
      return Make(TYPE_FP8_E4M3, io_type, pack);
    }
    KLLM_THROW("no quantized MatMul layer for weight " + weight_name);
  }

  // A layer of the class that goes with `weight_type`, from an explicit parameter pack.
  std::shared_ptr<BaseLayer> Make(DataType weight_type, DataType io_type, const std::vector<std::any>& pack) {
    std::shared_ptr<BaseLayer> layer;
    // fp16 and bf16 for both layers; fp32 for the FP8 layer only (the reference registers no fp32 group layer, and
    // its float instantiation of that GEMM is empty)
    if constexpr (std::is_same<T, float>::value) {
      if (io_type == TYPE_FP32 && weight_type == TYPE_FP8_E4M3) layer = std::make_shared<Fp8MatMulLayer<T>>();
    } else {
      const bool io_ok = io_type == TYPE_FP16 || io_type == TYPE_BF16;
      if (io_ok && weight_type == TYPE_I4_GROUP) layer = std::make_shared<GroupMatMulLayer<T, TYPE_I4_GROUP>>();
      if (io_ok && weight_type == TYPE_FP8_E4M3) layer = std::make_shared<Fp8MatMulLayer<T>>();
    }
    if (!layer) {
      std::ostringstream os;
      os << "no layer class for weight type " << weight_type << " with activations of type " << io_type;
      KLLM_THROW(os.str());
    }
    layer->Init(pack, context_, rank_);
    GrowWorkspace(layer->GetWorkSpaceSize());
    layer->SetWorkSpaceBuffer(workspace_);
    layer->Preprocess(config_);
    return layer;
  }

  std::shared_ptr<Tensor> Workspace() const { return workspace_; }

 private:
  // K x N of a projection under tensor parallelism: column-parallel projections keep the whole K and a slice of N,
  // row-parallel ones (o_proj, down_proj) a slice of K and the whole N.
  bool ProjectionShape(const std::string& name, size_t* k, size_t* n, bool* whole_k) const {
    const size_t tp = config_.tensor_para_size, hidden = config_.hidden_units;
    const size_t inter = config_.type == "qwen" ? config_.inter_size / 2 : config_.inter_size;
    const size_t qkv = config_.size_per_head * (config_.head_num + 2 * config_.num_key_value_heads);
    auto has = [&](const char* part) { return name.find(part) != std::string::npos; };
    if (has("query_key_value")) return *k = hidden, *n = qkv / tp, *whole_k = true, true;
    if (has("gate_proj") || has("up_proj")) return *k = hidden, *n = inter / tp, *whole_k = true, true;
    if (has("o_proj")) return *k = hidden / tp, *n = hidden, *whole_k = false, true;
    if (has("down_proj")) return *k = inter / tp, *n = hidden, *whole_k = false, true;
    return false;
  }

  void GrowWorkspace(size_t bytes) {
    if (bytes == 0 || (workspace_ && workspace_->GetTotalBytes() >= bytes)) return;
    if (workspace_) DestroyTensor(*workspace_, rank_);
    else workspace_ = std::make_shared<Tensor>();
    CreateTensor(*workspace_, {bytes}, TYPE_INT8, rank_, MEMORY_DEVICE);
  }

  ModelConfig config_;
  std::shared_ptr<Context> context_;
  int rank_;
  std::shared_ptr<Tensor> workspace_;
};

}  // namespace ksana_llm
