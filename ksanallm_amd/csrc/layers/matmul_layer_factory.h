// MatMulLayerFactory for the quantized MatMul layers: selection by (weight_type, input_type, output_type,
// quant_mode), K / N derived from the weight name, one shared INT8 workspace grown to the largest request, and the
// Init -> GetWorkSpaceSize -> SetWorkSpaceBuffer -> Preprocess sequence of
// KS/layers/matmul_layer_factory.h:26-49, 60-108, 152-182 (KS = src/ksana_llm of the KsanaLLM tree).  The
// unquantized MatMulLayer and the MoE layer of the reference are other paths and are not registered here.
#pragma once

#include <map>
#include <tuple>

#include "base_layer.h"
#include "fp8_matmul_layer.h"
#include "group_matmul_layer.h"

namespace ksana_llm {

template <typename T>
class MatMulLayerFactory {
 public:
  typedef std::shared_ptr<BaseLayer> (MatMulLayerFactory<T>::*BuildLayerFunc)();
  MatMulLayerFactory(std::shared_ptr<Tensor>& workspace_buffer, const ModelConfig& model_config, const int rank,
                     std::shared_ptr<Context> context) {
    context_ = context;
    rank_ = rank;
    model_config_ = model_config;
    workspace_buffer_ = workspace_buffer;

    builder_map_[{TYPE_FP8_E4M3, TYPE_FP16, TYPE_FP16, QUANT_FP8_E4M3}] =
        &MatMulLayerFactory<T>::template BuildLayer<Fp8MatMulLayer<T>>;
    builder_map_[{TYPE_FP8_E4M3, TYPE_BF16, TYPE_BF16, QUANT_FP8_E4M3}] =
        &MatMulLayerFactory<T>::template BuildLayer<Fp8MatMulLayer<T>>;
    // the reference registers the fp16 key only although it instantiates the layer for bf16 too
    // (matmul_layer_factory.h:45-48 vs nvidia/group_matmul_layer.cpp:171-175); bf16 is registered here as well
    builder_map_[{TYPE_I4_GROUP, TYPE_FP16, TYPE_FP16, QUANT_GPTQ}] =
        &MatMulLayerFactory<T>::template BuildLayer<GroupMatMulLayer<T, TYPE_I4_GROUP>>;
    builder_map_[{TYPE_I4_GROUP, TYPE_FP16, TYPE_FP16, QUANT_AWQ}] =
        &MatMulLayerFactory<T>::template BuildLayer<GroupMatMulLayer<T, TYPE_I4_GROUP>>;
    builder_map_[{TYPE_I4_GROUP, TYPE_BF16, TYPE_BF16, QUANT_GPTQ}] =
        &MatMulLayerFactory<T>::template BuildLayer<GroupMatMulLayer<T, TYPE_I4_GROUP>>;
    builder_map_[{TYPE_I4_GROUP, TYPE_BF16, TYPE_BF16, QUANT_AWQ}] =
        &MatMulLayerFactory<T>::template BuildLayer<GroupMatMulLayer<T, TYPE_I4_GROUP>>;
  }
  ~MatMulLayerFactory() {
    if (workspace_buffer_) {
      Tensor& tensor = *workspace_buffer_;
      DestroyTensor(tensor, rank_);
    }
  }
  template <typename ClassT>
  std::shared_ptr<BaseLayer> BuildLayer() {
    return std::make_shared<ClassT>();
  }

  std::shared_ptr<BaseLayer> AutoCreateLayer(std::shared_ptr<BaseWeight> base_weight, std::string weight_name,
                                             DataType weight_type, DataType input_type, DataType output_type,
                                             const std::vector<std::any>& init_params) {
    (void)weight_type;
    (void)init_params;
    if (model_config_.is_quant &&
        (model_config_.quant_config.method == QUANT_GPTQ || model_config_.quant_config.method == QUANT_AWQ)) {
      size_t hidden_size = model_config_.hidden_units;
      size_t inter_size = model_config_.inter_size;
      if (model_config_.type == "qwen") {
        inter_size /= 2;
      }
      size_t tp = model_config_.tensor_para_size;
      size_t qkv_size = model_config_.size_per_head * (model_config_.head_num + 2 * model_config_.num_key_value_heads);
      // the repacked weight no longer carries n / k in its shape: they come from the model config, by name
      std::map<std::string, std::tuple<size_t, size_t, bool>> kn_pairs;
      kn_pairs["query_key_value"] = std::make_tuple(hidden_size, qkv_size / tp, true);
      kn_pairs["o_proj"] = std::make_tuple(hidden_size / tp, hidden_size, false);
      kn_pairs["gate_proj"] = std::make_tuple(hidden_size, inter_size / tp, true);
      kn_pairs["up_proj"] = kn_pairs["gate_proj"];
      kn_pairs["down_proj"] = std::make_tuple(inter_size / tp, hidden_size, false);
      for (const auto& kn : kn_pairs) {
        if (weight_name.find(kn.first) != std::string::npos) {
          std::vector<std::any> group_matmul_param;
          group_matmul_param.push_back(static_cast<bool>(model_config_.quant_config.method == QUANT_AWQ));
          group_matmul_param.push_back(static_cast<bool>(model_config_.quant_config.desc_act));
          group_matmul_param.push_back(static_cast<bool>(std::get<2>(kn.second)));
          group_matmul_param.push_back(static_cast<GroupQuantBackend>(model_config_.quant_config.backend));
          group_matmul_param.push_back(model_config_.max_scheduler_token_num);
          group_matmul_param.push_back(std::get<1>(kn.second));
          group_matmul_param.push_back(std::get<0>(kn.second));
          group_matmul_param.push_back(model_config_.quant_config.group_size);
          group_matmul_param.push_back(true);
          return CreateLayer(TYPE_I4_GROUP, input_type, output_type, group_matmul_param, QUANT_GPTQ);
        }
      }
    }
    if (base_weight->GetModelWeights(weight_name).dtype == TYPE_FP8_E4M3) {
      std::vector<std::any> fp8_matmul_params;
      fp8_matmul_params.push_back(model_config_.max_scheduler_token_num);
      // weight is [n, k], k is shape[1]
      fp8_matmul_params.push_back(base_weight->GetModelWeights(weight_name).shape[1]);
      return CreateLayer(TYPE_FP8_E4M3, input_type, output_type, fp8_matmul_params, QUANT_FP8_E4M3);
    }
    KLLM_THROW("Not support weight " + weight_name + ": only the quantized MatMul layers are built here.");
  }

  std::shared_ptr<BaseLayer> CreateLayer(DataType weight_type, DataType input_type, DataType output_type,
                                         const std::vector<std::any>& init_params, QuantMode quant_mode = QUANT_NONE) {
    auto it = builder_map_.find({weight_type, input_type, output_type, quant_mode});
    if (it != builder_map_.end()) {
      std::shared_ptr<BaseLayer> layer = (this->*(it->second))();
      layer->Init(init_params, context_, rank_);
      size_t workspace_size = layer->GetWorkSpaceSize();
      if (workspace_buffer_ == nullptr && workspace_size > 0) {
        workspace_buffer_ = std::make_shared<Tensor>();
        Tensor& tensor = *workspace_buffer_;
        CreateTensor(tensor, {workspace_size}, DataType::TYPE_INT8, rank_, MemoryDevice::MEMORY_DEVICE);
      } else if (workspace_buffer_ && workspace_buffer_->GetTotalBytes() < workspace_size) {
        Tensor& tensor = *workspace_buffer_;
        DestroyTensor(tensor, rank_);
        CreateTensor(tensor, {workspace_size}, DataType::TYPE_INT8, rank_, MemoryDevice::MEMORY_DEVICE);
      }
      layer->SetWorkSpaceBuffer(workspace_buffer_);

      layer->Preprocess(model_config_);

      return layer;
    } else {
      std::ostringstream os;
      os << "Not support weight_type " << weight_type << ", input_type " << input_type << ", output_type "
         << output_type << ", quant_mode " << quant_mode << ".";
      KLLM_THROW(os.str());
    }
  }

  std::shared_ptr<Tensor> GetWorkSpaceBuffer() { return workspace_buffer_; }

 private:
  std::shared_ptr<Context> context_;
  int rank_;
  std::shared_ptr<Tensor> workspace_buffer_ = nullptr;
  ModelConfig model_config_;

  std::map<std::tuple<DataType, DataType, DataType, QuantMode>, BuildLayerFunc> builder_map_;
};

}  // namespace ksana_llm
