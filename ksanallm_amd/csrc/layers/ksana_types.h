// The vocabulary the quantized MatMul layers of ksana_llm speak, reduced to what this path touches, so that the
// layer shims in this directory keep the reference's names, argument meaning and error behaviour and compile
// outside the ksana_llm tree.  Inside the tree a maintainer includes the real headers instead (same names):
//   Status      KS/utils/status.h:20-80          DataType    KS/utils/device_types.h:103-124
//   TensorT     KS/utils/common_tensor.h:28-116  ContextT    KS/utils/common_context.h:21-97
//   QuantConfig KS/utils/environment.h:33-58     KLLM_THROW  KS/utils/logger.h:123
// (KS = src/ksana_llm of the KsanaLLM tree.)
#pragma once

#include <any>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace ksana_llm {

#define KLLM_THROW(msg) throw std::runtime_error(std::string(msg))

enum RetCode { RET_SUCCESS = 0, RET_INVALID_ARGUMENT = 1, RET_RUNTIME = 2 };

class Status {
 public:
  Status() {}
  explicit Status(RetCode code, const std::string& message = "") {
    if (code != RET_SUCCESS) state_ = std::make_shared<State>(State{code, message});
  }
  bool OK() const { return state_ == nullptr; }
  const std::string& GetMessage() const {
    static const std::string empty;
    return OK() ? empty : state_->message;
  }
  RetCode GetCode() const { return OK() ? RET_SUCCESS : state_->code; }

 private:
  struct State {
    RetCode code;
    std::string message;
  };
  std::shared_ptr<State> state_;
};

#define STATUS_CHECK_FAILURE(status)    \
  do {                                  \
    auto&& _status = (status);          \
    if (!_status.OK()) {                \
      KLLM_THROW(_status.GetMessage()); \
    }                                   \
  } while (0)

enum DataType {
  TYPE_INVALID, TYPE_BOOL, TYPE_UINT8, TYPE_UINT16, TYPE_UINT32, TYPE_UINT64, TYPE_INT8, TYPE_INT16, TYPE_INT32,
  TYPE_INT64, TYPE_BF16, TYPE_FP16, TYPE_FP32, TYPE_FP64, TYPE_BYTES, TYPE_FP8_E4M3, TYPE_I4_GROUP, TYPE_FP8_E5M2,
  TYPE_VOID, TYPE_POINTER
};

inline size_t GetTypeSize(DataType t) {
  switch (t) {
    case TYPE_BOOL: case TYPE_UINT8: case TYPE_INT8: case TYPE_BYTES: case TYPE_FP8_E4M3: case TYPE_FP8_E5M2:
      return 1;
    case TYPE_UINT16: case TYPE_INT16: case TYPE_BF16: case TYPE_FP16:
      return 2;
    case TYPE_UINT32: case TYPE_INT32: case TYPE_FP32:
      return 4;
    case TYPE_UINT64: case TYPE_INT64: case TYPE_FP64: case TYPE_POINTER:
      return 8;
    default:
      return 0;
  }
}

enum MemoryDevice { MEMORY_HOST, MEMORY_DEVICE };

// Element tags standing where the reference uses half / __nv_bfloat16 as the layer's template argument.
struct float16 {
  uint16_t bits;
};
struct bfloat16 {
  uint16_t bits;
};

template <typename T>
struct TypeTraits;
template <>
struct TypeTraits<float16> {
  static constexpr DataType kDataType = TYPE_FP16;
};
template <>
struct TypeTraits<bfloat16> {
  static constexpr DataType kDataType = TYPE_BF16;
};
template <>
struct TypeTraits<float> {  // Fp8MatMulLayer<float> only (KS/layers/matmul_layer_factory.h:38)
  static constexpr DataType kDataType = TYPE_FP32;
};

// Contiguous tensor over a raw pointer.  The side pointers are non-owning, as in the reference's weights map.
class Tensor {
 public:
  MemoryDevice device = MEMORY_DEVICE;
  DataType dtype = TYPE_INVALID;
  std::vector<size_t> shape;

  Tensor* scales = nullptr;
  Tensor* zeros = nullptr;
  Tensor* g_idx = nullptr;
  Tensor* perm = nullptr;
  Tensor* input_scales = nullptr;
  Tensor* weight_scales = nullptr;

  void* refer_ptr = nullptr;

  Tensor() {}
  Tensor(MemoryDevice dev, DataType dt, const std::vector<size_t>& shp, void* ptr)
      : device(dev), dtype(dt), shape(shp), refer_ptr(ptr) {}

  size_t GetElementNumber() const {
    if (shape.empty()) return 0;
    size_t n = 1;
    for (size_t s : shape) n *= s;
    return n;
  }
  size_t GetTotalBytes() const { return GetElementNumber() * GetTypeSize(dtype); }

  template <typename TP>
  TP* GetPtr() const {
    return reinterpret_cast<TP*>(refer_ptr);
  }
};

// Allocation helpers with the reference's names (KS/utils/memory_utils.h); device memory comes from hipMalloc.
Status CreateTensor(Tensor& tensor, const std::vector<size_t>& shape, DataType dtype, int rank, MemoryDevice device);
Status DestroyTensor(Tensor& tensor, int rank);

class Stream {
 public:
  explicit Stream(void* s = nullptr) : stream_(s) {}
  void*& Get() { return stream_; }  // hipStream_t

 private:
  void* stream_;
};

class Context {
 public:
  explicit Context(size_t tensor_parallel_size = 1) : compute_streams_(tensor_parallel_size) {}
  std::vector<Stream>& GetComputeStreams() { return compute_streams_; }

 private:
  std::vector<Stream> compute_streams_;
};

enum QuantMode { QUANT_NONE, QUANT_GPTQ, QUANT_AWQ, QUANT_FP8_E4M3, MOE_QUANT_NONE };
enum GroupQuantBackend { CUTLASS_BACKEND, MARLIN_BACKEND };

struct QuantConfig {
  QuantMode method = QUANT_NONE;
  size_t bits = 4;
  size_t group_size = 128;
  bool desc_act = false;
  GroupQuantBackend backend = CUTLASS_BACKEND;
  bool is_checkpoint_fp8_serialized = false;
  bool is_activation_scheme_static = false;
};

struct ModelConfig {
  std::string type;
  bool is_quant = false;
  QuantConfig quant_config;
  size_t hidden_units = 0;
  size_t inter_size = 0;
  size_t head_num = 0;
  size_t num_key_value_heads = 0;
  size_t size_per_head = 0;
  size_t tensor_para_size = 1;
  size_t max_batch_size = 128;
  size_t max_scheduler_token_num = 4096;
};

// Just enough of BaseWeight for a caller that looks a weight tensor up by name, as KsanaLLM's layer factory does.
class BaseWeight {
 public:
  virtual ~BaseWeight() {}
  virtual Tensor GetModelWeights(const std::string& weight_name) = 0;
};

}  // namespace ksana_llm
