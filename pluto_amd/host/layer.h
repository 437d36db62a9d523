// Layer interface of the attention path, with the names and contracts of
// src/llm/layer.h:25-185 so that layers written against the reference compile
// against this header: DataType, ActivationType, BackwardState, FwdResult and
// the Layer base class whose public fwd/bwd own hook dispatch and the
// state-identity check.
#pragma once

#include <cstdint>
#include <string_view>
#include <utility>
#include <vector>

#include "pluto_amd/host/executor.h"
#include "pluto_amd/host/status.h"

namespace pluto::llm {

using Buffer = hip::Buffer;
using BufferVec = std::vector<Buffer>;

enum class DataType { FP16, BF16, FP8, FP32, INT32 };

// Physical dtype and logical dimensions of one forward input or output.  A
// leading -2 is the symbolic batch dimension; it equals only itself
// (src/llm/layer.h:33-81).
class ActivationType {
 public:
  static constexpr int64_t kBatchDimension = -2;
  ActivationType(DataType data_type, std::vector<int64_t> dimensions)
      : data_type_(data_type), dimensions_(std::move(dimensions)) {}
  DataType data_type() const { return data_type_; }
  Span<const int64_t> dimensions() const { return MakeConstSpan(dimensions_); }
  bool operator==(const ActivationType& other) const {
    return data_type_ == other.data_type_ && dimensions_ == other.dimensions_;
  }
  bool operator!=(const ActivationType& other) const { return !(*this == other); }
  Status Validate() const {
    for (size_t i = 0; i < dimensions_.size(); ++i)
      if (dimensions_[i] <= 0 && !(i == 0 && dimensions_[i] == kBatchDimension))
        return InvalidArgumentError(
            "activation dimensions must be positive, except leading batch (-2)");
    return OkStatus();
  }

 private:
  DataType data_type_;
  std::vector<int64_t> dimensions_;
};

// The FP16 compute policy keeps FP32 activations (src/llm/layer.h:86-88).
inline DataType ActivationDataType(DataType compute_type) {
  return compute_type == DataType::FP16 ? DataType::FP32 : compute_type;
}

class Layer;
struct LayerHooks;

// Saved forward state; `layer` identifies the producer and bwd() rejects a
// state from any other instance (src/llm/layer.h:96-105).
struct BackwardState {
  const Layer* layer = nullptr;
  BufferVec intermediates;
  std::vector<BackwardState> children;
};

struct FwdResult {
  BufferVec outputs;
  BackwardState state;
};

class Layer {
 public:
  virtual ~Layer() = default;
  virtual std::string_view name() const = 0;
  virtual Span<const ActivationType> input_types() const = 0;
  virtual Span<const ActivationType> output_types() const = 0;

  // State is published only with a successful output; an installed
  // activation_hook sees the outputs before they are published.
  StatusOr<FwdResult> fwd(hip::Executor& executor, Span<const Buffer> inputs,
                          LayerHooks* hooks = nullptr) const;
  // Rejects states that were not produced by this instance before any work;
  // an installed gradient_hook sees the FP32 output gradients first.
  StatusOr<BufferVec> bwd(hip::Executor& executor, Span<const Buffer> output_gradients,
                          BackwardState state, LayerHooks* hooks = nullptr);

  virtual Span<Buffer> weights() = 0;
  virtual Span<Buffer> gradients() { return {}; }
  virtual DataType output_type() const = 0;

 private:
  virtual StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                                       LayerHooks* hooks) const = 0;
  virtual StatusOr<BufferVec> bwd_impl(hip::Executor& executor,
                                       Span<const Buffer> output_gradients, BackwardState state,
                                       LayerHooks* hooks) = 0;
};

}  // namespace pluto::llm
