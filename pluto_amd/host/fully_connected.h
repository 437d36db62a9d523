// A rectangular projection with a bias, FP32 master parameters and FP32
// gradients: the trainable FullyConnectedLayer of
// src/llm/layers/fully_connected.h:20-112 on MI355X.  Operands are multiplied
// as bfloat16 (BF16 policy) or IEEE half (FP16 policy, FP32 activations) and
// summed in FP32; widths need not be multiples of the compute tiles.  Each
// backward call overwrites the matrix and bias gradients, and reductions run
// in a fixed order, so repeated calls are bitwise stable.  The frozen imported
// single-token path (fully_connected.h:38-46) is not part of this library.
#pragma once

#include <cstdint>
#include <memory>

#include "pluto_amd/host/layer.h"

namespace pluto::llm {

class FullyConnectedLayer final : public Layer {
 public:
  std::string_view name() const override { return "FullyConnectedLayer"; }

  // sequence_length is activation rows per sample, not the batch size; it only
  // shapes the activation signatures, the kernels flatten batch and sequence.
  static StatusOr<std::unique_ptr<FullyConnectedLayer>> Create(hip::Executor& executor,
                                                               int input_dim, int output_dim,
                                                               DataType data_type,
                                                               int sequence_length = 1);
  static StatusOr<std::unique_ptr<FullyConnectedLayer>> Create(hip::Executor& executor,
                                                               int model_width, DataType data_type,
                                                               int sequence_length = 1) {
    return Create(executor, model_width, model_width, data_type, sequence_length);
  }

  // A scaled identity on the available diagonal; the bias is left as it is.
  Status InitializeIdentity(float scale = 1.0f);
  // mt19937_64(seed) through normal_distribution<float>, row-major.
  Status InitializeNormal(float standard_deviation, uint64_t seed);

  // {matrix [input_dim, output_dim], bias [output_dim]}, FP32.
  Span<Buffer> weights() override { return MakeSpan(weights_); }
  Span<Buffer> gradients() override { return MakeSpan(gradients_); }
  DataType output_type() const override { return output_type_; }
  Span<const ActivationType> input_types() const override { return MakeConstSpan(input_types_); }
  Span<const ActivationType> output_types() const override { return MakeConstSpan(output_types_); }

  int input_dim() const { return input_dim_; }
  int output_dim() const { return output_dim_; }

 private:
  FullyConnectedLayer(hip::Executor& executor, int input_dim, int output_dim, DataType data_type,
                      BufferVec weights, BufferVec gradients, int sequence_length);
  StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const override;
  StatusOr<BufferVec> bwd_impl(hip::Executor& executor, Span<const Buffer> output_gradients,
                               BackwardState state, LayerHooks* hooks) override;

  hip::Executor& executor_;
  int input_dim_, output_dim_;
  DataType output_type_;
  BufferVec weights_, gradients_;
  std::vector<ActivationType> input_types_, output_types_;
};

}  // namespace pluto::llm
