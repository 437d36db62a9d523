// A rectangular projection: FullyConnectedLayer of
// src/llm/layers/fully_connected.h:20-112 on MI355X.
// Trainable projections have a bias, FP32 master parameters and FP32
// gradients.  Operands are multiplied as bfloat16 (BF16 policy) or IEEE half
// (FP16 policy, FP32 activations) and summed in FP32; widths need not be
// multiples of the compute tiles.  Each backward call overwrites the matrix
// and bias gradients, and reductions run in a fixed order, so repeated calls
// are bitwise stable.
// Imported projections share frozen, biasless, output-major checkpoint
// weights without copying them, take and give one BF16 token [1, 1, width],
// compute in FP32, and have no gradients: initialization is a failed
// precondition and backward is unimplemented.
#pragma once

#include <cstdint>
#include <memory>
#include <optional>

#include "pluto_amd/host/layer.h"

namespace pluto::llm {

// Physical storage of an imported checkpoint matrix
// (src/llm/layers/matrix_common.h:10).  FP8 matrices come with FP32 block
// scales [ceil(output_dim/128), ceil(input_dim/128)].
enum class MatrixStorage { kBFloat16, kFloat32, kFp8E4M3 };
StatusOr<size_t> MatrixElementBytes(MatrixStorage storage);

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

  // Imports a biasless [output_dim, input_dim] matrix without copying it.  The
  // FP8 path quantizes its input in independent groups of 128 elements.
  static StatusOr<std::unique_ptr<FullyConnectedLayer>> Create(
      hip::Executor& executor, Buffer weights, MatrixStorage storage, int input_dim,
      int output_dim, std::optional<Buffer> scales = std::nullopt);

  // Bound of the imported single-token kernels; not a trainable-layer limit.
  static constexpr int kMaximumDimension = 1048576;

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
  // Engaged for an imported matrix; weights() then holds the matrix and, for
  // FP8, its block scales.
  std::optional<MatrixStorage> imported_storage() const { return imported_storage_; }

 private:
  FullyConnectedLayer(hip::Executor& executor, int input_dim, int output_dim, DataType data_type,
                      BufferVec weights, BufferVec gradients, int sequence_length);
  FullyConnectedLayer(hip::Executor& executor, int input_dim, int output_dim, BufferVec weights,
                      MatrixStorage storage);
  StatusOr<FwdResult> ImportedForward(hip::Executor& executor, Span<const Buffer> inputs) const;
  StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const override;
  StatusOr<BufferVec> bwd_impl(hip::Executor& executor, Span<const Buffer> output_gradients,
                               BackwardState state, LayerHooks* hooks) override;

  hip::Executor& executor_;
  int input_dim_, output_dim_;
  DataType output_type_;
  BufferVec weights_, gradients_;
  // Engaged only for the frozen output-major checkpoint representation.
  std::optional<MatrixStorage> imported_storage_;
  std::vector<ActivationType> input_types_, output_types_;
};

}  // namespace pluto::llm
