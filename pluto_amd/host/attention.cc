#include "pluto_amd/host/attention.h"

#include <limits>

#include "pluto_amd/host/layer_hooks.h"
#include "pluto_amd/host/layer_util.h"

namespace pluto::llm {
namespace {

int StorageCode(DataType type) { return type == DataType::BF16 ? PLUTO_HIP_BF16 : PLUTO_HIP_F32; }

// The optional quadratic tensor must be addressable before it is allocated
// (src/llm/layers/attention.cc:40-61).
StatusOr<size_t> ProbabilityBytes(int rows, int context_length, int num_heads) {
  size_t bytes = static_cast<size_t>(rows);
  for (size_t factor : {static_cast<size_t>(num_heads), static_cast<size_t>(context_length),
                        sizeof(float)}) {
    if (bytes > std::numeric_limits<size_t>::max() / factor)
      return ResourceExhaustedError("attention probabilities tensor byte size overflows size_t");
    bytes *= factor;
  }
  return bytes;
}

}  // namespace

AttentionLayer::AttentionLayer(hip::Executor& executor, int context_length, int num_heads,
                               int embedding_dim, DataType data_type)
    : executor_(executor), context_length_(context_length), num_heads_(num_heads),
      embedding_dim_(embedding_dim), output_type_(data_type) {
  const DataType storage = ActivationDataType(data_type);
  input_types_.emplace_back(storage, std::vector<int64_t>{ActivationType::kBatchDimension,
                                                          context_length, 3LL * embedding_dim});
  output_types_.emplace_back(storage, std::vector<int64_t>{ActivationType::kBatchDimension,
                                                           context_length, 1LL * embedding_dim});
}

// src/llm/layers/attention.cc:400-416
StatusOr<std::unique_ptr<AttentionLayer>> AttentionLayer::Create(hip::Executor& executor,
                                                                 int context_length, int num_heads,
                                                                 int embedding_dim,
                                                                 DataType data_type) {
  RETURN_IF_ERROR(internal::ValidateComputeType(data_type));
  if (context_length <= 0 || num_heads <= 0 || embedding_dim <= 0)
    return InvalidArgumentError("attention dimensions must all be positive");
  if (embedding_dim % num_heads != 0)
    return InvalidArgumentError("embedding_dim must be divisible by num_heads");
  return std::unique_ptr<AttentionLayer>(
      new AttentionLayer(executor, context_length, num_heads, embedding_dim, data_type));
}

// src/llm/layers/attention.cc:418-507
StatusOr<FwdResult> AttentionLayer::fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                                             LayerHooks* hooks) const {
  RETURN_IF_ERROR(internal::ValidateExecutor(executor_, executor, "AttentionLayer"));
  if (inputs.size() != 1) return InvalidArgumentError("AttentionLayer fwd expects packed Q/K/V");
  ASSIGN_OR_RETURN(int rows,
                   internal::ActivationRows(executor, inputs[0], 3 * embedding_dim_, output_type_,
                                            "attention packed Q/K/V input"));
  if (rows % context_length_ != 0)
    return InvalidArgumentError("attention rows must be divisible by context_length");
  const bool inspect = hooks != nullptr && static_cast<bool>(hooks->attention_probabilities_hook);
  size_t probability_bytes = 0;
  if (inspect) {
    ASSIGN_OR_RETURN(probability_bytes, ProbabilityBytes(rows, context_length_, num_heads_));
  }
  ASSIGN_OR_RETURN(auto output,
                   Buffer::Allocate(executor, static_cast<size_t>(rows) * embedding_dim_ *
                                                  internal::ActivationElementBytes(output_type_)));
  const size_t stats_bytes = static_cast<size_t>(rows) * num_heads_ * sizeof(float);
  ASSIGN_OR_RETURN(auto maxima, Buffer::Allocate(executor, stats_bytes));
  ASSIGN_OR_RETURN(auto normalizers, Buffer::Allocate(executor, stats_bytes));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_mha_forward(executor.stream(), StorageCode(output_type_), inputs[0].data(), rows,
                            context_length_, num_heads_, embedding_dim_, output.data(),
                            static_cast<float*>(maxima.data()),
                            static_cast<float*>(normalizers.data())),
      "attention forward launch"));
  if (inspect) {
    ASSIGN_OR_RETURN(auto probabilities, Buffer::Allocate(executor, probability_bytes));
    RETURN_IF_ERROR(hip::HipStatus(
        pluto_hip_mha_probabilities(executor.stream(), StorageCode(output_type_), inputs[0].data(),
                                    static_cast<const float*>(maxima.data()),
                                    static_cast<const float*>(normalizers.data()), rows,
                                    context_length_, num_heads_, embedding_dim_,
                                    static_cast<float*>(probabilities.data())),
        "attention probabilities launch"));
    const ActivationType type(DataType::FP32, {rows / context_length_, num_heads_,
                                               context_length_, context_length_});
    RETURN_IF_ERROR(hooks->attention_probabilities_hook(executor, name(), type, probabilities));
  }
  BackwardState state;
  state.intermediates = {inputs[0], output, std::move(maxima), std::move(normalizers)};
  return FwdResult{{std::move(output)}, std::move(state)};
}

// src/llm/layers/attention.cc:509-596
StatusOr<BufferVec> AttentionLayer::bwd_impl(hip::Executor& executor,
                                             Span<const Buffer> output_gradients,
                                             BackwardState state, LayerHooks*) {
  RETURN_IF_ERROR(internal::ValidateExecutor(executor_, executor, "AttentionLayer"));
  if (output_gradients.size() != 1 || state.intermediates.size() != 4)
    return InvalidArgumentError("AttentionLayer bwd received an incompatible gradient or state");
  ASSIGN_OR_RETURN(int rows, internal::MatrixRows(executor, output_gradients[0], embedding_dim_,
                                                  "attention output gradient"));
  if (rows % context_length_ != 0)
    return InvalidArgumentError("attention gradient rows must be divisible by context_length");
  const size_t element = internal::ActivationElementBytes(output_type_);
  RETURN_IF_ERROR(internal::ValidateBuffer(executor, state.intermediates[0],
                                           static_cast<size_t>(rows) * 3 * embedding_dim_ * element,
                                           "attention saved Q/K/V"));
  RETURN_IF_ERROR(internal::ValidateBuffer(executor, state.intermediates[1],
                                           static_cast<size_t>(rows) * embedding_dim_ * element,
                                           "attention saved output"));
  const size_t stats_bytes = static_cast<size_t>(rows) * num_heads_ * sizeof(float);
  RETURN_IF_ERROR(internal::ValidateBuffer(executor, state.intermediates[2], stats_bytes,
                                           "attention saved maxima"));
  RETURN_IF_ERROR(internal::ValidateBuffer(executor, state.intermediates[3], stats_bytes,
                                           "attention saved normalizers"));
  ASSIGN_OR_RETURN(auto gradient,
                   Buffer::Allocate(executor, static_cast<size_t>(rows) * 3 * embedding_dim_ *
                                                  sizeof(float)));
  // The reference allocates `deltas` here (attention.cc:544); the workspace
  // holds it together with the scratch of the matrix-core path.
  const size_t workspace_bytes = pluto_hip_mha_backward_workspace_bytes(
      StorageCode(output_type_), rows, context_length_, num_heads_, embedding_dim_);
  ASSIGN_OR_RETURN(auto workspace, Buffer::Allocate(executor, workspace_bytes));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_mha_backward(executor.stream(), StorageCode(output_type_),
                             state.intermediates[0].data(), state.intermediates[1].data(),
                             static_cast<const float*>(output_gradients[0].data()),
                             static_cast<const float*>(state.intermediates[2].data()),
                             static_cast<const float*>(state.intermediates[3].data()), rows,
                             context_length_, num_heads_, embedding_dim_,
                             static_cast<float*>(gradient.data()), workspace.data(),
                             workspace_bytes),
      "attention backward launch"));
  return BufferVec{std::move(gradient)};
}

}  // namespace pluto::llm
