#include "pluto_amd/host/sequence_delta_net.h"

#include <cmath>
#include <limits>

#include "pluto_amd/host/layer_util.h"

namespace pluto::llm {

SequenceDeltaNetLayer::SequenceDeltaNetLayer(
    hip::Executor& executor, cached_attention_ops::DeltaNetParameters p,
    std::shared_ptr<BlockParameter> convolution, std::shared_ptr<BlockParameter> a_log,
    std::shared_ptr<BlockParameter> dt_bias, std::shared_ptr<BlockParameter> norm,
    int sequence_length)
    : executor_(executor), parameters_(p), sequence_length_(sequence_length),
      parameters_owned_{std::move(convolution), std::move(a_log), std::move(dt_bias),
                        std::move(norm)},
      weights_{parameters_owned_[0]->value(), parameters_owned_[1]->value(),
               parameters_owned_[2]->value(), parameters_owned_[3]->value()} {
  const int64_t values = 1LL * p.value_heads * p.value_head_dim;
  input_types_ = {
      {DataType::BF16, {-2, sequence_length, 2LL * p.key_heads * p.key_head_dim + values}},
      {DataType::BF16, {-2, sequence_length, values}},
      {DataType::BF16, {-2, sequence_length, p.value_heads}},
      {DataType::BF16, {-2, sequence_length, p.value_heads}}};
  output_types_ = {{DataType::BF16, {-2, sequence_length, values}}};
}

// src/llm/layers/sequence_delta_net.cc:396-433
StatusOr<std::unique_ptr<SequenceDeltaNetLayer>> SequenceDeltaNetLayer::Create(
    hip::Executor& executor, cached_attention_ops::DeltaNetParameters p,
    std::shared_ptr<BlockParameter> convolution, std::shared_ptr<BlockParameter> a_log,
    std::shared_ptr<BlockParameter> dt_bias, std::shared_ptr<BlockParameter> norm,
    int sequence_length) {
  if (sequence_length < 1 || sequence_length > kMaximumSequenceLength || p.key_heads < 1 ||
      p.value_heads < 1 || p.value_heads % p.key_heads != 0 || p.key_head_dim < 1 ||
      p.key_head_dim > 128 || p.value_head_dim < 1 || p.value_head_dim > 256 ||
      p.conv_kernel_dim < 1 || p.conv_kernel_dim > 32 || !std::isfinite(p.rms_norm_epsilon) ||
      p.rms_norm_epsilon <= 0)
    return InvalidArgumentError("unsupported SequenceDeltaNetLayer shape");
  const int64_t channels =
      2LL * p.key_heads * p.key_head_dim + 1LL * p.value_heads * p.value_head_dim;
  if (channels * sequence_length > std::numeric_limits<int>::max() / 32)
    return InvalidArgumentError("SequenceDeltaNetLayer shape overflows");
  const std::shared_ptr<BlockParameter> parameters[] = {convolution, a_log, dt_bias, norm};
  const int64_t counts[] = {channels * p.conv_kernel_dim, p.value_heads, p.value_heads,
                            p.value_head_dim};
  for (int i = 0; i < 4; ++i) {
    if (!parameters[i] || parameters[i]->storage() != DataType::FP32)
      return InvalidArgumentError("DeltaNet parameters must be FP32");
    if (&parameters[i]->value().executor() != &executor ||
        parameters[i]->value().size_bytes() != static_cast<size_t>(counts[i]) * sizeof(float))
      return InvalidArgumentError("invalid DeltaNet buffer");
  }
  return std::unique_ptr<SequenceDeltaNetLayer>(
      new SequenceDeltaNetLayer(executor, p, std::move(convolution), std::move(a_log),
                                std::move(dt_bias), std::move(norm), sequence_length));
}

// src/llm/layers/sequence_delta_net.cc:435-480
StatusOr<FwdResult> SequenceDeltaNetLayer::fwd_impl(hip::Executor& executor,
                                                    Span<const Buffer> inputs,
                                                    LayerHooks*) const {
  if (&executor != &executor_ || inputs.size() != 4)
    return InvalidArgumentError("DeltaNet expects four inputs on its Executor");
  const auto& p = parameters_;
  const int t = sequence_length_;
  const int channels = 2 * p.key_heads * p.key_head_dim + p.value_heads * p.value_head_dim;
  const int output_width = p.value_heads * p.value_head_dim;
  const int widths[] = {channels, output_width, p.value_heads, p.value_heads};
  for (int i = 0; i < 4; ++i)
    if (&inputs[i].executor() != &executor ||
        inputs[i].size_bytes() != static_cast<size_t>(t) * widths[i] * 2)
      return InvalidArgumentError("invalid DeltaNet buffer");
  const pluto_hip_delta_params abi = cached_attention_ops::ToAbi(p);
  const size_t state_bytes =
      static_cast<size_t>(p.value_heads) * p.key_head_dim * p.value_head_dim * sizeof(float);
  ASSIGN_OR_RETURN(auto state_buffer, Buffer::Allocate(executor, state_bytes));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_memset_async(executor.stream(), state_buffer.data(), 0, state_bytes),
      "clear DeltaNet recurrent state"));
  const size_t workspace_bytes = pluto_hip_gdn_layer_workspace_bytes(&abi, 1, t);
  ASSIGN_OR_RETURN(auto workspace, Buffer::Allocate(executor, workspace_bytes));
  ASSIGN_OR_RETURN(auto output,
                   Buffer::Allocate(executor, static_cast<size_t>(t) * output_width * 2));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_gdn_layer_forward(executor.stream(), &abi, 1, t, inputs[0].data(),
                                  inputs[1].data(), inputs[2].data(), inputs[3].data(),
                                  static_cast<const float*>(weights_[0].data()),
                                  static_cast<const float*>(weights_[1].data()),
                                  static_cast<const float*>(weights_[2].data()),
                                  static_cast<const float*>(weights_[3].data()),
                                  static_cast<float*>(state_buffer.data()), output.data(),
                                  workspace.data(), workspace_bytes),
      "sequence DeltaNet forward"));
  BackwardState state;
  state.intermediates = {inputs[0], inputs[1], inputs[2], inputs[3], std::move(state_buffer)};
  return FwdResult{{std::move(output)}, std::move(state)};
}

// src/llm/layers/sequence_delta_net.cc:482-561.  The library's backward entry
// repeats the forward pass itself (keeping the states it needs in its
// workspace: one per 64-token chunk for 128 x 128 heads, one per token
// otherwise, where the reference saves every per-token state), so the saved
// state only supplies the four input handles.
StatusOr<BufferVec> SequenceDeltaNetLayer::bwd_impl(hip::Executor& executor,
                                                    Span<const Buffer> gradients,
                                                    BackwardState state, LayerHooks*) {
  if (&executor != &executor_ || gradients.size() != 1 || state.intermediates.size() != 5)
    return InvalidArgumentError("invalid DeltaNet backward state or gradient");
  const auto& p = parameters_;
  const int t = sequence_length_;
  if (t > kMaximumBackwardLength)
    return UnimplementedError(
        "SequenceDeltaNetLayer backward keeps one state per token and supports T<=65535");
  const size_t channels =
      2ull * p.key_heads * p.key_head_dim + 1ull * p.value_heads * p.value_head_dim;
  const size_t output_width = 1ull * p.value_heads * p.value_head_dim;
  const size_t rows = static_cast<size_t>(t);
  const auto& saved = state.intermediates;
  const size_t expected[] = {rows * channels * 2, rows * output_width * 2, rows * p.value_heads * 2,
                             rows * p.value_heads * 2};
  if (&gradients[0].executor() != &executor ||
      gradients[0].size_bytes() != rows * output_width * sizeof(float))
    return InvalidArgumentError(
        "SequenceDeltaNetLayer requires batch-one buffers of the declared sequence shape on its "
        "Executor");
  for (int i = 0; i < 4; ++i)
    if (&saved[i].executor() != &executor || saved[i].size_bytes() != expected[i])
      return InvalidArgumentError(
          "SequenceDeltaNetLayer requires batch-one buffers of the declared sequence shape on its "
          "Executor");
  ASSIGN_OR_RETURN(auto dqkv, Buffer::Allocate(executor, rows * channels * sizeof(float)));
  ASSIGN_OR_RETURN(auto dz, Buffer::Allocate(executor, rows * output_width * sizeof(float)));
  ASSIGN_OR_RETURN(auto da, Buffer::Allocate(executor, rows * p.value_heads * sizeof(float)));
  ASSIGN_OR_RETURN(auto db, Buffer::Allocate(executor, rows * p.value_heads * sizeof(float)));
  const pluto_hip_delta_params abi = cached_attention_ops::ToAbi(p);
  auto active_gradient = [](const std::shared_ptr<BlockParameter>& parameter) -> float* {
    return parameter->active() ? static_cast<float*>(parameter->gradient().data()) : nullptr;
  };
  float* const d_norm = active_gradient(parameters_owned_[3]);
  const size_t workspace_bytes =
      pluto_hip_gdn_layer_backward_workspace_bytes(&abi, t, d_norm != nullptr);
  ASSIGN_OR_RETURN(auto workspace, Buffer::Allocate(executor, workspace_bytes));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_gdn_layer_backward(
          executor.stream(), &abi, 1, t, saved[0].data(), saved[1].data(), saved[2].data(),
          saved[3].data(), static_cast<const float*>(weights_[0].data()),
          static_cast<const float*>(weights_[1].data()),
          static_cast<const float*>(weights_[2].data()),
          static_cast<const float*>(weights_[3].data()),
          static_cast<const float*>(gradients[0].data()), static_cast<float*>(dqkv.data()),
          static_cast<float*>(dz.data()), static_cast<float*>(da.data()),
          static_cast<float*>(db.data()), active_gradient(parameters_owned_[0]),
          active_gradient(parameters_owned_[1]), active_gradient(parameters_owned_[2]), d_norm,
          workspace.data(), workspace_bytes),
      "sequence DeltaNet backward"));
  return BufferVec{std::move(dqkv), std::move(dz), std::move(da), std::move(db)};
}

}  // namespace pluto::llm
