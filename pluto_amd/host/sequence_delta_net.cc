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

// The reference differentiates through the whole history
// (sequence_delta_net.cc:482-600); that kernel chain is not part of this library.
StatusOr<BufferVec> SequenceDeltaNetLayer::bwd_impl(hip::Executor&, Span<const Buffer>,
                                                    BackwardState, LayerHooks*) {
  return UnimplementedError(
      "SequenceDeltaNetLayer backward is not implemented by the MI355X attention path");
}

}  // namespace pluto::llm
