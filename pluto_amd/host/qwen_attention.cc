#include "pluto_amd/host/qwen_attention.h"

#include <cmath>
#include <optional>

#include "pluto_amd/host/layer_hooks.h"
#include "pluto_amd/host/layer_util.h"

namespace pluto::llm {

QwenAttentionLayer::QwenAttentionLayer(hip::Executor& executor, FullAttentionParameters p,
                                       std::shared_ptr<BlockParameter> q_norm,
                                       std::shared_ptr<BlockParameter> k_norm,
                                       int sequence_length, KeyValueCache* cache)
    : executor_(executor), parameters_(p), sequence_length_(sequence_length), cache_(cache),
      q_norm_(std::move(q_norm)), k_norm_(std::move(k_norm)),
      weights_{q_norm_->value(), k_norm_->value()} {
  const int64_t batch = ActivationType::kBatchDimension;
  input_types_ = {
      {DataType::BF16, {batch, sequence_length, 2LL * p.query_heads * p.head_dim}},
      {DataType::BF16, {batch, sequence_length, 1LL * p.key_value_heads * p.head_dim}},
      {DataType::BF16, {batch, sequence_length, 1LL * p.key_value_heads * p.head_dim}}};
  output_types_ = {{DataType::BF16, {batch, sequence_length, 1LL * p.query_heads * p.head_dim}}};
}

// src/llm/layers/qwen_attention.cc:290-335
StatusOr<std::unique_ptr<QwenAttentionLayer>> QwenAttentionLayer::Create(
    hip::Executor& executor, FullAttentionParameters p, std::shared_ptr<BlockParameter> q_norm,
    std::shared_ptr<BlockParameter> k_norm, int sequence_length, KeyValueCache* cache) {
  if (cache) {
    if (sequence_length != 1)
      return InvalidArgumentError("cached Qwen attention requires sequence_length == 1");
    if (p.query_heads <= 0 || p.key_value_heads <= 0 || p.head_dim <= 0)
      return InvalidArgumentError("QwenAttentionLayer dimensions must be positive");
    const int64_t query_width = 1LL * p.query_heads * p.head_dim;
    const int64_t key_width = 1LL * p.key_value_heads * p.head_dim;
    if (query_width > kMaximumDimension / 2 || key_width > kMaximumDimension)
      return InvalidArgumentError(
          "QwenAttentionLayer activation exceeds the layer dimension limit");
    RETURN_IF_ERROR(cached_attention_ops::ValidateCachedAttention(executor, p, *cache));
  } else {
    // Sequence execution does not use capacity: only its explicit sequence
    // length sizes the work.
    if (p.query_heads <= 0 || p.query_heads > 256 || p.key_value_heads <= 0 ||
        p.query_heads % p.key_value_heads || p.head_dim <= 0 || p.head_dim > 256 ||
        p.rotary_dim <= 0 || p.rotary_dim > p.head_dim || p.rotary_dim % 2 ||
        sequence_length <= 0 || sequence_length > kMaximumSequenceLength ||
        !(p.rms_norm_epsilon > 0) || !std::isfinite(p.rms_norm_epsilon) ||
        !(p.rope_theta > 0) || !std::isfinite(p.rope_theta))
      return InvalidArgumentError(
          "sequence Qwen attention requires valid GQA dimensions, D<=256 and 1<=T<=65535");
  }
  for (const auto& norm : {q_norm, k_norm})
    if (!norm || norm->storage() != DataType::FP32 ||
        norm->elements() != static_cast<size_t>(p.head_dim) ||
        &norm->value().executor() != &executor)
      return InvalidArgumentError(
          "Qwen attention norms must be FP32 head-width parameters on its Executor");
  return std::unique_ptr<QwenAttentionLayer>(new QwenAttentionLayer(
      executor, p, std::move(q_norm), std::move(k_norm), sequence_length, cache));
}

// src/llm/layers/qwen_attention.cc:337-349
StatusOr<std::unique_ptr<QwenAttentionLayer>> QwenAttentionLayer::Create(
    hip::Executor& executor, FullAttentionParameters parameters, Buffer q_norm, Buffer k_norm,
    int sequence_length, KeyValueCache* cache) {
  ASSIGN_OR_RETURN(auto query_parameter,
                   BlockParameter::Create(executor, std::move(q_norm), DataType::FP32));
  ASSIGN_OR_RETURN(auto key_parameter,
                   BlockParameter::Create(executor, std::move(k_norm), DataType::FP32));
  return Create(executor, parameters, std::move(query_parameter), std::move(key_parameter),
                sequence_length, cache);
}

// src/llm/layers/qwen_attention.cc:351-360
StatusOr<FwdResult> QwenAttentionLayer::fwd_impl(hip::Executor& executor,
                                                 Span<const Buffer> inputs,
                                                 LayerHooks* hooks) const {
  if (&executor != &executor_)
    return InvalidArgumentError("QwenAttentionLayer used with a different Executor");
  if (cache_) return CachedForward(executor, inputs, hooks);
  return SequenceForward(executor, inputs, hooks);
}

// src/llm/layers/qwen_attention.cc:362-369
StatusOr<BufferVec> QwenAttentionLayer::bwd_impl(hip::Executor& executor,
                                                 Span<const Buffer> gradients,
                                                 BackwardState state, LayerHooks*) {
  if (cache_)
    return UnimplementedError("QwenAttentionLayer with a KV cache supports inference only");
  return SequenceBackward(executor, gradients, std::move(state));
}

// src/llm/layers/qwen_attention.cc:371-412.  The decode kernels read and write
// bf16 directly, so the three ToFloat launches and the ToBFloat16 launch of
// the reference disappear.
StatusOr<FwdResult> QwenAttentionLayer::CachedForward(hip::Executor& executor,
                                                      Span<const Buffer> inputs,
                                                      LayerHooks* hooks) const {
  const auto& p = parameters_;
  const int output_width = p.query_heads * p.head_dim;
  const int counts[] = {2 * output_width, p.key_value_heads * p.head_dim,
                        p.key_value_heads * p.head_dim};
  RETURN_IF_ERROR(internal::ValidateBFloat16Inputs(executor, inputs, counts));
  RETURN_IF_ERROR(cached_attention_ops::ValidateCachedAttention(executor, p, *cache_));
  if (cache_->position() >= cache_->capacity())
    return ResourceExhaustedError("full-attention cache capacity reached");
  ASSIGN_OR_RETURN(auto output,
                   Buffer::Allocate(executor, static_cast<size_t>(output_width) * 2));
  std::optional<Buffer> probabilities;
  const int position = cache_->position();
  const int length = position + 1;
  if (hooks && hooks->attention_probabilities_hook) {
    ASSIGN_OR_RETURN(probabilities,
                     Buffer::Allocate(executor, static_cast<size_t>(p.query_heads) * length *
                                                    sizeof(float)));
  }
  const pluto_hip_attention_params abi = cached_attention_ops::ToAbi(p);
  const pluto_hip_kv_cache_view view = cache_->view();
  const size_t workspace_bytes = pluto_hip_gqa_decode_workspace_bytes(&abi, 1, &position, 0);
  ASSIGN_OR_RETURN(auto workspace, Buffer::Allocate(executor, workspace_bytes));
  float* const probability_rows[1] = {
      probabilities ? static_cast<float*>(probabilities->data()) : nullptr};
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_gqa_decode(executor.stream(), &abi, 1, PLUTO_HIP_BF16, inputs[0].data(),
                           inputs[1].data(), inputs[2].data(),
                           static_cast<const float*>(weights_[0].data()),
                           static_cast<const float*>(weights_[1].data()), &position, &view,
                           output.data(), probabilities ? probability_rows : nullptr, 0,
                           workspace.data(), workspace_bytes),
      "Qwen full attention"));
  RETURN_IF_ERROR(cache_->Advance());
  if (probabilities) {
    // One query and `length` keys, all causally visible.
    const ActivationType type(DataType::FP32, {1, p.query_heads, 1, length});
    RETURN_IF_ERROR(hooks->attention_probabilities_hook(executor, name(), type, *probabilities));
  }
  return FwdResult{{std::move(output)}, {}};
}

// src/llm/layers/qwen_attention.cc:414-448
StatusOr<FwdResult> QwenAttentionLayer::SequenceForward(hip::Executor& executor,
                                                        Span<const Buffer> inputs,
                                                        LayerHooks* hooks) const {
  const auto& p = parameters_;
  const int t = sequence_length_, d = p.head_dim, qh = p.query_heads, kh = p.key_value_heads;
  const size_t qn = static_cast<size_t>(t) * qh * d, kn = static_cast<size_t>(t) * kh * d;
  const size_t expected[] = {4 * qn, 2 * kn, 2 * kn};
  if (inputs.size() != 3)
    return InvalidArgumentError("sequence attention expects batch-one buffers on its Executor");
  for (int i = 0; i < 3; ++i)
    if (&inputs[i].executor() != &executor || inputs[i].size_bytes() != expected[i])
      return InvalidArgumentError("sequence attention expects batch-one buffers on its Executor");
  pluto_hip_attention_params abi = cached_attention_ops::ToAbi(p);
  abi.capacity = t;  // the private K/V scratch holds exactly this sequence
  // K/V scratch in the layout the kernels stream: bf16 head-major while values
  // are bf16 representable, FP32 token-major otherwise.
  pluto_hip_kv_cache_view view{};
  const size_t element = p.round_to_bfloat16 ? 2 : sizeof(float);
  ASSIGN_OR_RETURN(auto keys, Buffer::Allocate(executor, kn * element));
  ASSIGN_OR_RETURN(auto values, Buffer::Allocate(executor, kn * element));
  view.keys = keys.data();
  view.values = values.data();
  if (p.round_to_bfloat16) {
    view.dtype = PLUTO_HIP_BF16;
    view.token_stride = d;
    view.head_stride = 1LL * t * d;
  } else {
    view.dtype = PLUTO_HIP_F32;
    view.token_stride = 1LL * kh * d;
    view.head_stride = d;
  }
  const size_t workspace_bytes = pluto_hip_gqa_prefill_workspace_bytes(&abi, t);
  ASSIGN_OR_RETURN(auto workspace, Buffer::Allocate(executor, workspace_bytes));
  ASSIGN_OR_RETURN(auto output, Buffer::Allocate(executor, 2 * qn));
  ASSIGN_OR_RETURN(auto lse, Buffer::Allocate(executor, static_cast<size_t>(t) * qh * 4));
  // What the backward pass would otherwise recompute (the attention output
  // before the gate and its row statistics), where the library keeps it; an
  // empty buffer stands for "recompute".
  const size_t saved_bytes = pluto_hip_gqa_prefill_saved_bytes(&abi, t, view.dtype);
  ASSIGN_OR_RETURN(auto saved, Buffer::Allocate(executor, saved_bytes));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_gqa_prefill(executor.stream(), &abi, t, 0, inputs[0].data(), inputs[1].data(),
                            inputs[2].data(), static_cast<const float*>(weights_[0].data()),
                            static_cast<const float*>(weights_[1].data()), &view, output.data(),
                            static_cast<float*>(lse.data()),
                            saved_bytes ? saved.data() : nullptr, workspace.data(),
                            workspace_bytes),
      "sequence full attention forward"));
  if (hooks && hooks->attention_probabilities_hook) {
    ASSIGN_OR_RETURN(auto probabilities,
                     Buffer::Allocate(executor, static_cast<size_t>(t) * t * qh * sizeof(float)));
    RETURN_IF_ERROR(hip::HipStatus(
        pluto_hip_gqa_prefill_probabilities(executor.stream(), &abi, t, 0, &view, workspace.data(),
                                            workspace_bytes,
                                            static_cast<float*>(probabilities.data())),
        "sequence attention probabilities"));
    RETURN_IF_ERROR(hooks->attention_probabilities_hook(
        executor, name(), ActivationType(DataType::FP32, {1, qh, t, t}), probabilities));
  }
  BackwardState state;
  state.intermediates = {inputs[0], inputs[1], inputs[2], std::move(keys), std::move(values),
                         std::move(lse), std::move(saved)};
  return FwdResult{{std::move(output)}, std::move(state)};
}

// src/llm/layers/qwen_attention.cc:450-499.  The library's backward entry
// recomputes what the forward pass derived from the inputs except for the
// attention output and its row statistics, which it takes from the saved
// block when forward could fill one: the three input handles and that block
// are what is used of the saved state.
StatusOr<BufferVec> QwenAttentionLayer::SequenceBackward(hip::Executor& executor,
                                                         Span<const Buffer> gradients,
                                                         BackwardState state) {
  if (&executor != &executor_ || state.intermediates.size() != 7)
    return InvalidArgumentError("sequence attention backward Executor/state mismatch");
  const auto& p = parameters_;
  const int t = sequence_length_, d = p.head_dim, qh = p.query_heads, kh = p.key_value_heads;
  const size_t qn = static_cast<size_t>(t) * qh * d, kn = static_cast<size_t>(t) * kh * d;
  if (gradients.size() != 1 || &gradients[0].executor() != &executor ||
      gradients[0].size_bytes() != 4 * qn)
    return InvalidArgumentError("sequence attention expects batch-one buffers on its Executor");
  const auto& s = state.intermediates;
  pluto_hip_attention_params abi = cached_attention_ops::ToAbi(p);
  abi.capacity = t;
  ASSIGN_OR_RETURN(auto dqg, Buffer::Allocate(executor, 2 * qn * sizeof(float)));
  ASSIGN_OR_RETURN(auto dk, Buffer::Allocate(executor, kn * sizeof(float)));
  ASSIGN_OR_RETURN(auto dv, Buffer::Allocate(executor, kn * sizeof(float)));
  const bool q_active = q_norm_->active(), k_active = k_norm_->active();
  const size_t workspace_bytes =
      pluto_hip_gqa_prefill_backward_workspace_bytes(&abi, t, q_active, k_active);
  ASSIGN_OR_RETURN(auto workspace, Buffer::Allocate(executor, workspace_bytes));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_gqa_prefill_backward(
          executor.stream(), &abi, t, s[0].data(), s[1].data(), s[2].data(),
          static_cast<const float*>(weights_[0].data()),
          static_cast<const float*>(weights_[1].data()),
          static_cast<const float*>(gradients[0].data()),
          s[6].size_bytes() ? s[6].data() : nullptr, static_cast<float*>(dqg.data()),
          static_cast<float*>(dk.data()), static_cast<float*>(dv.data()),
          q_active ? static_cast<float*>(q_norm_->gradient().data()) : nullptr,
          k_active ? static_cast<float*>(k_norm_->gradient().data()) : nullptr, workspace.data(),
          workspace_bytes),
      "sequence full attention backward"));
  return BufferVec{std::move(dqg), std::move(dk), std::move(dv)};
}

}  // namespace pluto::llm
