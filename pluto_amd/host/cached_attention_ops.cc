#include "pluto_amd/host/cached_attention_ops.h"

#include <cmath>
#include <limits>
#include <vector>

namespace pluto::llm::cached_attention_ops {
namespace {

StatusOr<hip::Buffer> AllocateFloats(hip::Executor& executor, size_t count) {
  if (count > std::numeric_limits<size_t>::max() / sizeof(float))
    return ResourceExhaustedError("attention allocation size overflows");
  return hip::Buffer::Allocate(executor, count * sizeof(float));
}

}  // namespace

pluto_hip_attention_params ToAbi(const FullAttentionParameters& p) {
  pluto_hip_attention_params abi{};
  abi.query_heads = p.query_heads;
  abi.key_value_heads = p.key_value_heads;
  abi.head_dim = p.head_dim;
  abi.rotary_dim = p.rotary_dim;
  abi.capacity = p.capacity;
  abi.rms_norm_epsilon = p.rms_norm_epsilon;
  abi.rope_theta = p.rope_theta;
  abi.round_to_bfloat16 = p.round_to_bfloat16 ? 1 : 0;
  return abi;
}

pluto_hip_delta_params ToAbi(const DeltaNetParameters& p) {
  pluto_hip_delta_params abi{};
  abi.key_heads = p.key_heads;
  abi.value_heads = p.value_heads;
  abi.key_head_dim = p.key_head_dim;
  abi.value_head_dim = p.value_head_dim;
  abi.conv_kernel_dim = p.conv_kernel_dim;
  abi.rms_norm_epsilon = p.rms_norm_epsilon;
  abi.round_to_bfloat16 = p.round_to_bfloat16 ? 1 : 0;
  return abi;
}

// src/llm/layers/util/cached_attention_ops.cc:283-306
Status ValidateCachedAttention(hip::Executor& executor, const FullAttentionParameters& p,
                               const KeyValueCache& cache) {
  const pluto_hip_attention_params abi = ToAbi(p);
  if (pluto_hip_attention_params_validate(&abi) != 0)
    return InvalidArgumentError("invalid full-attention dimensions or parameters");
  if (&cache.executor() != &executor)
    return InvalidArgumentError("attention cache belongs to a different Executor");
  if (cache.capacity() != p.capacity || cache.key_value_heads() != p.key_value_heads ||
      cache.head_dim() != p.head_dim)
    return InvalidArgumentError("attention cache shape or capacity does not match parameters");
  if (cache.storage() == KeyValueCache::Storage::kBFloat16HeadMajor && !p.round_to_bfloat16)
    return InvalidArgumentError("a bfloat16 attention cache requires round_to_bfloat16");
  return OkStatus();
}

// src/llm/layers/util/cached_attention_ops.cc:308-353
Status CachedAttentionStep(hip::Executor& executor, const FullAttentionParameters& p,
                           KeyValueCache& cache, const float* q_gate, const float* k,
                           const float* v, const float* q_norm, const float* k_norm,
                           float* output, float* probabilities) {
  RETURN_IF_ERROR(ValidateCachedAttention(executor, p, cache));
  if (!q_gate || !k || !v || !q_norm || !k_norm || !output)
    return InvalidArgumentError("attention requires non-null device pointers");
  if (cache.position() >= cache.capacity())
    return ResourceExhaustedError("full-attention cache capacity reached");
  const pluto_hip_attention_params abi = ToAbi(p);
  const int position = cache.position();
  const pluto_hip_kv_cache_view view = cache.view();
  // Stream-ordered scratch for the prepared query and the split-K partials,
  // like the reference's temporary query storage (:321-323).
  const size_t workspace_bytes = pluto_hip_gqa_decode_workspace_bytes(&abi, 1, &position, 0);
  ASSIGN_OR_RETURN(auto workspace, hip::Buffer::Allocate(executor, workspace_bytes));
  float* const probability_rows[1] = {probabilities};
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_gqa_decode(executor.stream(), &abi, 1, PLUTO_HIP_F32, q_gate, k, v, q_norm, k_norm,
                           &position, &view, output, probabilities ? probability_rows : nullptr, 0,
                           workspace.data(), workspace_bytes),
      "Qwen full attention"));
  return cache.Advance();
}

namespace {

Status StepBatchAs(int io_dtype, hip::Executor& executor, const FullAttentionParameters& p,
                   Span<KeyValueCache* const> caches, const void* q_gate, const void* k,
                   const void* v, const float* q_norm, const float* k_norm, void* output) {
  if (caches.empty()) return InvalidArgumentError("attention batch must not be empty");
  if (!q_gate || !k || !v || !q_norm || !k_norm || !output)
    return InvalidArgumentError("attention requires non-null device pointers");
  std::vector<int> positions;
  std::vector<pluto_hip_kv_cache_view> views;
  for (KeyValueCache* cache : caches) {
    if (cache == nullptr) return InvalidArgumentError("attention requires a cache per sequence");
    RETURN_IF_ERROR(ValidateCachedAttention(executor, p, *cache));
    if (cache->position() >= cache->capacity())
      return ResourceExhaustedError("full-attention cache capacity reached");
    for (size_t other = 0; other < views.size(); ++other)
      if (caches[other] == cache)
        return InvalidArgumentError("a cache serves one sequence of the batch");
    positions.push_back(cache->position());
    views.push_back(cache->view());
  }
  const pluto_hip_attention_params abi = ToAbi(p);
  const int batch = static_cast<int>(caches.size());
  const size_t workspace_bytes =
      pluto_hip_gqa_decode_workspace_bytes(&abi, batch, positions.data(), 0);
  ASSIGN_OR_RETURN(auto workspace, hip::Buffer::Allocate(executor, workspace_bytes));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_gqa_decode(executor.stream(), &abi, batch, io_dtype, q_gate, k, v, q_norm,
                           k_norm, positions.data(), views.data(), output, nullptr, 0,
                           workspace.data(), workspace_bytes),
      "Qwen full attention"));
  for (KeyValueCache* cache : caches) RETURN_IF_ERROR(cache->Advance());
  return OkStatus();
}

}  // namespace

Status CachedAttentionStepBatch(hip::Executor& executor, const FullAttentionParameters& p,
                                Span<KeyValueCache* const> caches, const float* q_gate,
                                const float* k, const float* v, const float* q_norm,
                                const float* k_norm, float* output) {
  return StepBatchAs(PLUTO_HIP_F32, executor, p, caches, q_gate, k, v, q_norm, k_norm, output);
}

Status CachedAttentionStepBatchBFloat16(hip::Executor& executor, const FullAttentionParameters& p,
                                        Span<KeyValueCache* const> caches, const void* q_gate,
                                        const void* k, const void* v, const float* q_norm,
                                        const float* k_norm, void* output) {
  return StepBatchAs(PLUTO_HIP_BF16, executor, p, caches, q_gate, k, v, q_norm, k_norm, output);
}

// src/llm/layers/util/cached_attention_ops.cc:369-399
StatusOr<std::unique_ptr<DeltaNetState>> DeltaNetState::Create(hip::Executor& executor,
                                                               DeltaNetParameters p, int batch) {
  if (batch <= 0) return InvalidArgumentError("DeltaNet batch must be positive");
  if (p.key_heads <= 0 || p.value_heads <= 0 || p.value_heads % p.key_heads != 0 ||
      p.key_head_dim <= 0 || p.key_head_dim > 128 || p.value_head_dim <= 0 ||
      p.value_head_dim > 256 || p.conv_kernel_dim <= 0 || p.conv_kernel_dim > 32 ||
      !std::isfinite(p.rms_norm_epsilon) || p.rms_norm_epsilon <= 0.0f)
    return InvalidArgumentError("invalid DeltaNet dimensions or parameters");
  const size_t channels = 2 * static_cast<size_t>(p.key_heads) * p.key_head_dim +
                          static_cast<size_t>(p.value_heads) * p.value_head_dim;
  if (channels > static_cast<size_t>(std::numeric_limits<int>::max()) / p.conv_kernel_dim)
    return ResourceExhaustedError("DeltaNet dimensions exceed indexing limit");
  const size_t n = static_cast<size_t>(batch);
  ASSIGN_OR_RETURN(auto convolution, AllocateFloats(executor, n * channels * p.conv_kernel_dim));
  ASSIGN_OR_RETURN(auto recurrence,
                   AllocateFloats(executor, n * p.value_heads * p.key_head_dim * p.value_head_dim));
  const pluto_hip_delta_params abi = ToAbi(p);
  ASSIGN_OR_RETURN(auto workspace,
                   hip::Buffer::Allocate(executor,
                                         pluto_hip_gdn_step_batch_workspace_bytes(&abi, batch)));
  std::unique_ptr<DeltaNetState> result(new DeltaNetState(
      executor, p, batch, std::move(convolution), std::move(recurrence), std::move(workspace)));
  RETURN_IF_ERROR(result->Reset());
  return result;
}

// src/llm/layers/util/cached_attention_ops.cc:401-431
Status DeltaNetState::Step(const float* qkv, const float* z, const float* a, const float* b,
                           const float* conv_weight, const float* a_log, const float* dt_bias,
                           const float* norm_weight, float* output) {
  return StepAs(PLUTO_HIP_F32, qkv, z, a, b, conv_weight, a_log, dt_bias, norm_weight, output);
}

Status DeltaNetState::StepBFloat16(const void* qkv, const void* z, const void* a, const void* b,
                                   const float* conv_weight, const float* a_log,
                                   const float* dt_bias, const float* norm_weight, void* output) {
  return StepAs(PLUTO_HIP_BF16, qkv, z, a, b, conv_weight, a_log, dt_bias, norm_weight, output);
}

Status DeltaNetState::StepAs(int io_dtype, const void* qkv, const void* z, const void* a,
                             const void* b, const float* conv_weight, const float* a_log,
                             const float* dt_bias, const float* norm_weight, void* output) {
  if (!qkv || !z || !a || !b || !conv_weight || !a_log || !dt_bias || !norm_weight || !output)
    return InvalidArgumentError("DeltaNet requires non-null device pointers");
  const pluto_hip_delta_params abi = ToAbi(parameters_);
  return hip::HipStatus(
      pluto_hip_gdn_step_batch(executor_.stream(), &abi, batch_, io_dtype,
                               static_cast<float*>(convolution_state_.data()),
                               static_cast<float*>(recurrent_state_.data()), qkv, z, a, b,
                               conv_weight, a_log, dt_bias, norm_weight, output, workspace_.data(),
                               workspace_.size_bytes()),
      "Qwen gated delta step");
}

// src/llm/layers/util/cached_attention_ops.cc:433-443
Status DeltaNetState::Reset() {
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_memset_async(executor_.stream(), convolution_state_.data(), 0,
                             convolution_state_.size_bytes()),
      "reset Qwen convolution state"));
  return hip::HipStatus(pluto_hip_memset_async(executor_.stream(), recurrent_state_.data(), 0,
                                               recurrent_state_.size_bytes()),
                        "reset Qwen recurrent state");
}

Status DeltaNetState::Reset(int sequence) {
  if (sequence < 0 || sequence >= batch_)
    return InvalidArgumentError(StrCat("no sequence ", sequence, " in a state of ", batch_));
  for (hip::Buffer* state : {&convolution_state_, &recurrent_state_}) {
    const size_t each = state->size_bytes() / batch_;
    RETURN_IF_ERROR(hip::HipStatus(
        pluto_hip_memset_async(executor_.stream(),
                               static_cast<char*>(state->data()) + each * sequence, 0, each),
        "reset one sequence of the Qwen delta-net state"));
  }
  return OkStatus();
}

}  // namespace pluto::llm::cached_attention_ops
