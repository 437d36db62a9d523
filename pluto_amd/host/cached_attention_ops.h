// Single-token cached attention and the single-token gated delta-net state:
// the functions of src/llm/layers/util/cached_attention_ops.h:13-95 over the
// C ABI.  Pointers are contiguous device FP32 arrays exactly as in the
// reference; BF16 values are represented exactly in them.
#pragma once

#include <memory>

#include "pluto_amd/host/executor.h"
#include "pluto_amd/host/key_value_cache.h"

namespace pluto::llm::cached_attention_ops {

struct FullAttentionParameters {
  int query_heads = 24;
  int key_value_heads = 4;
  int head_dim = 256;
  int rotary_dim = 64;
  int capacity = 4096;
  float rms_norm_epsilon = 1e-6f;
  float rope_theta = 10000000.0f;
  bool round_to_bfloat16 = true;
};

pluto_hip_attention_params ToAbi(const FullAttentionParameters& parameters);

// Parameter limits, and the cache's Executor, KV shape and capacity must
// match.  A full cache is still compatible.  No GPU work.
Status ValidateCachedAttention(hip::Executor& executor, const FullAttentionParameters& parameters,
                               const KeyValueCache& cache);

// One token of batch-one causal attention against an externally owned cache,
// whose position is the only sequence counter.  q_gate [query_heads, 2,
// head_dim], k/v [key_value_heads, head_dim], q_norm/k_norm [head_dim]
// zero-centred; output [query_heads, head_dim] after sigmoid gating; optional
// probabilities [query_heads, position()+1].  Validates pointers and remaining
// capacity before GPU work and advances the cache once after every launch
// succeeded.  A kBFloat16HeadMajor cache requires round_to_bfloat16.
Status CachedAttentionStep(hip::Executor& executor, const FullAttentionParameters& parameters,
                           KeyValueCache& cache, const float* q_gate, const float* k,
                           const float* v, const float* q_norm, const float* k_norm,
                           float* output, float* probabilities = nullptr);

// The same step for caches.size() independent sequences in one set of
// launches: what a decoder step lifted from batch one (Model::Step,
// src/llm/qwen/model.cc:405-428) to a batch feeds the cached attention with.
// q_gate [batch, query_heads, 2, head_dim], k/v [batch, key_value_heads,
// head_dim], output [batch, query_heads, head_dim]; sequence s attends to
// caches[s] at that cache's own position.  Every cache is validated (and must
// have room) before any GPU work; all advance together after the launches
// succeeded.  No probabilities.
Status CachedAttentionStepBatch(hip::Executor& executor,
                                const FullAttentionParameters& parameters,
                                Span<KeyValueCache* const> caches, const float* q_gate,
                                const float* k, const float* v, const float* q_norm,
                                const float* k_norm, float* output);
// The batched step on bf16 activations: q_gate, k, v and output hold bf16
// elements, as the projections either side of the attention produce and take
// them (what QwenAttentionLayer::CachedForward does for one sequence without
// its casts).  The norm weights stay FP32.
Status CachedAttentionStepBatchBFloat16(hip::Executor& executor,
                                        const FullAttentionParameters& parameters,
                                        Span<KeyValueCache* const> caches, const void* q_gate,
                                        const void* k, const void* v, const float* q_norm,
                                        const float* k_norm, void* output);

struct DeltaNetParameters {
  int key_heads = 16;
  int value_heads = 48;
  int key_head_dim = 128;
  int value_head_dim = 128;
  int conv_kernel_dim = 4;
  float rms_norm_epsilon = 1e-6f;
  bool round_to_bfloat16 = true;
};

pluto_hip_delta_params ToAbi(const DeltaNetParameters& parameters);

// Single-token causal depthwise convolution + gated delta rule.  The recurrent
// matrix stays FP32 even when activation rounding is enabled.
class DeltaNetState final {
 public:
  DeltaNetState(const DeltaNetState&) = delete;
  DeltaNetState& operator=(const DeltaNetState&) = delete;
  // batch > 1: that many independent sequences, advanced together; every
  // activation of Step then carries a leading [batch] axis (the reference's
  // state is the batch-one case).
  static StatusOr<std::unique_ptr<DeltaNetState>> Create(hip::Executor& executor,
                                                         DeltaNetParameters parameters,
                                                         int batch = 1);
  int batch() const { return batch_; }

  // qkv packs [all Q, all K, all V]; z [value_heads, value_head_dim]; a, b,
  // a_log, dt_bias [value_heads]; conv_weight [qkv_channels, conv_kernel_dim]
  // oldest to newest; norm_weight [value_head_dim], a plain multiplier.
  // Output has z's shape, after RMSNorm and SiLU(z) gating.
  Status Step(const float* qkv, const float* z, const float* a, const float* b,
              const float* conv_weight, const float* a_log, const float* dt_bias,
              const float* norm_weight, float* output);
  // The same step on bf16 activations (qkv, z, a, b and output hold bf16
  // elements; weights and both states stay FP32): what DeltaNetLayer feeds it,
  // without the casts either side.  Output = the FP32 step's, rounded to bf16.
  Status StepBFloat16(const void* qkv, const void* z, const void* a, const void* b,
                      const float* conv_weight, const float* a_log, const float* dt_bias,
                      const float* norm_weight, void* output);
  Status Reset();
  // One sequence of the batch back to its initial (zero) state; the others keep
  // theirs.  Both states are laid out sequence by sequence.
  Status Reset(int sequence);

 private:
  DeltaNetState(hip::Executor& executor, DeltaNetParameters parameters, int batch,
                hip::Buffer convolution_state, hip::Buffer recurrent_state, hip::Buffer workspace)
      : executor_(executor), parameters_(parameters), batch_(batch),
        convolution_state_(std::move(convolution_state)),
        recurrent_state_(std::move(recurrent_state)), workspace_(std::move(workspace)) {}
  Status StepAs(int io_dtype, const void* qkv, const void* z, const void* a, const void* b,
                const float* conv_weight, const float* a_log, const float* dt_bias,
                const float* norm_weight, void* output);
  hip::Executor& executor_;
  DeltaNetParameters parameters_;
  int batch_;
  hip::Buffer convolution_state_;
  hip::Buffer recurrent_state_;
  hip::Buffer workspace_;  // convolved QKV and core output of one token
};

}  // namespace pluto::llm::cached_attention_ops
