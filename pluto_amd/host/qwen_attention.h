// QwenAttentionLayer, the class of src/llm/layers/qwen_attention.h:11-101 for
// MI355X: grouped-query attention of one sequence with an RMS norm on every
// query and key head, rotary embedding on the leading rotary_dim channels, a
// causal softmax and a sigmoid gate on the output.
//
//   inputs   bf16 query|gate [T, query_heads, 2, head_dim], bf16 keys and bf16
//            values [T, kv_heads, head_dim]
//   output   bf16 [T, query_heads, head_dim]
//
// Which of two modes a layer runs in is fixed at Create by the cache pointer
// and by nothing else:
//   no cache   the whole sequence at once, nothing persistent read or written.
//              One prepare launch and one flash-attention launch over scratch
//              keys/values, for up to kMaximumSequenceLength tokens (the
//              reference stops at 128, where its [heads, T, T] probability
//              tensor is still small; here that tensor exists only while an
//              attention_probabilities_hook wants it).  bwd returns the
//              gradients of all three inputs and adds the norm gradients of
//              trainable norms.
//   a cache    one token per fwd, appended to the borrowed KeyValueCache, whose
//              position moves although fwd is const.  The cache must outlive
//              the layer, belongs to this layer alone, and must be Reset before
//              another sequence and after any fwd that failed (a failing hook
//              counts).  bwd is rejected.
// Calls on one layer must not overlap; the Executor outlives the layer.
#pragma once

#include <memory>

#include "pluto_amd/host/block_parameter.h"
#include "pluto_amd/host/cached_attention_ops.h"
#include "pluto_amd/host/key_value_cache.h"
#include "pluto_amd/host/layer.h"

namespace pluto::llm {

using FullAttentionParameters = cached_attention_ops::FullAttentionParameters;

class QwenAttentionLayer final : public Layer {
 public:
  static constexpr int kMaximumDimension = 1048576;     // widest token row accepted
  static constexpr int kMaximumSequenceLength = 65535;  // no-cache mode

  // Norm weights shared with their owner (an optimizer may train them); with a
  // cache, sequence_length has to be 1.
  static StatusOr<std::unique_ptr<QwenAttentionLayer>> Create(
      hip::Executor& executor, FullAttentionParameters parameters,
      std::shared_ptr<BlockParameter> q_norm, std::shared_ptr<BlockParameter> k_norm,
      int sequence_length, KeyValueCache* cache = nullptr);
  // Norm weights given as plain FP32 buffers: frozen, no gradient storage.
  static StatusOr<std::unique_ptr<QwenAttentionLayer>> Create(
      hip::Executor& executor, FullAttentionParameters parameters, Buffer q_norm, Buffer k_norm,
      int sequence_length, KeyValueCache* cache = nullptr);

  std::string_view name() const override { return "QwenAttentionLayer"; }
  DataType output_type() const override { return DataType::BF16; }
  Span<Buffer> weights() override { return Span<Buffer>(weights_, 2); }
  Span<const ActivationType> input_types() const override { return MakeConstSpan(input_types_); }
  Span<const ActivationType> output_types() const override { return MakeConstSpan(output_types_); }

 private:
  QwenAttentionLayer(hip::Executor& executor, FullAttentionParameters parameters,
                     std::shared_ptr<BlockParameter> q_norm,
                     std::shared_ptr<BlockParameter> k_norm, int sequence_length,
                     KeyValueCache* cache);
  StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const override;
  StatusOr<BufferVec> bwd_impl(hip::Executor& executor, Span<const Buffer> gradients,
                               BackwardState state, LayerHooks* hooks) override;
  // the two modes of fwd_impl; CachedForward hands an installed probability
  // hook one row per query head, [1, query_heads, 1, tokens so far]
  StatusOr<FwdResult> CachedForward(hip::Executor& executor, Span<const Buffer> inputs,
                                    LayerHooks* hooks) const;
  StatusOr<FwdResult> SequenceForward(hip::Executor& executor, Span<const Buffer> inputs,
                                      LayerHooks* hooks) const;
  // FP32 gradients of query|gate, keys and values; a norm's gradient is added
  // to its BlockParameter only while that parameter is being trained
  StatusOr<BufferVec> SequenceBackward(hip::Executor& executor, Span<const Buffer> gradients,
                                       BackwardState state);

  std::vector<ActivationType> input_types_, output_types_;
  hip::Executor& executor_;
  FullAttentionParameters parameters_;
  int sequence_length_;
  KeyValueCache* cache_;  // borrowed; null = whole-sequence mode
  std::shared_ptr<BlockParameter> q_norm_, k_norm_;
  Buffer weights_[2];  // the two norms' FP32 values, query norm first
};

}  // namespace pluto::llm
