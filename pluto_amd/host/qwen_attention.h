// Batch-one Qwen grouped-query attention: per-head Q/K RMSNorm, partial RoPE,
// causal attention and sigmoid output gating -- QwenAttentionLayer of
// src/llm/layers/qwen_attention.h:11-101 on MI355X.  Inputs are physical BF16
// [T, query_heads, 2, head_dim] query/gate and [T, KV_heads, head_dim] K/V;
// the output is BF16 [T, query_heads, head_dim].
//
// A null cache selects stateless whole-sequence attention ("prefill"): one
// prepare launch and one flash-attention launch over a private K/V scratch, for
// any sequence length up to kMaximumSequenceLength (the reference stops at 128
// because it materialises the quadratic probability tensor; here that tensor is
// only produced when an attention_probabilities_hook asks for it).  Backward
// through the sequence path is not part of this library and reports
// Unimplemented.
//
// A nonnull cache selects single-token decoding and rejects backward.  The
// cache is borrowed, must outlive the layer and must not be shared between
// layers; its position advances even though fwd is const.  Reset it before a
// new sequence or after any failed forward (including hooks).
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
  // Bounds converted projection scratch for cached, single-token inference.
  static constexpr int kMaximumDimension = 1048576;
  static constexpr int kMaximumSequenceLength = 65535;

  // Shares resident FP32 norm parameters.  The cache pointer alone selects the
  // execution mode; cached attention requires sequence_length == 1.
  static StatusOr<std::unique_ptr<QwenAttentionLayer>> Create(
      hip::Executor& executor, FullAttentionParameters parameters,
      std::shared_ptr<BlockParameter> q_norm, std::shared_ptr<BlockParameter> k_norm,
      int sequence_length, KeyValueCache* cache = nullptr);
  // Imports frozen FP32 norm buffers.
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
  // Appends one token to the borrowed cache and optionally reports its
  // [1, query_heads, 1, prefix_length] attention probabilities.
  StatusOr<FwdResult> CachedForward(hip::Executor& executor, Span<const Buffer> inputs,
                                    LayerHooks* hooks) const;
  // Whole causal sequence, without reading or updating any persistent cache.
  StatusOr<FwdResult> SequenceForward(hip::Executor& executor, Span<const Buffer> inputs,
                                      LayerHooks* hooks) const;

  // Returns FP32 Q/gate, K and V gradients; accumulates norm gradients only
  // into parameters that are active.
  StatusOr<BufferVec> SequenceBackward(hip::Executor& executor, Span<const Buffer> gradients,
                                       BackwardState state);

  hip::Executor& executor_;
  FullAttentionParameters parameters_;
  std::shared_ptr<BlockParameter> q_norm_, k_norm_;
  int sequence_length_;
  Buffer weights_[2];     // Resident FP32 query/key norm values, in that order.
  KeyValueCache* cache_;  // Nonowning; null means stateless sequence attention.
  std::vector<ActivationType> input_types_, output_types_;
};

}  // namespace pluto::llm
