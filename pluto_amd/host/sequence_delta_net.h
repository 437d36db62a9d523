// Stateless whole-sequence counterpart of DeltaNetLayer:
// SequenceDeltaNetLayer of src/llm/layers/sequence_delta_net.h:11-74.  A call
// consumes the entire sequence, starting from zero convolution and recurrent
// history.  Inputs are BF16 [1,T,QKV], [1,T,V], [1,T,H], [1,T,H]; the output is
// BF16 [1,T,V].  QKV packs all Q, then all K, then all V.  The forward pass
// runs the chunked (64-token) matrix-core scan instead of a token loop, so any
// sequence length up to kMaximumSequenceLength is accepted (the reference
// stops at 128).  The per-token state snapshots the reference keeps for its
// backward pass are not produced by forward: backward repeats the forward pass
// and keeps the states it needs in its own scratch.
#pragma once

#include <memory>

#include "pluto_amd/host/block_parameter.h"
#include "pluto_amd/host/cached_attention_ops.h"
#include "pluto_amd/host/layer.h"

namespace pluto::llm {

class SequenceDeltaNetLayer final : public Layer {
 public:
  static constexpr int kMaximumSequenceLength = 1 << 20;
  // bwd keeps one recurrent state per token in scratch (as the reference does)
  static constexpr int kMaximumBackwardLength = 65535;

  // Convolution is [QKV,kernel], A_log and dt_bias are [value_heads], and
  // norm is [value_head_dim], a plain multiplier rather than 1 + weight.
  static StatusOr<std::unique_ptr<SequenceDeltaNetLayer>> Create(
      hip::Executor& executor, cached_attention_ops::DeltaNetParameters parameters,
      std::shared_ptr<BlockParameter> convolution, std::shared_ptr<BlockParameter> a_log,
      std::shared_ptr<BlockParameter> dt_bias, std::shared_ptr<BlockParameter> norm,
      int sequence_length);

  std::string_view name() const override { return "SequenceDeltaNetLayer"; }
  DataType output_type() const override { return DataType::BF16; }
  Span<Buffer> weights() override { return Span<Buffer>(weights_, 4); }
  Span<const ActivationType> input_types() const override { return MakeConstSpan(input_types_); }
  Span<const ActivationType> output_types() const override { return MakeConstSpan(output_types_); }

 private:
  SequenceDeltaNetLayer(hip::Executor& executor,
                        cached_attention_ops::DeltaNetParameters parameters,
                        std::shared_ptr<BlockParameter> convolution,
                        std::shared_ptr<BlockParameter> a_log,
                        std::shared_ptr<BlockParameter> dt_bias,
                        std::shared_ptr<BlockParameter> norm, int sequence_length);
  StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const override;
  StatusOr<BufferVec> bwd_impl(hip::Executor& executor, Span<const Buffer> gradients,
                               BackwardState state, LayerHooks* hooks) override;

  hip::Executor& executor_;
  cached_attention_ops::DeltaNetParameters parameters_;
  int sequence_length_;
  std::shared_ptr<BlockParameter> parameters_owned_[4];
  Buffer weights_[4];
  std::vector<ActivationType> input_types_, output_types_;
};

}  // namespace pluto::llm
