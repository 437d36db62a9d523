// Inference-only, batch-one causal convolution and gated delta-rule layer:
// DeltaNetLayer of src/llm/layers/delta_net.h:10-67.  Each fwd consumes one
// token's packed QKV, gate Z, time-step A and update B projections (physical
// BF16) and advances persistent FP32 convolution/recurrent state.  Const fwd is
// stateful, so concurrent calls are not supported.  Reset before a new
// sequence or after any failed forward.  Backward is unsupported.
#pragma once

#include <memory>

#include "pluto_amd/host/cached_attention_ops.h"
#include "pluto_amd/host/layer.h"

namespace pluto::llm {

using DeltaNetParameters = cached_attention_ops::DeltaNetParameters;

class DeltaNetLayer final : public Layer {
 public:
  static constexpr int kMaximumDimension = 1048576;

  // FP32 weights: convolution [QKV, kernel], A_log [value_heads], dt_bias
  // [value_heads], RMS multiplier [value_dim].
  static StatusOr<std::unique_ptr<DeltaNetLayer>> Create(hip::Executor& executor,
                                                         DeltaNetParameters parameters,
                                                         Buffer convolution, Buffer a_log,
                                                         Buffer dt_bias, Buffer norm);

  std::string_view name() const override { return "DeltaNetLayer"; }
  DataType output_type() const override { return DataType::BF16; }
  Span<Buffer> weights() override { return Span<Buffer>(weights_, 4); }
  Span<const ActivationType> input_types() const override { return MakeConstSpan(input_types_); }
  Span<const ActivationType> output_types() const override { return MakeConstSpan(output_types_); }
  Status Reset();

 private:
  DeltaNetLayer(hip::Executor& executor, DeltaNetParameters parameters, Buffer convolution,
                Buffer a_log, Buffer dt_bias, Buffer norm,
                std::unique_ptr<cached_attention_ops::DeltaNetState> cache);
  StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const override;
  StatusOr<BufferVec> bwd_impl(hip::Executor& executor, Span<const Buffer> gradients,
                               BackwardState state, LayerHooks* hooks) override;

  hip::Executor& executor_;
  DeltaNetParameters parameters_;
  Buffer weights_[4];
  std::unique_ptr<cached_attention_ops::DeltaNetState> cache_;
  std::vector<ActivationType> input_types_, output_types_;
};

}  // namespace pluto::llm
