// DeltaNetLayer, the class of src/llm/layers/delta_net.h:10-67 for MI355X: one
// decoded token per fwd through a causal depthwise convolution and the gated
// delta rule, for a single sequence and for inference only.
//
//   inputs   four bf16 buffers of one token: q | k | v packed, the output gate
//            z, the time-step projection a and the update-strength projection b
//   output   one bf16 buffer [value_heads * value_head_dim]: the recurrence's
//            result after the per-head RMS norm and the SiLU(z) gate (the
//            output projection is the caller's next layer)
//   state    FP32 convolution taps and FP32 recurrent matrices, owned by the
//            layer and advanced by every fwd although fwd is const: calls must
//            not overlap, and Reset() has to precede a new sequence and follow
//            any fwd that failed (a failing hook counts)
//   bwd      always Unimplemented
// The Executor passed to Create must stay alive as long as the layer.
#pragma once

#include <memory>

#include "pluto_amd/host/cached_attention_ops.h"
#include "pluto_amd/host/layer.h"

namespace pluto::llm {

using DeltaNetParameters = cached_attention_ops::DeltaNetParameters;

class DeltaNetLayer final : public Layer {
 public:
  // widest activation accepted (the packed q | k | v row included); checked
  // before any state is allocated
  static constexpr int kMaximumDimension = 1048576;

  // The weights are FP32 device buffers on `executor`, in the order of
  // weights(): convolution taps [q|k|v channels, conv_kernel_dim], A_log and
  // dt_bias [value_heads], and the norm multiplier [value_head_dim].
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

  std::vector<ActivationType> input_types_, output_types_;
  hip::Executor& executor_;  // the only executor fwd accepts
  DeltaNetParameters parameters_;
  Buffer weights_[4];
  // convolution taps, recurrent matrices and the step's workspace
  std::unique_ptr<cached_attention_ops::DeltaNetState> cache_;
};

}  // namespace pluto::llm
