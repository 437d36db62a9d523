// GPT-2 style causal multi-head attention over a packed [Q | K | V]
// activation: AttentionLayer of src/llm/layers/attention.h:24-71 on MI355X.
// Forward keeps the FP32 row maximum and normalizer; backward recomputes
// probability tiles from them.  dQ tiles are query-owned, dK/dV tiles
// key-owned, reductions run in a fixed order without atomics, so results are
// bitwise repeatable.  An attention_probabilities_hook triggers a separate pass
// that materialises the FP32 probabilities and leaves results unchanged.
#pragma once

#include <memory>

#include "pluto_amd/host/layer.h"

namespace pluto::llm {

class AttentionLayer final : public Layer {
 public:
  std::string_view name() const override { return "AttentionLayer"; }

  // data_type FP16 keeps FP32 activations, BF16 stores bfloat16; FP8 is
  // Unimplemented.  Attention restarts at every context_length boundary.
  static StatusOr<std::unique_ptr<AttentionLayer>> Create(hip::Executor& executor,
                                                          int context_length, int num_heads,
                                                          int embedding_dim, DataType data_type);

  Span<Buffer> weights() override { return {}; }
  DataType output_type() const override { return output_type_; }
  Span<const ActivationType> input_types() const override { return MakeConstSpan(input_types_); }
  Span<const ActivationType> output_types() const override { return MakeConstSpan(output_types_); }

 private:
  AttentionLayer(hip::Executor& executor, int context_length, int num_heads, int embedding_dim,
                 DataType data_type);
  StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const override;
  StatusOr<BufferVec> bwd_impl(hip::Executor& executor, Span<const Buffer> output_gradients,
                               BackwardState state, LayerHooks* hooks) override;

  hip::Executor& executor_;
  int context_length_, num_heads_, embedding_dim_;
  DataType output_type_;
  std::vector<ActivationType> input_types_, output_types_;
};

}  // namespace pluto::llm
