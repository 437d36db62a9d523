// The attention branch of a decoder block for several sequences decoded
// together.  The reference builds this branch per layer for one sequence
// (CreateAttentionBranch, src/llm/qwen/model.cc:174-274: imported projections,
// then QwenAttentionLayer over a KeyValueCache or DeltaNetLayer, then the output
// projection) and Model::Step (model.cc:405-428) drives it one token at a
// time.  The two classes here are that branch, without its input norm, lifted
// to `batch` sequences that each own a cache or a recurrent state: one fwd
// takes the normalised hidden rows of all sequences, bf16 [batch, model_width],
// and returns the branch output, bf16 [batch, model_width].
//
// Row s of the result is what the reference's chain of batch-one layers gives
// for sequence s: bit for bit up to eight sequences, and to the summation order
// of the projections beyond that (their many-token kernel runs on the matrix
// cores).  All activations between the stages stay bf16 in buffers allocated
// at Create; a step issues 6 (full attention) or 7 (delta-net) launches and
// allocates its result and the attention's workspace.  Like the layers they are
// made of, both are stateful behind a const fwd: calls must not overlap, and
// after a failed fwd Reset() comes first.  Hooks see the branch's output only.
#pragma once

#include <memory>
#include <vector>

#include "pluto_amd/host/cached_attention_ops.h"
#include "pluto_amd/host/fully_connected.h"
#include "pluto_amd/host/key_value_cache.h"
#include "pluto_amd/host/layer.h"

namespace pluto::llm {

namespace internal {

// Imported projections of one branch and the bf16 rows they write, all
// allocated once: stage i holds the output of projection i for every sequence
// (the last projection has none: it writes the branch's result).
class ProjectionSet {
 public:
  // Checks that projection i is an imported matrix on `executor` of
  // shape[i] = {input_dim, output_dim}, and allocates the stages for `batch`.
  static StatusOr<ProjectionSet> Create(hip::Executor& executor, int batch,
                                        std::vector<std::unique_ptr<FullyConnectedLayer>> layers,
                                        const std::vector<std::pair<int, int>>& shape);
  // Projection `which` of `batch` bf16 rows at `input`, into `output`.
  Status Run(int which, const void* input, void* output) const;
  // Projections 0 .. count-1 of the same rows into their stages: one call when
  // they share a storage kind (the loader gives a model's matrices one), one
  // call each otherwise; the results are the same bits either way.
  Status RunFirst(int count, const void* input) const;
  void* stage(int which) const { return stages_[which].data(); }
  int output_dim(int which) const { return layers_[which]->output_dim(); }

 private:
  ProjectionSet() = default;
  hip::Executor* executor_ = nullptr;
  int batch_ = 0;
  std::vector<std::unique_ptr<FullyConnectedLayer>> layers_;
  std::vector<Buffer> stages_;
  std::vector<Buffer> workspace_;  // one element: the largest any projection needs
};

}  // namespace internal

class BatchedFullAttentionBranch final : public Layer {
 public:
  // The four projections are imported FullyConnectedLayers as the model loader
  // makes them (model.cc:196-205,235-236): query|gate [width -> 2 q], key and
  // value [width -> kv], output [q -> width], with q = query_heads * head_dim
  // and kv = key_value_heads * head_dim.  q_norm and k_norm are FP32
  // [head_dim].  One cache per sequence is created here, of
  // parameters.capacity tokens each, in `storage`.
  static StatusOr<std::unique_ptr<BatchedFullAttentionBranch>> Create(
      hip::Executor& executor, cached_attention_ops::FullAttentionParameters parameters, int batch,
      std::unique_ptr<FullyConnectedLayer> query_gate, std::unique_ptr<FullyConnectedLayer> key,
      std::unique_ptr<FullyConnectedLayer> value, std::unique_ptr<FullyConnectedLayer> output,
      Buffer q_norm, Buffer k_norm,
      KeyValueCache::Storage storage = KeyValueCache::Storage::kBFloat16HeadMajor);

  std::string_view name() const override { return "AttentionBranch"; }
  DataType output_type() const override { return DataType::BF16; }
  Span<Buffer> weights() override { return MakeSpan(norms_); }
  Span<const ActivationType> input_types() const override { return MakeConstSpan(types_); }
  Span<const ActivationType> output_types() const override { return MakeConstSpan(types_); }

  int batch() const { return static_cast<int>(caches_.size()); }
  // Sequences advance together but need not be equally long: one that ended
  // is reset alone (cache(s).Reset()) and starts again at position 0.
  KeyValueCache& cache(int sequence) { return *caches_[sequence]; }
  void Reset();

 private:
  BatchedFullAttentionBranch(hip::Executor& executor,
                             cached_attention_ops::FullAttentionParameters parameters,
                             internal::ProjectionSet projections)
      : executor_(executor), parameters_(parameters), projections_(std::move(projections)) {}
  StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const override;
  StatusOr<BufferVec> bwd_impl(hip::Executor& executor, Span<const Buffer> gradients,
                               BackwardState state, LayerHooks* hooks) override;

  hip::Executor& executor_;
  cached_attention_ops::FullAttentionParameters parameters_;
  internal::ProjectionSet projections_;  // query|gate, key, value, output
  std::vector<ActivationType> types_;
  std::vector<std::unique_ptr<KeyValueCache>> caches_;
  std::vector<KeyValueCache*> borrowed_;
  std::vector<Buffer> norms_;    // q_norm, k_norm
  std::vector<Buffer> attended_;  // one element: bf16 [batch, q], the output projection's input
};

class BatchedDeltaNetBranch final : public Layer {
 public:
  // Projections as model.cc:238-251,272-273 loads them: q|k|v [width -> 2 k + v],
  // z [width -> v], a and b [width -> value_heads], output [v -> width], with
  // k = key_heads * key_head_dim and v = value_heads * value_head_dim; then the
  // four FP32 weights of DeltaNetLayer::Create.
  static StatusOr<std::unique_ptr<BatchedDeltaNetBranch>> Create(
      hip::Executor& executor, cached_attention_ops::DeltaNetParameters parameters, int batch,
      std::unique_ptr<FullyConnectedLayer> qkv, std::unique_ptr<FullyConnectedLayer> z,
      std::unique_ptr<FullyConnectedLayer> a, std::unique_ptr<FullyConnectedLayer> b,
      std::unique_ptr<FullyConnectedLayer> output, Buffer convolution, Buffer a_log,
      Buffer dt_bias, Buffer norm);

  std::string_view name() const override { return "AttentionBranch"; }
  DataType output_type() const override { return DataType::BF16; }
  Span<Buffer> weights() override { return MakeSpan(weights_); }
  Span<const ActivationType> input_types() const override { return MakeConstSpan(types_); }
  Span<const ActivationType> output_types() const override { return MakeConstSpan(types_); }

  int batch() const { return state_->batch(); }
  Status Reset() { return state_->Reset(); }
  // One sequence back to its initial state, the others untouched.
  Status Reset(int sequence) { return state_->Reset(sequence); }

 private:
  BatchedDeltaNetBranch(hip::Executor& executor,
                        cached_attention_ops::DeltaNetParameters parameters,
                        internal::ProjectionSet projections)
      : executor_(executor), parameters_(parameters), projections_(std::move(projections)) {}
  StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const override;
  StatusOr<BufferVec> bwd_impl(hip::Executor& executor, Span<const Buffer> gradients,
                               BackwardState state, LayerHooks* hooks) override;

  hip::Executor& executor_;
  cached_attention_ops::DeltaNetParameters parameters_;
  internal::ProjectionSet projections_;  // q|k|v, z, a, b, output
  std::vector<ActivationType> types_;
  std::vector<Buffer> weights_;  // convolution, A_log, dt_bias, norm
  std::unique_ptr<cached_attention_ops::DeltaNetState> state_;
  std::vector<Buffer> mixed_;  // one element: bf16 [batch, v], the output projection's input
};

}  // namespace pluto::llm
