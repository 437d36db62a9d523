#include "pluto_amd/host/decoder_branch.h"

#include <algorithm>

#include "pluto_amd/host/layer_util.h"

namespace pluto::llm {
namespace internal {
namespace {

int StorageCode(MatrixStorage storage) {
  switch (storage) {
    case MatrixStorage::kBFloat16: return PLUTO_HIP_MATRIX_BF16;
    case MatrixStorage::kFloat32: return PLUTO_HIP_MATRIX_F32;
    case MatrixStorage::kFp8E4M3: return PLUTO_HIP_MATRIX_FP8_E4M3;
  }
  return -1;
}

}  // namespace

StatusOr<ProjectionSet> ProjectionSet::Create(
    hip::Executor& executor, int batch, std::vector<std::unique_ptr<FullyConnectedLayer>> layers,
    const std::vector<std::pair<int, int>>& shape) {
  if (batch <= 0 || batch > PLUTO_HIP_IMPORTED_MAX_TOKENS)
    return InvalidArgumentError(StrCat("decoder batch must be in [1, ",
                                       PLUTO_HIP_IMPORTED_MAX_TOKENS, "]; got ", batch));
  ProjectionSet set;
  set.executor_ = &executor;
  set.batch_ = batch;
  size_t workspace_bytes = 0;
  for (size_t i = 0; i < layers.size(); ++i) {
    FullyConnectedLayer* layer = layers[i].get();
    if (layer == nullptr || !layer->imported_storage())
      return InvalidArgumentError(StrCat("projection ", i, " is not an imported matrix"));
    if (layer->input_dim() != shape[i].first || layer->output_dim() != shape[i].second)
      return InvalidArgumentError(StrCat("projection ", i, " is ", layer->input_dim(), " -> ",
                                         layer->output_dim(), "; the branch needs ",
                                         shape[i].first, " -> ", shape[i].second));
    for (const Buffer& weight : layer->weights())
      if (&weight.executor() != &executor)
        return InvalidArgumentError(StrCat("projection ", i, " belongs to a different Executor"));
    workspace_bytes = std::max(
        workspace_bytes, pluto_hip_dense_imported_batch_workspace_bytes(batch, layer->input_dim()));
    if (i + 1 == layers.size()) break;  // the last projection writes the branch's result
    ASSIGN_OR_RETURN(auto stage, Buffer::Allocate(executor, static_cast<size_t>(batch) *
                                                                layer->output_dim() * 2));
    set.stages_.push_back(std::move(stage));
  }
  ASSIGN_OR_RETURN(auto workspace, Buffer::Allocate(executor, std::max<size_t>(workspace_bytes, 256)));
  set.workspace_.push_back(std::move(workspace));
  set.layers_ = std::move(layers);
  return set;
}

Status ProjectionSet::Run(int which, const void* input, void* output) const {
  FullyConnectedLayer& layer = *layers_[which];
  const Span<Buffer> weights = layer.weights();
  const float* scales =
      weights.size() == 2 ? static_cast<const float*>(weights[1].data()) : nullptr;
  return hip::HipStatus(
      pluto_hip_dense_imported_forward_batch(
          executor_->stream(), StorageCode(*layer.imported_storage()), weights[0].data(), scales,
          input, batch_, layer.input_dim(), layer.output_dim(), output, workspace_[0].data(),
          workspace_[0].size_bytes()),
      "imported projection launch");
}

Status ProjectionSet::RunFirst(int count, const void* input) const {
  bool alike = count <= PLUTO_HIP_IMPORTED_MAX_MATRICES;
  for (int i = 1; i < count && alike; ++i)
    alike = *layers_[i]->imported_storage() == *layers_[0]->imported_storage() &&
            layers_[i]->input_dim() == layers_[0]->input_dim();
  if (!alike) {
    for (int which = 0; which < count; ++which)
      RETURN_IF_ERROR(Run(which, input, stage(which)));
    return OkStatus();
  }
  const void* weights[PLUTO_HIP_IMPORTED_MAX_MATRICES];
  const float* scales[PLUTO_HIP_IMPORTED_MAX_MATRICES];
  int output_dims[PLUTO_HIP_IMPORTED_MAX_MATRICES];
  void* outputs[PLUTO_HIP_IMPORTED_MAX_MATRICES];
  for (int i = 0; i < count; ++i) {
    const Span<Buffer> buffers = layers_[i]->weights();
    weights[i] = buffers[0].data();
    scales[i] = buffers.size() == 2 ? static_cast<const float*>(buffers[1].data()) : nullptr;
    output_dims[i] = layers_[i]->output_dim();
    outputs[i] = stage(i);
  }
  return hip::HipStatus(
      pluto_hip_dense_imported_forward_many(
          executor_->stream(), StorageCode(*layers_[0]->imported_storage()), count, weights,
          scales, output_dims, input, batch_, layers_[0]->input_dim(), outputs,
          workspace_[0].data(), workspace_[0].size_bytes()),
      "imported projections launch");
}

}  // namespace internal

namespace {

std::vector<ActivationType> HiddenRows(int width) {
  return {ActivationType(DataType::BF16, {ActivationType::kBatchDimension, 1, int64_t{width}})};
}

Status CheckHidden(hip::Executor& expected, hip::Executor& executor, Span<const Buffer> inputs,
                   int batch, int width) {
  RETURN_IF_ERROR(internal::ValidateExecutor(expected, executor, "AttentionBranch"));
  if (inputs.size() != 1) return InvalidArgumentError("AttentionBranch fwd expects one input");
  return internal::ValidateBuffer(executor, inputs[0], static_cast<size_t>(batch) * width * 2,
                                  "bf16 hidden rows of the batch");
}

}  // namespace

// ---- full attention ---------------------------------------------------------

StatusOr<std::unique_ptr<BatchedFullAttentionBranch>> BatchedFullAttentionBranch::Create(
    hip::Executor& executor, cached_attention_ops::FullAttentionParameters p, int batch,
    std::unique_ptr<FullyConnectedLayer> query_gate, std::unique_ptr<FullyConnectedLayer> key,
    std::unique_ptr<FullyConnectedLayer> value, std::unique_ptr<FullyConnectedLayer> output,
    Buffer q_norm, Buffer k_norm, KeyValueCache::Storage storage) {
  const pluto_hip_attention_params abi = cached_attention_ops::ToAbi(p);
  if (pluto_hip_attention_params_validate(&abi) != 0)
    return InvalidArgumentError("invalid full-attention dimensions or parameters");
  if (output == nullptr) return InvalidArgumentError("projection 3 is not an imported matrix");
  const int q = p.query_heads * p.head_dim, kv = p.key_value_heads * p.head_dim;
  const int width = output->output_dim();
  for (const Buffer* norm : {&q_norm, &k_norm})
    RETURN_IF_ERROR(internal::ValidateBuffer(executor, *norm, sizeof(float) * p.head_dim,
                                             "attention norm weight"));
  std::vector<std::unique_ptr<FullyConnectedLayer>> layers;
  layers.push_back(std::move(query_gate));
  layers.push_back(std::move(key));
  layers.push_back(std::move(value));
  layers.push_back(std::move(output));
  ASSIGN_OR_RETURN(auto projections,
                   internal::ProjectionSet::Create(executor, batch, std::move(layers),
                                                   {{width, 2 * q}, {width, kv}, {width, kv},
                                                    {q, width}}));
  std::unique_ptr<BatchedFullAttentionBranch> branch(
      new BatchedFullAttentionBranch(executor, p, std::move(projections)));
  branch->types_ = HiddenRows(width);
  branch->norms_ = {std::move(q_norm), std::move(k_norm)};
  for (int s = 0; s < batch; ++s) {
    ASSIGN_OR_RETURN(auto cache, KeyValueCache::Create(executor, p.capacity, p.key_value_heads,
                                                       p.head_dim, storage));
    RETURN_IF_ERROR(cached_attention_ops::ValidateCachedAttention(executor, p, *cache));
    branch->borrowed_.push_back(cache.get());
    branch->caches_.push_back(std::move(cache));
  }
  ASSIGN_OR_RETURN(auto attended, Buffer::Allocate(executor, static_cast<size_t>(batch) * q * 2));
  branch->attended_.push_back(std::move(attended));
  return branch;
}

void BatchedFullAttentionBranch::Reset() {
  for (auto& cache : caches_) cache->Reset();
}

StatusOr<FwdResult> BatchedFullAttentionBranch::fwd_impl(hip::Executor& executor,
                                                         Span<const Buffer> inputs,
                                                         LayerHooks*) const {
  const int width = projections_.output_dim(3);
  RETURN_IF_ERROR(CheckHidden(executor_, executor, inputs, batch(), width));
  // nothing is launched for a batch one of whose caches is full
  for (const KeyValueCache* cache : borrowed_)
    if (cache->position() >= cache->capacity())
      return ResourceExhaustedError("full-attention cache capacity reached");
  ASSIGN_OR_RETURN(auto result, Buffer::Allocate(executor, inputs[0].size_bytes()));
  const void* hidden = inputs[0].data();
  RETURN_IF_ERROR(projections_.RunFirst(3, hidden));
  RETURN_IF_ERROR(cached_attention_ops::CachedAttentionStepBatchBFloat16(
      executor, parameters_, Span<KeyValueCache* const>(borrowed_.data(), borrowed_.size()),
      projections_.stage(0), projections_.stage(1), projections_.stage(2),
      static_cast<const float*>(norms_[0].data()), static_cast<const float*>(norms_[1].data()),
      attended_[0].data()));
  RETURN_IF_ERROR(projections_.Run(3, attended_[0].data(), result.data()));
  FwdResult forward;
  forward.outputs.push_back(std::move(result));
  return forward;
}

StatusOr<BufferVec> BatchedFullAttentionBranch::bwd_impl(hip::Executor&, Span<const Buffer>,
                                                         BackwardState, LayerHooks*) {
  return UnimplementedError("the batched decoder branch supports cached inference only");
}

// ---- delta-net --------------------------------------------------------------

StatusOr<std::unique_ptr<BatchedDeltaNetBranch>> BatchedDeltaNetBranch::Create(
    hip::Executor& executor, cached_attention_ops::DeltaNetParameters p, int batch,
    std::unique_ptr<FullyConnectedLayer> qkv, std::unique_ptr<FullyConnectedLayer> z,
    std::unique_ptr<FullyConnectedLayer> a, std::unique_ptr<FullyConnectedLayer> b,
    std::unique_ptr<FullyConnectedLayer> output, Buffer convolution, Buffer a_log, Buffer dt_bias,
    Buffer norm) {
  // the state validates the parameters before any of them is multiplied here
  ASSIGN_OR_RETURN(auto state, cached_attention_ops::DeltaNetState::Create(executor, p, batch));
  if (output == nullptr) return InvalidArgumentError("projection 4 is not an imported matrix");
  const int keys = p.key_heads * p.key_head_dim, values = p.value_heads * p.value_head_dim;
  const int channels = 2 * keys + values, width = output->output_dim();
  const Buffer* weights[] = {&convolution, &a_log, &dt_bias, &norm};
  const size_t floats[] = {static_cast<size_t>(channels) * p.conv_kernel_dim,
                           static_cast<size_t>(p.value_heads), static_cast<size_t>(p.value_heads),
                           static_cast<size_t>(p.value_head_dim)};
  for (int i = 0; i < 4; ++i)
    RETURN_IF_ERROR(internal::ValidateBuffer(executor, *weights[i], floats[i] * sizeof(float),
                                             "delta-net weight"));
  std::vector<std::unique_ptr<FullyConnectedLayer>> layers;
  layers.push_back(std::move(qkv));
  layers.push_back(std::move(z));
  layers.push_back(std::move(a));
  layers.push_back(std::move(b));
  layers.push_back(std::move(output));
  ASSIGN_OR_RETURN(auto projections,
                   internal::ProjectionSet::Create(executor, batch, std::move(layers),
                                                   {{width, channels}, {width, values},
                                                    {width, p.value_heads},
                                                    {width, p.value_heads}, {values, width}}));
  std::unique_ptr<BatchedDeltaNetBranch> branch(
      new BatchedDeltaNetBranch(executor, p, std::move(projections)));
  branch->types_ = HiddenRows(width);
  branch->weights_ = {std::move(convolution), std::move(a_log), std::move(dt_bias),
                      std::move(norm)};
  branch->state_ = std::move(state);
  ASSIGN_OR_RETURN(auto mixed, Buffer::Allocate(executor, static_cast<size_t>(batch) * values * 2));
  branch->mixed_.push_back(std::move(mixed));
  return branch;
}

StatusOr<FwdResult> BatchedDeltaNetBranch::fwd_impl(hip::Executor& executor,
                                                    Span<const Buffer> inputs, LayerHooks*) const {
  const int width = projections_.output_dim(4);
  RETURN_IF_ERROR(CheckHidden(executor_, executor, inputs, batch(), width));
  ASSIGN_OR_RETURN(auto result, Buffer::Allocate(executor, inputs[0].size_bytes()));
  const void* hidden = inputs[0].data();
  RETURN_IF_ERROR(projections_.RunFirst(4, hidden));
  auto weight = [this](int i) { return static_cast<const float*>(weights_[i].data()); };
  RETURN_IF_ERROR(state_->StepBFloat16(projections_.stage(0), projections_.stage(1),
                                       projections_.stage(2), projections_.stage(3), weight(0),
                                       weight(1), weight(2), weight(3), mixed_[0].data()));
  RETURN_IF_ERROR(projections_.Run(4, mixed_[0].data(), result.data()));
  FwdResult forward;
  forward.outputs.push_back(std::move(result));
  return forward;
}

StatusOr<BufferVec> BatchedDeltaNetBranch::bwd_impl(hip::Executor&, Span<const Buffer>,
                                                    BackwardState, LayerHooks*) {
  return UnimplementedError("the batched decoder branch supports cached inference only");
}

}  // namespace pluto::llm
