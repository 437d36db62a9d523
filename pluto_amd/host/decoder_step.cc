#include "pluto_amd/host/decoder_step.h"

#include "pluto_amd/host/layer_util.h"

namespace pluto::llm {
namespace {

ActivationType HiddenRows(int width) {
  return ActivationType(DataType::BF16, {ActivationType::kBatchDimension, 1, int64_t{width}});
}

}  // namespace

StatusOr<std::unique_ptr<BatchedDecoderStep>> BatchedDecoderStep::Create(
    hip::Executor& executor, int batch, int width, int capacity,
    std::vector<std::unique_ptr<Layer>> layers, std::vector<BatchedFullAttentionBranch*> attention,
    std::vector<BatchedDeltaNetBranch*> delta_net) {
  if (batch <= 0 || width <= 0 || capacity <= 0)
    return InvalidArgumentError("decoder step batch, width and capacity must be positive");
  if (layers.empty()) return InvalidArgumentError("decoder step needs at least one layer");
  const ActivationType rows = HiddenRows(width);
  for (size_t i = 0; i < layers.size(); ++i) {
    const Layer* layer = layers[i].get();
    if (layer == nullptr) return InvalidArgumentError(StrCat("decoder layer ", i, " is null"));
    if (layer->input_types().size() != 1 || layer->output_types().size() != 1 ||
        !(layer->input_types()[0] == rows) || !(layer->output_types()[0] == rows))
      return InvalidArgumentError(
          StrCat("decoder layer ", i, " (", layer->name(), ") does not map bf16 rows of width ",
                 width, " to rows of the same type"));
  }
  for (BatchedFullAttentionBranch* branch : attention) {
    if (branch == nullptr || branch->batch() != batch)
      return InvalidArgumentError("an attention branch is missing or has a different batch");
    for (int s = 0; s < batch; ++s)
      if (branch->cache(s).capacity() < capacity)
        return InvalidArgumentError("an attention cache is smaller than the step's capacity");
  }
  for (BatchedDeltaNetBranch* branch : delta_net)
    if (branch == nullptr || branch->batch() != batch)
      return InvalidArgumentError("a delta-net branch is missing or has a different batch");
  std::unique_ptr<BatchedDecoderStep> step(new BatchedDecoderStep(executor, width, capacity));
  step->positions_.assign(batch, 0);
  step->layers_ = std::move(layers);
  step->attention_ = std::move(attention);
  step->delta_net_ = std::move(delta_net);
  // caches and states may have been used before they were handed over
  RETURN_IF_ERROR(step->Reset());
  return step;
}

Status BatchedDecoderStep::Step(const Buffer& hidden, LayerHooks* hooks) {
  if (poisoned_) return FailedPreconditionError("Reset the decoder caches after a failed Step");
  RETURN_IF_ERROR(internal::ValidateBuffer(executor_, hidden,
                                           static_cast<size_t>(batch()) * width_ * 2,
                                           "bf16 hidden rows of the batch"));
  for (int s = 0; s < batch(); ++s)
    if (positions_[s] >= capacity_)
      return InvalidArgumentError(StrCat("context capacity exhausted for sequence ", s));
  // Hooks or later layers can fail after some caches advance.  Never consume
  // that mixed history until Reset has restored every cache.
  poisoned_ = true;
  hidden_.reset();
  Buffer rows = hidden;
  for (const std::unique_ptr<Layer>& layer : layers_) {
    ASSIGN_OR_RETURN(auto result, layer->fwd(executor_, {rows}, hooks));
    if (result.outputs.size() != 1)
      return InternalError(StrCat(layer->name(), " returned ", result.outputs.size(), " outputs"));
    rows = std::move(result.outputs[0]);
  }
  hidden_ = std::move(rows);
  for (int& position : positions_) ++position;
  poisoned_ = false;
  return OkStatus();
}

StatusOr<Buffer> BatchedDecoderStep::Hidden() const {
  if (!hidden_ || poisoned_)
    return FailedPreconditionError("the hidden rows require a successful Step");
  return *hidden_;
}

Status BatchedDecoderStep::Reset() {
  for (BatchedFullAttentionBranch* branch : attention_) branch->Reset();
  for (BatchedDeltaNetBranch* branch : delta_net_) RETURN_IF_ERROR(branch->Reset());
  for (int& position : positions_) position = 0;
  hidden_.reset();
  poisoned_ = false;
  return OkStatus();
}

Status BatchedDecoderStep::Reset(int sequence) {
  if (sequence < 0 || sequence >= batch())
    return InvalidArgumentError(StrCat("no sequence ", sequence, " in a batch of ", batch()));
  if (poisoned_)
    return FailedPreconditionError("after a failed Step only a full Reset restores the caches");
  for (BatchedFullAttentionBranch* branch : attention_) branch->cache(sequence).Reset();
  for (BatchedDeltaNetBranch* branch : delta_net_) RETURN_IF_ERROR(branch->Reset(sequence));
  positions_[sequence] = 0;
  return OkStatus();
}

}  // namespace pluto::llm
