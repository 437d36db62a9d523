#include "pluto_amd/host/layer.h"

#include "pluto_amd/host/layer_hooks.h"

namespace pluto::llm {
namespace {

Status CheckHookBuffers(hip::Executor& executor, Span<const Buffer> buffers) {
  for (size_t i = 0; i < buffers.size(); ++i)
    if (&buffers[i].executor() != &executor)
      return InvalidArgumentError(StrCat("hook buffer ", i, " belongs to another executor"));
  return OkStatus();
}

Status CheckReplacements(hip::Executor& executor, Span<const Buffer> original,
                         Span<const Buffer> replacement) {
  RETURN_IF_ERROR(CheckHookBuffers(executor, replacement));
  for (size_t i = 0; i < original.size(); ++i)
    if (replacement[i].size_bytes() != original[i].size_bytes())
      return InvalidArgumentError(StrCat("hook changed buffer ", i, " byte size"));
  return OkStatus();
}

}  // namespace

// src/llm/layer.cc:35-54
StatusOr<FwdResult> Layer::fwd(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const {
  ASSIGN_OR_RETURN(auto result, fwd_impl(executor, inputs, hooks));
  if (hooks != nullptr && hooks->activation_hook) {
    const auto types = output_types();
    if (result.outputs.size() != types.size())
      return InvalidArgumentError(
          "activation hook requires one activation type per forward output");
    RETURN_IF_ERROR(CheckHookBuffers(executor, MakeConstSpan(result.outputs)));
    // keep the original handles alive across the callback so that replacing a
    // handle cannot queue its free before the callback has queued its reads
    const BufferVec original = result.outputs;
    RETURN_IF_ERROR(hooks->activation_hook(executor, name(), types, MakeSpan(result.outputs)));
    RETURN_IF_ERROR(
        CheckReplacements(executor, MakeConstSpan(original), MakeConstSpan(result.outputs)));
  }
  result.state.layer = this;
  return result;
}

// src/llm/layer.cc:56-84
StatusOr<BufferVec> Layer::bwd(hip::Executor& executor, Span<const Buffer> output_gradients,
                               BackwardState state, LayerHooks* hooks) {
  if (state.layer != this)
    return InvalidArgumentError("bwd requires a state from this layer's successful fwd");
  if (hooks == nullptr || !hooks->gradient_hook)
    return bwd_impl(executor, output_gradients, std::move(state), hooks);
  const auto types = output_types();
  if (output_gradients.size() > types.size())
    return InvalidArgumentError("gradient hook received more gradients than forward output types");
  RETURN_IF_ERROR(CheckHookBuffers(executor, output_gradients));
  std::vector<ActivationType> gradient_types;
  for (size_t i = 0; i < output_gradients.size(); ++i) {
    const auto dims = types[i].dimensions();
    gradient_types.emplace_back(DataType::FP32, std::vector<int64_t>(dims.begin(), dims.end()));
  }
  BufferVec gradients(output_gradients.begin(), output_gradients.end());
  RETURN_IF_ERROR(hooks->gradient_hook(executor, name(), MakeConstSpan(gradient_types),
                                       MakeSpan(gradients)));
  RETURN_IF_ERROR(CheckReplacements(executor, output_gradients, MakeConstSpan(gradients)));
  return bwd_impl(executor, MakeConstSpan(gradients), std::move(state), hooks);
}

}  // namespace pluto::llm
