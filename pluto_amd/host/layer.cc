// Hook dispatch and the state-identity check of the Layer base class.  The
// behaviour implemented is the one src/llm/layer.h:135-160 documents (and
// src/llm/layer.cc:35-84 has): a hook sees buffer handles it may swap for others
// of the same byte size on the same executor; forward state is published only
// after the hook accepted the outputs; backward refuses foreign state before
// anything else happens.
#include "pluto_amd/host/layer.h"

#include <functional>

#include "pluto_amd/host/layer_hooks.h"

namespace pluto::llm {
namespace {

// The handles one hook call may replace.  `offered_` is what the layer (or the
// caller) produced and stays referenced until this object dies, so a handle the
// hook drops is released only after the hook has queued whatever reads of it
// it wanted; `current_` is what the hook leaves behind.
class HookExchange {
 public:
  using Hook = std::function<Status(hip::Executor&, std::string_view, Span<const ActivationType>,
                                    Span<hip::Buffer>)>;

  HookExchange(hip::Executor& executor, Span<const Buffer> handles)
      : executor_(executor), offered_(handles.begin(), handles.end()), current_(offered_) {}

  Status Offer(const Hook& hook, std::string_view layer, Span<const ActivationType> types) {
    RETURN_IF_ERROR(AllOnExecutor(offered_));
    RETURN_IF_ERROR(hook(executor_, layer, types, MakeSpan(current_)));
    // The hook got a span, so the count cannot have changed; the owner and
    // the extent of each handle can.
    RETURN_IF_ERROR(AllOnExecutor(current_));
    for (size_t slot = 0; slot < offered_.size(); ++slot) {
      const size_t before = offered_[slot].size_bytes(), after = current_[slot].size_bytes();
      if (after != before)
        return InvalidArgumentError(StrCat("hook changed buffer ", slot, " byte size from ",
                                           before, " to ", after));
    }
    return OkStatus();
  }

  BufferVec& current() { return current_; }

 private:
  Status AllOnExecutor(const BufferVec& handles) const {
    size_t slot = 0;
    for (const Buffer& handle : handles) {
      if (&handle.executor() != &executor_)
        return InvalidArgumentError(StrCat("hook buffer ", slot, " belongs to another executor"));
      ++slot;
    }
    return OkStatus();
  }

  hip::Executor& executor_;
  const BufferVec offered_;
  BufferVec current_;
};

}  // namespace

StatusOr<FwdResult> Layer::fwd(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks* hooks) const {
  StatusOr<FwdResult> produced = fwd_impl(executor, inputs, hooks);
  if (!produced.ok()) return produced.status();
  FwdResult result = std::move(produced).value();
  const bool observed = hooks != nullptr && static_cast<bool>(hooks->activation_hook);
  if (observed) {
    const Span<const ActivationType> types = output_types();
    if (types.size() != result.outputs.size())
      return InvalidArgumentError(
          "activation hook requires one activation type per forward output");
    HookExchange exchange(executor, MakeConstSpan(result.outputs));
    RETURN_IF_ERROR(exchange.Offer(hooks->activation_hook, name(), types));
    result.outputs = exchange.current();
  }
  // only now is the state one that bwd() accepts
  result.state.layer = this;
  return result;
}

StatusOr<BufferVec> Layer::bwd(hip::Executor& executor, Span<const Buffer> output_gradients,
                               BackwardState state, LayerHooks* hooks) {
  if (state.layer != this)
    return InvalidArgumentError("bwd requires a state from this layer's successful fwd");
  const bool observed = hooks != nullptr && static_cast<bool>(hooks->gradient_hook);
  if (!observed) return bwd_impl(executor, output_gradients, std::move(state), hooks);

  // The hook is told the gradients are FP32 tensors shaped like the outputs
  // they belong to; a layer may receive fewer gradients than it has outputs.
  const Span<const ActivationType> outputs = output_types();
  const size_t count = output_gradients.size();
  if (count > outputs.size())
    return InvalidArgumentError("gradient hook received more gradients than forward output types");
  std::vector<ActivationType> described;
  described.reserve(count);
  for (size_t i = 0; i < count; ++i) {
    const Span<const int64_t> shape = outputs[i].dimensions();
    described.push_back(ActivationType(DataType::FP32, {shape.begin(), shape.end()}));
  }
  // The exchange works on copies of the handles: the caller's own stay as
  // they were, whatever the hook substitutes.
  HookExchange exchange(executor, output_gradients);
  RETURN_IF_ERROR(exchange.Offer(hooks->gradient_hook, name(), MakeConstSpan(described)));
  return bwd_impl(executor, MakeConstSpan(exchange.current()), std::move(state), hooks);
}

}  // namespace pluto::llm
