// Optional synchronous host callbacks around asynchronous layer work, as in
// src/llm/layer_hooks.h:46-109.  Only the callbacks the attention path can
// reach are declared: activation_hook, gradient_hook and
// attention_probabilities_hook (the combinator callbacks belong to layers that
// are outside this path).
#pragma once

#include <functional>
#include <string_view>

#include "pluto_amd/host/executor.h"
#include "pluto_amd/host/status.h"

namespace pluto::llm {

class ActivationType;

struct LayerHooks {
  // After a successful fwd_impl, before outputs are published.  Handles may be
  // replaced by buffers of the same byte size on the same executor.
  std::function<Status(hip::Executor& executor, std::string_view layer_name,
                       Span<const ActivationType> activation_types, Span<hip::Buffer> activations)>
      activation_hook;
  // After the state-identity check and before bwd_impl; FP32 gradients of the
  // forward outputs.
  std::function<Status(hip::Executor& executor, std::string_view layer_name,
                       Span<const ActivationType> activation_types, Span<hip::Buffer> gradients)>
      gradient_hook;
  // Contiguous FP32 probabilities [batch, heads, query, key] (zeros above the
  // diagonal) for sequence attention, [1, heads, 1, history] for cached
  // attention.  Read-only; costs a separate pass and a quadratic buffer.
  std::function<Status(hip::Executor& executor, std::string_view layer_name,
                       const ActivationType& probabilities_type, const hip::Buffer& probabilities)>
      attention_probabilities_hook;
};

}  // namespace pluto::llm
