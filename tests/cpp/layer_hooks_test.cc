// Hook dispatch of the Layer base class and the DeltaNetLayer wrapper through
// the host API.  The hook cases check the behaviours src/llm/layer.h:135-160
// promises (the reference exercises them in src/llm/layer_hooks_test.cc:436-600)
// on a pass-through layer defined here.
#include "pluto_amd/host/delta_net.h"
#include "pluto_amd/host/layer_hooks.h"
#include "tests/cpp/test_support.h"

namespace pluto::llm {
namespace {

using testing::BFloat16;
using testing::NewExecutor;
using testing::Read;
using testing::Upload;
using testing::Values;

// Forwards its inputs as outputs (or a fixed list of outputs, or an error),
// saves them as intermediates, and records what bwd_impl receives.
class PassThrough final : public Layer {
 public:
  explicit PassThrough(int outputs = 1) {
    for (int i = 0; i < outputs; ++i)
      types_.emplace_back(DataType::BF16,
                          std::vector<int64_t>{ActivationType::kBatchDimension, 4 + i});
  }
  std::string_view name() const override { return "PassThrough"; }
  Span<const ActivationType> input_types() const override { return MakeConstSpan(types_); }
  Span<const ActivationType> output_types() const override { return MakeConstSpan(types_); }
  Span<Buffer> weights() override { return {}; }
  DataType output_type() const override { return DataType::BF16; }

  Status forward_status = OkStatus();
  bool fresh_copy = false;      // outputs are new buffers holding the inputs' bytes
  BufferVec forced_outputs;     // when non-empty, returned instead of the inputs
  mutable int forward_calls = 0;
  int backward_calls = 0;
  BufferVec received;

 private:
  StatusOr<FwdResult> fwd_impl(hip::Executor& executor, Span<const Buffer> inputs,
                               LayerHooks*) const override {
    ++forward_calls;
    if (!forward_status.ok()) return forward_status;
    FwdResult result;
    if (!forced_outputs.empty()) {
      result.outputs = forced_outputs;
      return result;
    }
    for (const Buffer& input : inputs) {
      if (!fresh_copy) {
        result.outputs.push_back(input);
        result.state.intermediates.push_back(input);
        continue;
      }
      ASSIGN_OR_RETURN(auto copy, Buffer::Allocate(executor, input.size_bytes()));
      RETURN_IF_ERROR(hip::HipStatus(
          pluto_hip_memcpy_async(executor.stream(), copy.data(), input.data(), input.size_bytes(),
                                 3),
          "copy"));
      result.outputs.push_back(std::move(copy));
    }
    return result;
  }
  StatusOr<BufferVec> bwd_impl(hip::Executor&, Span<const Buffer> gradients, BackwardState,
                               LayerHooks*) override {
    ++backward_calls;
    received.assign(gradients.begin(), gradients.end());
    return received;
  }
  std::vector<ActivationType> types_;
};

TEST(LayerHooksTest, ForeignStateIsRefusedBeforeAnyHookRuns) {
  auto executor = NewExecutor();
  PassThrough first, other;
  auto input = Upload<float>(*executor, Values(16, 0.1));
  ASSERT_TRUE(input.ok());
  int hook_calls = 0;
  LayerHooks hooks;
  hooks.gradient_hook = [&](hip::Executor&, std::string_view, Span<const ActivationType>,
                            Span<Buffer>) {
    ++hook_calls;
    return OkStatus();
  };
  auto forward = first.fwd(*executor, {*input}, &hooks);
  ASSERT_TRUE(forward.ok());
  EXPECT_TRUE(forward->state.layer == &first);
  EXPECT_TRUE(IsInvalidArgument(
      other.bwd(*executor, {*input}, std::move(forward->state), &hooks).status()));
  EXPECT_EQ(other.backward_calls, 0);
  EXPECT_EQ(hook_calls, 0);
  // no hooks installed: the owner is still checked
  EXPECT_TRUE(IsInvalidArgument(other.bwd(*executor, {*input}, BackwardState{}).status()));
  EXPECT_EQ(other.backward_calls, 0);
}

TEST(LayerHooksTest, FailedForwardPublishesNothingAndCallbackErrorsStopTheCall) {
  auto executor = NewExecutor();
  PassThrough layer;
  auto input = Upload<float>(*executor, Values(16, 0.1));
  ASSERT_TRUE(input.ok());
  int activation_calls = 0;
  LayerHooks hooks;
  hooks.activation_hook = [&](hip::Executor&, std::string_view name, Span<const ActivationType>,
                              Span<Buffer>) {
    ++activation_calls;
    EXPECT_EQ(name, "PassThrough");
    return OkStatus();
  };
  layer.forward_status = FailedPreconditionError("forward body failed");
  auto broken = layer.fwd(*executor, {*input}, &hooks);
  EXPECT_TRUE(broken.status().code() == StatusCode::kFailedPrecondition);
  EXPECT_EQ(activation_calls, 0);
  layer.forward_status = OkStatus();

  hooks.activation_hook = [](hip::Executor&, std::string_view, Span<const ActivationType>,
                             Span<Buffer>) { return CancelledError("activation callback"); };
  auto stopped = layer.fwd(*executor, {*input}, &hooks);
  EXPECT_TRUE(stopped.status().code() == StatusCode::kCancelled);
  EXPECT_TRUE(testing::Contains(stopped.status().message(), "activation callback"));

  hooks.activation_hook = {};
  auto forward = layer.fwd(*executor, {*input}, &hooks);
  ASSERT_TRUE(forward.ok());
  hooks.gradient_hook = [](hip::Executor&, std::string_view, Span<const ActivationType>,
                           Span<Buffer>) { return CancelledError("gradient callback"); };
  auto backward = layer.bwd(*executor, {*input}, std::move(forward->state), &hooks);
  EXPECT_TRUE(backward.status().code() == StatusCode::kCancelled);
  EXPECT_EQ(layer.backward_calls, 0);
}

TEST(LayerHooksTest, ReplacementsLeaveTheCallersAndTheSavedHandlesAlone) {
  auto executor = NewExecutor();
  PassThrough layer;
  auto original = Upload<float>(*executor, std::vector<float>(16, 2.0f));
  auto replacement = Upload<float>(*executor, std::vector<float>(16, 5.0f));
  ASSERT_TRUE(original.ok());
  ASSERT_TRUE(replacement.ok());
  LayerHooks hooks;
  hooks.activation_hook = [&](hip::Executor&, std::string_view, Span<const ActivationType> types,
                              Span<Buffer> buffers) {
    EXPECT_EQ(types.size(), 1u);
    EXPECT_EQ(buffers.size(), 1u);
    buffers[0] = *replacement;
    return OkStatus();
  };
  auto forward = layer.fwd(*executor, {*original}, &hooks);
  ASSERT_TRUE(forward.ok());
  EXPECT_TRUE(forward->outputs[0].data() == replacement->data());
  ASSERT_EQ(forward->state.intermediates.size(), 1u);
  EXPECT_TRUE(forward->state.intermediates[0].data() == original->data());
  for (float value : Read<float>(*original)) EXPECT_EQ(value, 2.0f);

  hooks.gradient_hook = [&](hip::Executor&, std::string_view, Span<const ActivationType> types,
                            Span<Buffer> buffers) {
    EXPECT_EQ(types[0], ActivationType(DataType::FP32, {ActivationType::kBatchDimension, 4}));
    buffers[0] = *replacement;
    return OkStatus();
  };
  BufferVec incoming{*original};
  auto backward = layer.bwd(*executor, MakeConstSpan(incoming), std::move(forward->state), &hooks);
  ASSERT_TRUE(backward.ok());
  EXPECT_TRUE(incoming[0].data() == original->data());
  ASSERT_EQ(layer.received.size(), 1u);
  EXPECT_TRUE(layer.received[0].data() == replacement->data());
}

TEST(LayerHooksTest, ReplacedOutputStaysAllocatedWhileTheCallbackCopiesFromIt) {
  auto executor = NewExecutor();
  PassThrough layer;
  layer.fresh_copy = true;  // the only reference to the output is the layer's result
  auto input = Upload<float>(*executor, std::vector<float>(16, 7.0f));
  ASSERT_TRUE(input.ok());
  LayerHooks hooks;
  hooks.activation_hook = [](hip::Executor& executor, std::string_view,
                             Span<const ActivationType>, Span<Buffer> buffers) -> Status {
    const void* old_bytes = buffers[0].data();
    const size_t size = buffers[0].size_bytes();
    ASSIGN_OR_RETURN(auto replacement, Buffer::Allocate(executor, size));
    buffers[0] = std::move(replacement);
    // the dropped handle must not have been freed yet: this copy reads it
    return hip::HipStatus(
        pluto_hip_memcpy_async(executor.stream(), buffers[0].data(), old_bytes, size, 3),
        "copy out of the replaced output");
  };
  auto forward = layer.fwd(*executor, {*input}, &hooks);
  ASSERT_TRUE(forward.ok());
  EXPECT_TRUE(forward->outputs[0].data() != input->data());
  for (float value : Read<float>(forward->outputs[0])) EXPECT_EQ(value, 7.0f);
}

TEST(LayerHooksTest, WrongSizeAndForeignExecutorReplacementsAreRejected) {
  auto executor = NewExecutor();
  auto elsewhere = NewExecutor();
  auto input = Buffer::Allocate(*executor, 16 * sizeof(float));
  auto wrong_size = Buffer::Allocate(*executor, 17 * sizeof(float));
  auto foreign = Buffer::Allocate(*elsewhere, 16 * sizeof(float));
  ASSERT_TRUE(input.ok());
  ASSERT_TRUE(wrong_size.ok());
  ASSERT_TRUE(foreign.ok());
  PassThrough layer;
  for (const Buffer& replacement : {*wrong_size, *foreign}) {
    LayerHooks hooks;
    hooks.activation_hook = [&](hip::Executor&, std::string_view, Span<const ActivationType>,
                                Span<Buffer> buffers) {
      buffers[0] = replacement;
      return OkStatus();
    };
    EXPECT_TRUE(IsInvalidArgument(layer.fwd(*executor, {*input}, &hooks).status()));
    hooks.activation_hook = {};
    auto forward = layer.fwd(*executor, {*input}, &hooks);
    ASSERT_TRUE(forward.ok());
    hooks.gradient_hook = [&](hip::Executor&, std::string_view, Span<const ActivationType>,
                              Span<Buffer> buffers) {
      buffers[0] = replacement;
      return OkStatus();
    };
    EXPECT_TRUE(IsInvalidArgument(
        layer.bwd(*executor, {*input}, std::move(forward->state), &hooks).status()));
    EXPECT_EQ(layer.backward_calls, 0);
  }
  // a foreign buffer offered to the hook is refused before the hook sees it
  int calls = 0;
  LayerHooks hooks;
  hooks.gradient_hook = [&](hip::Executor&, std::string_view, Span<const ActivationType>,
                            Span<Buffer>) {
    ++calls;
    return OkStatus();
  };
  auto forward = layer.fwd(*executor, {*input}, &hooks);
  ASSERT_TRUE(forward.ok());
  EXPECT_TRUE(IsInvalidArgument(
      layer.bwd(*executor, {*foreign}, std::move(forward->state), &hooks).status()));
  EXPECT_EQ(calls, 0);
}

TEST(LayerHooksTest, CountsThatDoNotMatchTheSignatureNeverReachAHook) {
  auto executor = NewExecutor();
  auto input = Buffer::Allocate(*executor, 64);
  ASSERT_TRUE(input.ok());
  PassThrough layer;
  int calls = 0;
  LayerHooks hooks;
  auto count = [&](hip::Executor&, std::string_view, Span<const ActivationType>, Span<Buffer>) {
    ++calls;
    return OkStatus();
  };
  hooks.activation_hook = count;
  hooks.gradient_hook = count;
  layer.forced_outputs = {*input, *input};  // two outputs, one declared type
  EXPECT_TRUE(IsInvalidArgument(layer.fwd(*executor, {*input}, &hooks).status()));
  EXPECT_EQ(calls, 0);
  layer.forced_outputs.clear();
  auto forward = layer.fwd(*executor, {*input}, &hooks);
  ASSERT_TRUE(forward.ok());
  EXPECT_EQ(calls, 1);
  EXPECT_TRUE(IsInvalidArgument(
      layer.bwd(*executor, {*input, *input}, std::move(forward->state), &hooks).status()));
  EXPECT_EQ(calls, 1);
  EXPECT_EQ(layer.backward_calls, 0);
  // fewer gradients than outputs is a layer's own business: the hook sees a prefix
  PassThrough two(2);
  auto both = two.fwd(*executor, {*input, *input}, &hooks);
  ASSERT_TRUE(both.ok());
  hooks.gradient_hook = [&](hip::Executor&, std::string_view, Span<const ActivationType> types,
                            Span<Buffer> buffers) {
    EXPECT_EQ(types.size(), 1u);
    EXPECT_EQ(buffers.size(), 1u);
    EXPECT_EQ(types[0], ActivationType(DataType::FP32, {ActivationType::kBatchDimension, 4}));
    return OkStatus();
  };
  EXPECT_TRUE(two.bwd(*executor, {*input}, std::move(both->state), &hooks).ok());
  EXPECT_EQ(two.backward_calls, 1);
  // without callbacks nothing about counts is checked by the base class
  layer.forced_outputs = {*input, *input};
  LayerHooks empty;
  EXPECT_TRUE(layer.fwd(*executor, {*input}, &empty).ok());
  EXPECT_TRUE(layer.fwd(*executor, {*input}).ok());
}

// ---- DeltaNetLayer ---------------------------------------------------------

struct DeltaWeights {
  Buffer convolution, a_log, dt_bias, norm;
};

StatusOr<DeltaWeights> MakeWeights(hip::Executor& executor, const DeltaNetParameters& p) {
  const int channels = 2 * p.key_heads * p.key_head_dim + p.value_heads * p.value_head_dim;
  ASSIGN_OR_RETURN(auto convolution,
                   Upload<float>(executor, Values(channels * p.conv_kernel_dim, 0.73, 0.6)));
  ASSIGN_OR_RETURN(auto a_log, Upload<float>(executor, Values(p.value_heads, 0.18, 0.5)));
  ASSIGN_OR_RETURN(auto dt_bias, Upload<float>(executor, Values(p.value_heads, -0.7, 0.3)));
  ASSIGN_OR_RETURN(auto norm, Upload<float>(executor, Values(p.value_head_dim, 0.5, 0.6)));
  return DeltaWeights{std::move(convolution), std::move(a_log), std::move(dt_bias),
                      std::move(norm)};
}

DeltaNetParameters SmallDelta() {
  DeltaNetParameters p;
  p.key_heads = 2;
  p.value_heads = 6;
  p.key_head_dim = 5;
  p.value_head_dim = 7;
  p.conv_kernel_dim = 4;
  return p;
}

TEST(DeltaNetLayerTest, CreateChecksDimensionsWeightsAndExecutor) {
  auto executor = NewExecutor();
  auto elsewhere = NewExecutor();
  const DeltaNetParameters p = SmallDelta();
  auto w = MakeWeights(*executor, p);
  auto foreign = MakeWeights(*elsewhere, p);
  ASSERT_TRUE(w.ok());
  ASSERT_TRUE(foreign.ok());
  auto layer = DeltaNetLayer::Create(*executor, p, w->convolution, w->a_log, w->dt_bias, w->norm);
  ASSERT_TRUE(layer.ok());
  const int64_t batch = ActivationType::kBatchDimension;
  ASSERT_EQ((*layer)->input_types().size(), 4u);
  EXPECT_EQ((*layer)->input_types()[0], ActivationType(DataType::BF16, {batch, 1, 62}));
  EXPECT_EQ((*layer)->input_types()[1], ActivationType(DataType::BF16, {batch, 1, 42}));
  EXPECT_EQ((*layer)->input_types()[2], ActivationType(DataType::BF16, {batch, 1, 6}));
  EXPECT_EQ((*layer)->input_types()[3], ActivationType(DataType::BF16, {batch, 1, 6}));
  ASSERT_EQ((*layer)->output_types().size(), 1u);
  EXPECT_EQ((*layer)->output_types()[0], ActivationType(DataType::BF16, {batch, 1, 42}));
  EXPECT_EQ((*layer)->weights().size(), 4u);
  EXPECT_EQ((*layer)->name(), "DeltaNetLayer");

  for (int field = 0; field < 5; ++field) {
    DeltaNetParameters bad = p;
    int* fields[] = {&bad.key_heads, &bad.value_heads, &bad.key_head_dim, &bad.value_head_dim,
                     &bad.conv_kernel_dim};
    *fields[field] = 0;
    EXPECT_TRUE(IsInvalidArgument(
        DeltaNetLayer::Create(*executor, bad, w->convolution, w->a_log, w->dt_bias, w->norm)
            .status()));
  }
  DeltaNetParameters wide = p;
  wide.key_heads = 1 << 20;  // 2 * key width alone passes the layer width limit
  wide.value_heads = 1 << 20;
  EXPECT_TRUE(IsInvalidArgument(
      DeltaNetLayer::Create(*executor, wide, w->convolution, w->a_log, w->dt_bias, w->norm)
          .status()));
  wide.key_heads = wide.key_head_dim = wide.value_heads = wide.value_head_dim = 2147483647;
  EXPECT_TRUE(IsInvalidArgument(
      DeltaNetLayer::Create(*executor, wide, w->convolution, w->a_log, w->dt_bias, w->norm)
          .status()));
  // each weight: wrong extent, then the right extent on another executor
  EXPECT_TRUE(IsInvalidArgument(
      DeltaNetLayer::Create(*executor, p, w->a_log, w->a_log, w->dt_bias, w->norm).status()));
  EXPECT_TRUE(IsInvalidArgument(
      DeltaNetLayer::Create(*executor, p, w->convolution, w->norm, w->dt_bias, w->norm).status()));
  EXPECT_TRUE(IsInvalidArgument(
      DeltaNetLayer::Create(*executor, p, w->convolution, w->a_log, w->norm, w->norm).status()));
  EXPECT_TRUE(IsInvalidArgument(
      DeltaNetLayer::Create(*executor, p, w->convolution, w->a_log, w->dt_bias, w->a_log)
          .status()));
  EXPECT_TRUE(IsInvalidArgument(
      DeltaNetLayer::Create(*executor, p, foreign->convolution, w->a_log, w->dt_bias, w->norm)
          .status()));
  EXPECT_TRUE(IsInvalidArgument(
      DeltaNetLayer::Create(*executor, p, w->convolution, w->a_log, w->dt_bias, foreign->norm)
          .status()));
  // what only the state object knows: value heads in whole groups of key heads
  DeltaNetParameters ungrouped = p;
  ungrouped.value_heads = 5;
  auto uw = MakeWeights(*executor, ungrouped);
  ASSERT_TRUE(uw.ok());
  EXPECT_TRUE(IsInvalidArgument(DeltaNetLayer::Create(*executor, ungrouped, uw->convolution,
                                                      uw->a_log, uw->dt_bias, uw->norm)
                                    .status()));
}

TEST(DeltaNetLayerTest, ForwardIsTheFloatStepBetweenCastsAndRejectsBadInputs) {
  auto executor = NewExecutor();
  auto elsewhere = NewExecutor();
  for (const bool full_width : {false, true}) {
    DeltaNetParameters p = SmallDelta();
    if (full_width) p.key_head_dim = p.value_head_dim = 128;
    const int channels = 2 * p.key_heads * p.key_head_dim + p.value_heads * p.value_head_dim;
    const int values = p.value_heads * p.value_head_dim;
    auto w = MakeWeights(*executor, p);
    ASSERT_TRUE(w.ok());
    auto layer =
        DeltaNetLayer::Create(*executor, p, w->convolution, w->a_log, w->dt_bias, w->norm);
    ASSERT_TRUE(layer.ok());
    auto state = cached_attention_ops::DeltaNetState::Create(*executor, p);
    ASSERT_TRUE(state.ok());
    for (int token = 0; token < 5; ++token) {
      const auto qkv = testing::RoundedToBFloat16(Values(channels, 0.3 + 0.71 * token));
      const auto z = testing::RoundedToBFloat16(Values(values, -0.6 + 0.27 * token));
      const auto a = testing::RoundedToBFloat16(Values(p.value_heads, 0.1 + 0.1 * token));
      const auto b = testing::RoundedToBFloat16(Values(p.value_heads, -0.7 + 0.3 * token));
      auto qkv16 = Upload<BFloat16>(*executor, qkv), z16 = Upload<BFloat16>(*executor, z),
           a16 = Upload<BFloat16>(*executor, a), b16 = Upload<BFloat16>(*executor, b);
      auto qkv32 = Upload<float>(*executor, qkv), z32 = Upload<float>(*executor, z),
           a32 = Upload<float>(*executor, a), b32 = Upload<float>(*executor, b);
      ASSERT_TRUE(qkv16.ok() && z16.ok() && a16.ok() && b16.ok());
      ASSERT_TRUE(qkv32.ok() && z32.ok() && a32.ok() && b32.ok());
      auto forward = (*layer)->fwd(*executor, {*qkv16, *z16, *a16, *b16});
      ASSERT_TRUE(forward.ok());
      ASSERT_EQ(forward->outputs.size(), 1u);
      ASSERT_EQ(forward->outputs[0].size_bytes(), static_cast<size_t>(values) * 2);
      auto expected = Buffer::Allocate(*executor, static_cast<size_t>(values) * sizeof(float));
      ASSERT_TRUE(expected.ok());
      auto f = [](const Buffer& buffer) { return static_cast<const float*>(buffer.data()); };
      ASSERT_TRUE((*state)
                      ->Step(f(*qkv32), f(*z32), f(*a32), f(*b32), f(w->convolution), f(w->a_log),
                             f(w->dt_bias), f(w->norm), static_cast<float*>(expected->data()))
                      .ok());
      const auto got = Read<BFloat16>(forward->outputs[0]);
      const auto want = testing::RoundedToBFloat16(Read<float>(*expected));
      int differing = 0;
      for (int i = 0; i < values; ++i) differing += got[i] != want[i];
      EXPECT_EQ(differing, 0) << "token" << token << "full width" << full_width;
    }
    // Reset replays the first token bit for bit
    const auto qkv = Values(channels, 0.3), z = Values(values, -0.6);
    const auto a = Values(p.value_heads, 0.1), b = Values(p.value_heads, -0.7);
    auto qkv16 = Upload<BFloat16>(*executor, qkv), z16 = Upload<BFloat16>(*executor, z),
         a16 = Upload<BFloat16>(*executor, a), b16 = Upload<BFloat16>(*executor, b);
    ASSERT_TRUE(qkv16.ok() && z16.ok() && a16.ok() && b16.ok());
    ASSERT_TRUE((*layer)->Reset().ok());
    auto once = (*layer)->fwd(*executor, {*qkv16, *z16, *a16, *b16});
    ASSERT_TRUE((*layer)->Reset().ok());
    auto again = (*layer)->fwd(*executor, {*qkv16, *z16, *a16, *b16});
    ASSERT_TRUE(once.ok() && again.ok());
    EXPECT_TRUE(Read<BFloat16>(once->outputs[0]) == Read<BFloat16>(again->outputs[0]));

    // wrong count, wrong extent, other executor, no backward
    EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*qkv16, *z16, *a16}).status()));
    EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*z16, *z16, *a16, *b16}).status()));
    EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*qkv16, *z16, *a16, *z16}).status()));
    EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*elsewhere, {*qkv16, *z16, *a16, *b16}).status()));
    EXPECT_TRUE(IsUnimplemented(
        (*layer)->bwd(*executor, {once->outputs[0]}, std::move(once->state)).status()));
  }
}

}  // namespace
}  // namespace pluto::llm
