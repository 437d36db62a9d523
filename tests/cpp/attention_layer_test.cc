// AttentionLayer through the host API; cases follow
// src/llm/layers/attention_test.cc and src/llm/layer_test.cc, with the CPU
// oracle as the numerical reference.
#include "pluto_amd/host/attention.h"
#include "pluto_amd/host/layer_hooks.h"
#include "tests/cpp/test_support.h"

namespace pluto::llm {
namespace {

using testing::BFloat16;
using testing::Contains;
using testing::NewExecutor;
using testing::Read;
using testing::Upload;
using testing::Values;

constexpr int kTokens = 32, kWidth = 32, kContext = 4, kHeads = 2;

TEST(AttentionLayerTest, CreateRejectsUnsupportedPoliciesAndShapes) {
  auto executor = NewExecutor();
  EXPECT_TRUE(IsUnimplemented(
      AttentionLayer::Create(*executor, 4, 2, 32, DataType::FP8).status()));
  EXPECT_TRUE(IsUnimplemented(
      AttentionLayer::Create(*executor, 4, 2, 32, DataType::FP32).status()));
  EXPECT_TRUE(IsInvalidArgument(AttentionLayer::Create(*executor, 0, 2, 32, DataType::FP16).status()));
  EXPECT_TRUE(IsInvalidArgument(AttentionLayer::Create(*executor, 4, 0, 32, DataType::FP16).status()));
  EXPECT_TRUE(IsInvalidArgument(AttentionLayer::Create(*executor, 4, 3, 32, DataType::FP16).status()));
  auto layer = AttentionLayer::Create(*executor, 4, 2, 32, DataType::BF16);
  ASSERT_TRUE(layer.ok());
  EXPECT_EQ((*layer)->input_types()[0],
            ActivationType(DataType::BF16, {ActivationType::kBatchDimension, 4, 96}));
  EXPECT_EQ((*layer)->output_types()[0],
            ActivationType(DataType::BF16, {ActivationType::kBatchDimension, 4, 32}));
  EXPECT_TRUE((*layer)->weights().empty());
  EXPECT_EQ((*layer)->name(), "AttentionLayer");
}

TEST(AttentionLayerTest, FlashAttentionIsCausalAndHasCorrectSingleTokenGradient) {
  auto executor = NewExecutor();
  auto attention = AttentionLayer::Create(*executor, kContext, kHeads, kWidth, DataType::FP16);
  ASSERT_TRUE(attention.ok());
  constexpr int kPacked = 3 * kWidth;
  std::vector<float> input(kTokens * kPacked, 0.0f);
  input[0] = input[kWidth] = input[2 * kWidth] = 1.0f;
  input[kPacked] = input[kPacked + kWidth] = input[kPacked + 2 * kWidth] = 2.0f;
  input[2 * kPacked + 2 * kWidth] = 4.0f;  // a future value position zero must not see
  auto input_buffer = Upload<float>(*executor, input);
  ASSERT_TRUE(input_buffer.ok());
  auto output = (*attention)->fwd(*executor, {*input_buffer});
  ASSERT_TRUE(output.ok());
  EXPECT_TRUE(output->state.layer == attention->get());
  std::vector<float> output_gradient(kTokens * kWidth, 0.0f);
  output_gradient[0] = 1.0f;
  auto gradient_buffer = Upload<float>(*executor, output_gradient);
  ASSERT_TRUE(gradient_buffer.ok());
  auto input_gradient = (*attention)->bwd(*executor, {*gradient_buffer}, std::move(output->state));
  ASSERT_TRUE(input_gradient.ok());
  ASSERT_EQ(input_gradient->size(), 1u);
  const auto host_output = Read<float>(output->outputs[0]);
  const auto host_gradient = Read<float>(input_gradient->front());
  const float scale = 1.0f / std::sqrt(static_cast<float>(kWidth / kHeads));
  const float first = std::exp(2.0f * scale), second = std::exp(4.0f * scale);
  EXPECT_NEAR(host_output[0], 1.0f, 1e-6f);
  EXPECT_NEAR(host_output[kWidth], (first + 2.0f * second) / (first + second), 1e-5f);
  EXPECT_NEAR(host_gradient[0], 0.0f, 1e-6f);
  EXPECT_NEAR(host_gradient[kWidth], 0.0f, 1e-6f);
  EXPECT_NEAR(host_gradient[2 * kWidth], 1.0f, 1e-6f);
  EXPECT_NEAR(host_gradient[kPacked], 0.0f, 1e-6f);
}

void CompareWithOracle(DataType policy, int rows, int context, int heads, int width) {
  auto executor = NewExecutor();
  auto layer = AttentionLayer::Create(*executor, context, heads, width, policy);
  ASSERT_TRUE(layer.ok());
  const bool bf16 = policy == DataType::BF16;
  auto qkv = Values(static_cast<size_t>(rows) * 3 * width, 0.3, 0.9);
  if (bf16) qkv = testing::RoundedToBFloat16(qkv);
  const auto d_out = Values(static_cast<size_t>(rows) * width, 1.7, 0.5);
  auto input = bf16 ? Upload<BFloat16>(*executor, qkv) : Upload<float>(*executor, qkv);
  auto gradient = Upload<float>(*executor, d_out);
  ASSERT_TRUE(input.ok());
  ASSERT_TRUE(gradient.ok());
  auto forward = (*layer)->fwd(*executor, {*input});
  ASSERT_TRUE(forward.ok());
  const auto out = bf16 ? Read<BFloat16>(forward->outputs[0]) : Read<float>(forward->outputs[0]);
  ASSERT_EQ(forward->state.intermediates.size(), 4u);
  const auto maxima = Read<float>(forward->state.intermediates[2]);
  const auto normalizers = Read<float>(forward->state.intermediates[3]);
  auto backward = (*layer)->bwd(*executor, {*gradient}, std::move(forward->state));
  ASSERT_TRUE(backward.ok());
  const auto d_qkv = Read<float>((*backward)[0]);

  // The oracle takes the same physical storage the layer saw.
  std::vector<BFloat16> bits(qkv.size());
  for (size_t i = 0; i < qkv.size(); ++i) bits[i] = pluto_oracle_f32_to_bf16(qkv[i]);
  const void* oracle_in = bf16 ? static_cast<const void*>(bits.data()) : qkv.data();
  std::vector<float> want_out_f(out.size()), want_max(maxima.size()), want_norm(maxima.size()),
      want_grad(d_qkv.size());
  std::vector<BFloat16> want_out_b(out.size());
  void* oracle_out = bf16 ? static_cast<void*>(want_out_b.data()) : want_out_f.data();
  const int dtype = bf16 ? PLUTO_ORACLE_BF16 : PLUTO_ORACLE_F32;
  ASSERT_EQ(pluto_oracle_mha_fwd(dtype, oracle_in, rows, context, heads, width, oracle_out,
                                 want_max.data(), want_norm.data(), 0, rows / context, 0, heads), 0);
  ASSERT_EQ(pluto_oracle_mha_bwd(dtype, oracle_in, oracle_out, d_out.data(), rows, context, heads,
                                 width, want_grad.data(), 0, rows / context, 0, heads), 0);
  const double tolerance = bf16 ? 2e-2 : 1e-4;
  double worst_out = 0, worst_grad = 0, scale_grad = 0;
  for (size_t i = 0; i < out.size(); ++i) {
    const double want = bf16 ? pluto_oracle_bf16_to_f32(want_out_b[i]) : want_out_f[i];
    worst_out = std::max(worst_out, std::fabs(out[i] - want));
  }
  for (size_t i = 0; i < d_qkv.size(); ++i) {
    worst_grad = std::max(worst_grad, std::fabs(double(d_qkv[i]) - want_grad[i]));
    scale_grad = std::max(scale_grad, std::fabs(double(want_grad[i])));
  }
  EXPECT_LE(worst_out, tolerance);
  EXPECT_LE(worst_grad, tolerance * scale_grad);
  for (size_t i = 0; i < maxima.size(); ++i) {
    EXPECT_NEAR(maxima[i], want_max[i], 1e-4 + 1e-4 * std::fabs(want_max[i]));
    EXPECT_NEAR(normalizers[i], want_norm[i], (bf16 ? 2e-2 : 1e-4) * want_norm[i]);
  }
}

TEST(AttentionLayerTest, Float32ForwardAndBackwardMatchTheOracle) {
  CompareWithOracle(DataType::FP16, 24, 12, 3, 21);  // odd head width: generic kernels
}

TEST(AttentionLayerTest, BFloat16MatrixCorePathMatchesTheOracle) {
  CompareWithOracle(DataType::BF16, 512, 256, 2, 128);  // head width 64: MFMA kernels
}

TEST(AttentionLayerTest, ForwardAndBackwardAreBitwiseRepeatable) {
  auto executor = NewExecutor();
  auto layer = AttentionLayer::Create(*executor, 128, 4, 256, DataType::BF16);
  ASSERT_TRUE(layer.ok());
  auto input = Upload<BFloat16>(*executor, Values(256 * 768, 0.1));
  auto gradient = Upload<float>(*executor, Values(256 * 256, 0.7));
  ASSERT_TRUE(input.ok());
  ASSERT_TRUE(gradient.ok());
  std::vector<float> first_out, first_grad;
  for (int repetition = 0; repetition < 3; ++repetition) {
    auto forward = (*layer)->fwd(*executor, {*input});
    ASSERT_TRUE(forward.ok());
    auto backward = (*layer)->bwd(*executor, {*gradient}, std::move(forward->state));
    ASSERT_TRUE(backward.ok());
    const auto out = Read<BFloat16>(forward->outputs[0]);
    const auto grad = Read<float>((*backward)[0]);
    if (repetition == 0) {
      first_out = out;
      first_grad = grad;
    } else {
      EXPECT_TRUE(out == first_out);
      EXPECT_TRUE(grad == first_grad);
    }
  }
}

TEST(AttentionLayerTest, SavedForwardStateSurvivesAnotherForwardPass) {
  auto executor = NewExecutor();
  auto layer = AttentionLayer::Create(*executor, 8, 2, 16, DataType::FP16);
  ASSERT_TRUE(layer.ok());
  auto a = Upload<float>(*executor, Values(16 * 48, 0.1));
  auto b = Upload<float>(*executor, Values(16 * 48, 2.1));
  auto gradient = Upload<float>(*executor, Values(16 * 16, 0.7));
  ASSERT_TRUE(a.ok());
  ASSERT_TRUE(b.ok());
  ASSERT_TRUE(gradient.ok());
  auto alone = (*layer)->fwd(*executor, {*a});
  ASSERT_TRUE(alone.ok());
  auto expected = (*layer)->bwd(*executor, {*gradient}, std::move(alone->state));
  ASSERT_TRUE(expected.ok());
  auto first = (*layer)->fwd(*executor, {*a});
  auto second = (*layer)->fwd(*executor, {*b});
  ASSERT_TRUE(first.ok());
  ASSERT_TRUE(second.ok());
  auto actual = (*layer)->bwd(*executor, {*gradient}, std::move(first->state));
  ASSERT_TRUE(actual.ok());
  EXPECT_TRUE(Read<float>((*actual)[0]) == Read<float>((*expected)[0]));
}

TEST(AttentionLayerTest, ProbabilityHookSeesCausalRowsAndLeavesResultsUnchanged) {
  auto executor = NewExecutor();
  constexpr int kRows = 12, kT = 6, kH = 2, kE = 10;
  auto layer = AttentionLayer::Create(*executor, kT, kH, kE, DataType::FP16);
  ASSERT_TRUE(layer.ok());
  auto input = Upload<float>(*executor, Values(kRows * 3 * kE, 0.4));
  ASSERT_TRUE(input.ok());
  auto plain = (*layer)->fwd(*executor, {*input});
  ASSERT_TRUE(plain.ok());
  int calls = 0;
  LayerHooks hooks;
  hooks.attention_probabilities_hook = [&](hip::Executor&, std::string_view name,
                                           const ActivationType& type, const Buffer& buffer) {
    ++calls;
    EXPECT_EQ(name, "AttentionLayer");
    EXPECT_EQ(type, ActivationType(DataType::FP32, {kRows / kT, kH, kT, kT}));
    const auto probabilities = Read<float>(buffer);
    EXPECT_EQ(probabilities.size(), size_t{kRows / kT * kH * kT * kT});
    for (int row = 0; row < kRows / kT * kH * kT; ++row) {
      double sum = 0;
      for (int key = 0; key < kT; ++key) {
        const float value = probabilities[row * kT + key];
        if (key > row % kT) EXPECT_EQ(value, 0.0f);
        sum += value;
      }
      EXPECT_NEAR(sum, 1.0, 2e-6);
    }
    return OkStatus();
  };
  auto inspected = (*layer)->fwd(*executor, {*input}, &hooks);
  ASSERT_TRUE(inspected.ok());
  EXPECT_EQ(calls, 1);
  EXPECT_TRUE(Read<float>(inspected->outputs[0]) == Read<float>(plain->outputs[0]));
}

TEST(AttentionLayerTest, ProbabilityHookFailurePreventsOutputPublication) {
  auto executor = NewExecutor();
  auto layer = AttentionLayer::Create(*executor, 2, 1, 7, DataType::FP16);
  ASSERT_TRUE(layer.ok());
  auto input = Upload<float>(*executor, std::vector<float>(2 * 3 * 7, 0.25f));
  ASSERT_TRUE(input.ok());
  int probability_calls = 0, activation_calls = 0;
  LayerHooks hooks;
  hooks.attention_probabilities_hook = [&](hip::Executor&, std::string_view, const ActivationType&,
                                           const Buffer&) {
    ++probability_calls;
    return CancelledError("probability inspection stopped");
  };
  hooks.activation_hook = [&](hip::Executor&, std::string_view, Span<const ActivationType>,
                              Span<Buffer>) {
    ++activation_calls;
    return OkStatus();
  };
  auto failed = (*layer)->fwd(*executor, {*input}, &hooks);
  ASSERT_FALSE(failed.ok());
  EXPECT_TRUE(failed.status().code() == StatusCode::kCancelled);
  EXPECT_TRUE(Contains(failed.status().message(), "probability inspection stopped"));
  EXPECT_EQ(probability_calls, 1);
  EXPECT_EQ(activation_calls, 0);
  hooks.attention_probabilities_hook = {};
  auto successful = (*layer)->fwd(*executor, {*input}, &hooks);
  ASSERT_TRUE(successful.ok());
  EXPECT_EQ(probability_calls, 1);
  EXPECT_EQ(activation_calls, 1);
}

TEST(AttentionLayerTest, ForwardRejectsBadInputsBeforeWork) {
  auto executor = NewExecutor();
  auto other = NewExecutor();
  auto layer = AttentionLayer::Create(*executor, 4, 1, 16, DataType::FP16);
  ASSERT_TRUE(layer.ok());
  auto partial = hip::Buffer::Allocate(*executor, 3 * 48 * sizeof(float));
  auto ragged = hip::Buffer::Allocate(*executor, 4 * 48 * sizeof(float) + 4);
  auto foreign = hip::Buffer::Allocate(*other, 4 * 48 * sizeof(float));
  auto good = hip::Buffer::Allocate(*executor, 4 * 48 * sizeof(float));
  ASSERT_TRUE(partial.ok());
  ASSERT_TRUE(ragged.ok());
  ASSERT_TRUE(foreign.ok());
  ASSERT_TRUE(good.ok());
  auto result = (*layer)->fwd(*executor, {*partial});
  EXPECT_TRUE(IsInvalidArgument(result.status()));
  EXPECT_TRUE(Contains(result.status().message(), "divisible by context_length"));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*ragged}).status()));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*foreign}).status()));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*good, *good}).status()));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*other, {*foreign}).status()));
}

TEST(AttentionLayerTest, BackwardRejectsForeignOrUnusedStates) {
  auto executor = NewExecutor();
  auto first = AttentionLayer::Create(*executor, 4, 1, 16, DataType::FP16);
  auto second = AttentionLayer::Create(*executor, 4, 1, 16, DataType::FP16);
  ASSERT_TRUE(first.ok());
  ASSERT_TRUE(second.ok());
  auto input = Upload<float>(*executor, Values(4 * 48, 0.2));
  auto gradient = Upload<float>(*executor, Values(4 * 16, 0.2));
  ASSERT_TRUE(input.ok());
  ASSERT_TRUE(gradient.ok());
  EXPECT_TRUE(IsInvalidArgument((*first)->bwd(*executor, {*gradient}, BackwardState{}).status()));
  auto forward = (*first)->fwd(*executor, {*input});
  ASSERT_TRUE(forward.ok());
  EXPECT_TRUE(IsInvalidArgument(
      (*second)->bwd(*executor, {*gradient}, forward->state).status()));
  EXPECT_TRUE((*first)->bwd(*executor, {*gradient}, std::move(forward->state)).ok());
}

TEST(AttentionLayerTest, BackwardRejectsPartialSequencesBeforeGatheringQueries) {
  auto executor = NewExecutor();
  constexpr int kC = 4, kW = 16, kR = 3;
  auto attention = AttentionLayer::Create(*executor, kC, 1, kW, DataType::FP16);
  auto qkv = hip::Buffer::Allocate(*executor, kR * 3 * kW * sizeof(float));
  auto output = hip::Buffer::Allocate(*executor, kR * kW * sizeof(float));
  auto gradient = hip::Buffer::Allocate(*executor, kR * kW * sizeof(float));
  auto statistics = hip::Buffer::Allocate(*executor, kR * sizeof(float));
  ASSERT_TRUE(attention.ok());
  BackwardState state;
  state.layer = attention->get();
  state.intermediates = {*qkv, *output, *statistics, *statistics};
  auto result = (*attention)->bwd(*executor, {*gradient}, std::move(state));
  ASSERT_FALSE(result.ok());
  EXPECT_TRUE(IsInvalidArgument(result.status()));
  EXPECT_TRUE(Contains(result.status().message(), "divisible by context_length"));
}

TEST(AttentionLayerTest, BackwardRejectsInvalidSoftmaxStatistics) {
  auto executor = NewExecutor();
  auto other = NewExecutor();
  constexpr int kC = 4, kH = 2, kW = 32, kR = 2 * kC;
  constexpr size_t kStatisticsBytes = kR * kH * sizeof(float);
  auto attention = AttentionLayer::Create(*executor, kC, kH, kW, DataType::FP16);
  auto qkv = hip::Buffer::Allocate(*executor, kR * 3 * kW * sizeof(float));
  auto output = hip::Buffer::Allocate(*executor, kR * kW * sizeof(float));
  auto gradient = hip::Buffer::Allocate(*executor, kR * kW * sizeof(float));
  auto statistics = hip::Buffer::Allocate(*executor, kStatisticsBytes);
  auto shorter = hip::Buffer::Allocate(*executor, kStatisticsBytes - sizeof(float));
  auto longer = hip::Buffer::Allocate(*executor, kStatisticsBytes + sizeof(float));
  auto foreign = hip::Buffer::Allocate(*other, kStatisticsBytes);
  ASSERT_TRUE(attention.ok());
  for (int index : {2, 3})
    for (const auto& invalid : {*shorter, *longer, *foreign}) {
      BackwardState state;
      state.layer = attention->get();
      state.intermediates = {*qkv, *output, *statistics, *statistics};
      state.intermediates[index] = invalid;
      auto result = (*attention)->bwd(*executor, {*gradient}, std::move(state));
      ASSERT_FALSE(result.ok());
      EXPECT_TRUE(IsInvalidArgument(result.status()));
      EXPECT_TRUE(Contains(result.status().message(),
                           index == 2 ? "saved maxima" : "saved normalizers"));
    }
}

TEST(AttentionLayerTest, GradientHookSeesFloatGradientsBeforeBackward) {
  auto executor = NewExecutor();
  auto layer = AttentionLayer::Create(*executor, 4, 1, 16, DataType::BF16);
  ASSERT_TRUE(layer.ok());
  auto input = Upload<BFloat16>(*executor, Values(4 * 48, 0.2));
  auto gradient = Upload<float>(*executor, Values(4 * 16, 0.2));
  auto zeros = Upload<float>(*executor, std::vector<float>(4 * 16, 0.0f));
  ASSERT_TRUE(input.ok());
  auto forward = (*layer)->fwd(*executor, {*input});
  ASSERT_TRUE(forward.ok());
  LayerHooks hooks;
  int calls = 0;
  hooks.gradient_hook = [&](hip::Executor&, std::string_view, Span<const ActivationType> types,
                            Span<Buffer> gradients) {
    ++calls;
    EXPECT_EQ(types.size(), 1u);
    EXPECT_EQ(types[0], ActivationType(DataType::FP32, {ActivationType::kBatchDimension, 4, 16}));
    gradients[0] = *zeros;  // same byte size, same executor: accepted
    return OkStatus();
  };
  auto backward = (*layer)->bwd(*executor, {*gradient}, std::move(forward->state), &hooks);
  ASSERT_TRUE(backward.ok());
  EXPECT_EQ(calls, 1);
  for (float value : Read<float>((*backward)[0])) EXPECT_EQ(value, 0.0f);
}

}  // namespace
}  // namespace pluto::llm
