// FullyConnectedLayer through the host API; the first two cases follow
// src/llm/layers/fully_connected_test.cc:19-131, the others compare with the
// CPU oracle and check the gradient-overwrite and repeatability contracts.
#include "pluto_amd/host/fully_connected.h"

#include "tests/cpp/test_support.h"

namespace pluto::llm {
namespace {

using testing::BFloat16;
using testing::NewExecutor;
using testing::Read;
using testing::Upload;
using testing::Values;

constexpr int kTokens = 32, kWidth = 32;

TEST(FullyConnectedLayerTest, CreateValidatesItsArguments) {
  auto executor = NewExecutor();
  EXPECT_TRUE(IsInvalidArgument(
      FullyConnectedLayer::Create(*executor, 8, 8, DataType::FP16, 0).status()));
  EXPECT_TRUE(IsInvalidArgument(FullyConnectedLayer::Create(*executor, 0, 8, DataType::FP16).status()));
  EXPECT_TRUE(IsInvalidArgument(FullyConnectedLayer::Create(*executor, 8, -1, DataType::FP16).status()));
  EXPECT_TRUE(IsUnimplemented(FullyConnectedLayer::Create(*executor, 8, 8, DataType::FP8).status()));
  auto layer = FullyConnectedLayer::Create(*executor, 24, 40, DataType::BF16, 6);
  ASSERT_TRUE(layer.ok());
  EXPECT_EQ((*layer)->name(), "FullyConnectedLayer");
  EXPECT_EQ((*layer)->input_types()[0],
            ActivationType(DataType::BF16, {ActivationType::kBatchDimension, 6, 24}));
  EXPECT_EQ((*layer)->output_types()[0],
            ActivationType(DataType::BF16, {ActivationType::kBatchDimension, 6, 40}));
  ASSERT_EQ((*layer)->weights().size(), 2u);
  ASSERT_EQ((*layer)->gradients().size(), 2u);
  EXPECT_EQ((*layer)->weights()[0].size_bytes(), 24u * 40u * sizeof(float));
  EXPECT_EQ((*layer)->weights()[1].size_bytes(), 40u * sizeof(float));
  // parameters and gradients start at zero
  for (const Buffer& buffer : (*layer)->weights())
    for (float value : Read<float>(buffer)) EXPECT_EQ(value, 0.0f);
  for (const Buffer& buffer : (*layer)->gradients())
    for (float value : Read<float>(buffer)) EXPECT_EQ(value, 0.0f);
  EXPECT_TRUE(IsInvalidArgument((*layer)->InitializeNormal(0.0f, 1)));
}

TEST(FullyConnectedLayerTest, IdentityDenseLayerHasIdentityForwardAndBackward) {
  auto executor = NewExecutor();
  std::vector<float> input(kTokens * kWidth), output_gradient(input.size());
  for (size_t index = 0; index < input.size(); ++index) {
    input[index] = static_cast<float>(static_cast<int>(index % 17) - 8) / 8;
    output_gradient[index] = static_cast<float>(static_cast<int>(index % 9) - 4) / 8;
  }
  auto input_buffer = Upload<float>(*executor, input);
  auto gradient_buffer = Upload<float>(*executor, output_gradient);
  ASSERT_TRUE(input_buffer.ok());
  ASSERT_TRUE(gradient_buffer.ok());
  auto dense = FullyConnectedLayer::Create(*executor, kWidth, DataType::FP16);
  ASSERT_TRUE(dense.ok());
  ASSERT_TRUE((*dense)->InitializeIdentity().ok());
  auto output = (*dense)->fwd(*executor, {*input_buffer});
  ASSERT_TRUE(output.ok());
  auto input_gradients = (*dense)->bwd(*executor, {*gradient_buffer}, std::move(output->state));
  ASSERT_TRUE(input_gradients.ok());
  ASSERT_EQ(input_gradients->size(), 1u);
  const auto host_output = Read<float>(output->outputs[0]);
  const auto host_input_gradient = Read<float>(input_gradients->front());
  for (size_t index = 0; index < input.size(); ++index) {
    EXPECT_NEAR(host_output[index], input[index], 1e-6f);
    EXPECT_NEAR(host_input_gradient[index], output_gradient[index], 1e-6f);
  }
}

TEST(FullyConnectedLayerTest, RectangularProjectionUsesDistinctInputAndOutputWidths) {
  auto executor = NewExecutor();
  constexpr int kOutputWidth = 48;
  auto dense = FullyConnectedLayer::Create(*executor, kWidth, kOutputWidth, DataType::FP16);
  ASSERT_TRUE(dense.ok());
  ASSERT_EQ((*dense)->input_dim(), kWidth);
  ASSERT_EQ((*dense)->output_dim(), kOutputWidth);
  ASSERT_TRUE((*dense)->InitializeIdentity().ok());
  std::vector<float> input(kTokens * kWidth);
  for (size_t index = 0; index < input.size(); ++index) input[index] = static_cast<float>(index % 7);
  auto input_buffer = Upload<float>(*executor, input);
  ASSERT_TRUE(input_buffer.ok());
  auto output = (*dense)->fwd(*executor, {*input_buffer});
  ASSERT_TRUE(output.ok());
  const auto host_output = Read<float>(output->outputs[0]);
  for (int row = 0; row < kTokens; ++row) {
    for (int column = 0; column < kWidth; ++column)
      EXPECT_EQ(host_output[row * kOutputWidth + column], input[row * kWidth + column]);
    for (int column = kWidth; column < kOutputWidth; ++column)
      EXPECT_EQ(host_output[row * kOutputWidth + column], 0.0f);
  }
}

void CompareWithOracle(DataType policy, int rows, int input_dim, int output_dim) {
  auto executor = NewExecutor();
  auto layer = FullyConnectedLayer::Create(*executor, input_dim, output_dim, policy);
  ASSERT_TRUE(layer.ok());
  ASSERT_TRUE((*layer)->InitializeNormal(0.05f, 7).ok());
  const bool bf16 = policy == DataType::BF16;
  auto x = Values(static_cast<size_t>(rows) * input_dim, 0.4, 0.8);
  if (bf16) x = testing::RoundedToBFloat16(x);
  const auto bias = Values(output_dim, 2.1, 0.3);
  const auto dy = Values(static_cast<size_t>(rows) * output_dim, 1.3, 0.6);
  auto bias_buffer = Upload<float>(*executor, bias);
  ASSERT_TRUE(bias_buffer.ok());
  ASSERT_EQ(pluto_hip_memcpy_async(executor->stream(), (*layer)->weights()[1].data(),
                                   bias_buffer->data(), bias_buffer->size_bytes(), 3), 0);
  auto input = bf16 ? Upload<BFloat16>(*executor, x) : Upload<float>(*executor, x);
  auto gradient = Upload<float>(*executor, dy);
  ASSERT_TRUE(input.ok());
  ASSERT_TRUE(gradient.ok());
  const auto matrix = Read<float>((*layer)->weights()[0]);
  auto forward = (*layer)->fwd(*executor, {*input});
  ASSERT_TRUE(forward.ok());
  const auto y = bf16 ? Read<BFloat16>(forward->outputs[0]) : Read<float>(forward->outputs[0]);
  auto backward = (*layer)->bwd(*executor, {*gradient}, std::move(forward->state));
  ASSERT_TRUE(backward.ok());
  const auto dx = Read<float>((*backward)[0]);
  const auto dw = Read<float>((*layer)->gradients()[0]);
  const auto db = Read<float>((*layer)->gradients()[1]);

  const int dtype = bf16 ? PLUTO_ORACLE_BF16 : PLUTO_ORACLE_F32;
  std::vector<float> want_y(y.size()), want_dx(dx.size()), want_dw(dw.size()), want_db(db.size());
  ASSERT_EQ(pluto_oracle_dense_forward(dtype, rows, input_dim, output_dim, x.data(), matrix.data(),
                                       bias.data(), want_y.data()), 0);
  ASSERT_EQ(pluto_oracle_dense_backward(dtype, rows, input_dim, output_dim, x.data(), matrix.data(),
                                        dy.data(), want_dx.data(), want_dw.data(), want_db.data()), 0);
  auto worst = [](const std::vector<float>& got, const std::vector<float>& want) {
    double error = 0, scale = 1e-30;
    for (size_t i = 0; i < got.size(); ++i) {
      error = std::max(error, std::fabs(double(got[i]) - want[i]));
      scale = std::max(scale, std::fabs(double(want[i])));
    }
    return error / scale;
  };
  // FP32 sums of identical 16-bit products in a different order; BF16 output
  // may differ by one rounding step.
  EXPECT_LE(worst(y, want_y), bf16 ? 1e-2 : 1e-5);
  EXPECT_LE(worst(dx, want_dx), 1e-5);
  EXPECT_LE(worst(dw, want_dw), 1e-5);
  EXPECT_LE(worst(db, want_db), 1e-5);
}

TEST(FullyConnectedLayerTest, OddWidthsMatchTheOracle) {
  CompareWithOracle(DataType::FP16, 37, 21, 45);
  CompareWithOracle(DataType::BF16, 37, 21, 45);
}

TEST(FullyConnectedLayerTest, MatrixCorePathMatchesTheOracle) {
  CompareWithOracle(DataType::FP16, 300, 128, 192);
  CompareWithOracle(DataType::BF16, 300, 128, 192);
}

TEST(FullyConnectedLayerTest, BackwardOverwritesGradientsAndIsBitwiseRepeatable) {
  auto executor = NewExecutor();
  auto layer = FullyConnectedLayer::Create(*executor, 128, 64, DataType::BF16);
  ASSERT_TRUE(layer.ok());
  ASSERT_TRUE((*layer)->InitializeNormal(0.1f, 3).ok());
  const int rows = 700;
  auto input = Upload<BFloat16>(*executor, Values(static_cast<size_t>(rows) * 128, 0.2));
  auto gradient = Upload<float>(*executor, Values(static_cast<size_t>(rows) * 64, 0.9));
  ASSERT_TRUE(input.ok());
  ASSERT_TRUE(gradient.ok());
  std::vector<float> first_dw, first_db, first_dx;
  for (int pass = 0; pass < 2; ++pass) {
    auto forward = (*layer)->fwd(*executor, {*input});
    ASSERT_TRUE(forward.ok());
    auto backward = (*layer)->bwd(*executor, {*gradient}, std::move(forward->state));
    ASSERT_TRUE(backward.ok());
    const auto dx = Read<float>((*backward)[0]);
    const auto dw = Read<float>((*layer)->gradients()[0]);
    const auto db = Read<float>((*layer)->gradients()[1]);
    if (pass == 0) {
      first_dx = dx, first_dw = dw, first_db = db;
    } else {
      EXPECT_TRUE(dx == first_dx);
      EXPECT_TRUE(dw == first_dw);  // overwritten, not accumulated
      EXPECT_TRUE(db == first_db);
    }
  }
}

TEST(FullyConnectedLayerTest, RejectsMismatchedBuffers) {
  auto executor = NewExecutor();
  auto other = NewExecutor();
  auto layer = FullyConnectedLayer::Create(*executor, 16, 8, DataType::FP16);
  ASSERT_TRUE(layer.ok());
  auto input = Upload<float>(*executor, Values(5 * 16, 0.1));
  ASSERT_TRUE(input.ok());
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*input, *input}).status()));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*other, {*input}).status()));
  auto ragged = Upload<float>(*executor, Values(5 * 16 + 3, 0.1));
  ASSERT_TRUE(ragged.ok());
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*ragged}).status()));
  auto forward = (*layer)->fwd(*executor, {*input});
  ASSERT_TRUE(forward.ok());
  auto wrong = Upload<float>(*executor, Values(4 * 8, 0.1));  // 4 rows against 5 saved
  ASSERT_TRUE(wrong.ok());
  EXPECT_TRUE(IsInvalidArgument(
      (*layer)->bwd(*executor, {*wrong}, std::move(forward->state)).status()));
}

}  // namespace
}  // namespace pluto::llm
