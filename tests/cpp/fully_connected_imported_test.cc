// Imported FullyConnectedLayer projections through the host API; the cases
// follow src/llm/layers/fully_connected_imported_test.cc:93-336 with the CPU
// oracle in the place of that file's scalar projection.
#include "pluto_amd/host/fully_connected.h"
#include "tests/cpp/test_support.h"

namespace pluto::llm {
namespace {

using testing::BFloat16;
using testing::NewExecutor;
using testing::Read;
using testing::Upload;

using testing::UploadRaw;

std::vector<uint8_t> Fp8(const std::vector<float>& values) { return testing::Fp8Codes(values); }

TEST(ImportedLinearTest, SharesAllStorageWithoutMastersOrGradients) {
  auto executor = NewExecutor();
  const std::vector<float> matrix = {1, 2, 3, 4, 5, 6};
  auto input = Upload<BFloat16>(*executor, {1, 0, -1});
  auto fp32 = Upload<float>(*executor, matrix);
  auto bf16 = Upload<BFloat16>(*executor, matrix);
  auto fp8 = UploadRaw<uint8_t>(*executor, Fp8(matrix));
  auto scales = Upload<float>(*executor, {1});
  ASSERT_TRUE(input.ok());
  ASSERT_TRUE(fp32.ok());
  ASSERT_TRUE(bf16.ok());
  ASSERT_TRUE(fp8.ok());
  ASSERT_TRUE(scales.ok());
  for (MatrixStorage storage :
       {MatrixStorage::kFloat32, MatrixStorage::kBFloat16, MatrixStorage::kFp8E4M3}) {
    const Buffer& weights = storage == MatrixStorage::kFloat32    ? *fp32
                            : storage == MatrixStorage::kBFloat16 ? *bf16
                                                                  : *fp8;
    auto layer = FullyConnectedLayer::Create(
        *executor, weights, storage, 3, 2,
        storage == MatrixStorage::kFp8E4M3 ? std::optional<Buffer>(*scales) : std::nullopt);
    ASSERT_TRUE(layer.ok());
    EXPECT_TRUE((*layer)->weights()[0].data() == weights.data());
    EXPECT_EQ((*layer)->weights().size(), storage == MatrixStorage::kFp8E4M3 ? 2u : 1u);
    if (storage == MatrixStorage::kFp8E4M3)
      EXPECT_TRUE((*layer)->weights()[1].data() == scales->data());
    EXPECT_TRUE((*layer)->gradients().empty());
    EXPECT_EQ((*layer)->input_types()[0], ActivationType(DataType::BF16, {1, 1, 3}));
    EXPECT_EQ((*layer)->output_types()[0], ActivationType(DataType::BF16, {1, 1, 2}));
    EXPECT_TRUE((*layer)->output_type() == DataType::BF16);
    EXPECT_EQ((*layer)->input_dim(), 3);
    EXPECT_EQ((*layer)->output_dim(), 2);
    EXPECT_TRUE(IsFailedPrecondition((*layer)->InitializeIdentity()));
    EXPECT_TRUE(IsFailedPrecondition((*layer)->InitializeNormal(1, 123)));
    auto result = (*layer)->fwd(*executor, {*input});
    ASSERT_TRUE(result.ok());
    EXPECT_TRUE(Read<BFloat16>(result->outputs[0]) == (std::vector<float>{-2, -2}));
    EXPECT_TRUE(result->state.intermediates.empty());
    EXPECT_TRUE(IsUnimplemented(
        (*layer)->bwd(*executor, {result->outputs[0]}, std::move(result->state)).status()));
  }
}

TEST(ImportedLinearTest, BlockScalesTailsAndRealWidthMatchScalarProjection) {
  auto executor = NewExecutor();
  // Straddles the row tiles and the 128 x 128 scale blocks, and includes the
  // checkpoint's 5120-wide input; every storage sees the same bf16 token.
  for (const auto& [cols, rows] : {std::pair{263, 259}, std::pair{5120, 131}}) {
    std::vector<float> source(static_cast<size_t>(cols) * rows), input(cols);
    for (size_t i = 0; i < source.size(); ++i)
      source[i] = 1.9f * std::sin(static_cast<float>(i % 1009) * 0.037f);
    for (int c = 0; c < cols; ++c)
      input[c] = pluto_oracle_bf16_round(std::cos(c * 0.123f) * 0.25f);
    const int scale_cols = (cols + 127) / 128, scale_rows = (rows + 127) / 128;
    std::vector<float> scales(static_cast<size_t>(scale_cols) * scale_rows);
    for (int r = 0; r < scale_rows; ++r)
      for (int c = 0; c < scale_cols; ++c) scales[r * scale_cols + c] = (r + 1) * (c + 1) * 0.03125f;
    std::vector<BFloat16> bits(source.size());
    for (size_t i = 0; i < source.size(); ++i) bits[i] = pluto_oracle_f32_to_bf16(source[i]);
    const std::vector<uint8_t> codes = Fp8(source);
    auto df32 = Upload<float>(*executor, source);
    auto dbf16 = UploadRaw<BFloat16>(*executor, bits);
    auto dfp8 = UploadRaw<uint8_t>(*executor, codes);
    auto dx = Upload<BFloat16>(*executor, input);
    auto ds = Upload<float>(*executor, scales);
    ASSERT_TRUE(df32.ok());
    ASSERT_TRUE(dbf16.ok());
    ASSERT_TRUE(dfp8.ok());
    ASSERT_TRUE(dx.ok());
    ASSERT_TRUE(ds.ok());
    for (MatrixStorage storage :
         {MatrixStorage::kFloat32, MatrixStorage::kBFloat16, MatrixStorage::kFp8E4M3}) {
      const bool fp8 = storage == MatrixStorage::kFp8E4M3;
      const Buffer& weights = storage == MatrixStorage::kFloat32 ? *df32 : fp8 ? *dfp8 : *dbf16;
      auto layer = FullyConnectedLayer::Create(*executor, weights, storage, cols, rows,
                                               fp8 ? std::optional<Buffer>(*ds) : std::nullopt);
      ASSERT_TRUE(layer.ok());
      auto result = (*layer)->fwd(*executor, {*dx});
      ASSERT_TRUE(result.ok());
      const auto actual = Read<BFloat16>(result->outputs[0]);
      ASSERT_EQ(actual.size(), static_cast<size_t>(rows));
      std::vector<float> expected(rows);
      const void* host_weights = storage == MatrixStorage::kFloat32
                                     ? static_cast<const void*>(source.data())
                                     : fp8 ? static_cast<const void*>(codes.data())
                                           : static_cast<const void*>(bits.data());
      const int code = storage == MatrixStorage::kFloat32 ? PLUTO_ORACLE_MATRIX_F32
                       : fp8                              ? PLUTO_ORACLE_MATRIX_FP8_E4M3
                                                          : PLUTO_ORACLE_MATRIX_BF16;
      ASSERT_EQ(pluto_oracle_imported_matvec(code, host_weights, fp8 ? scales.data() : nullptr,
                                             input.data(), cols, rows, expected.data()), 0);
      for (int r = 0; r < rows; ++r)
        EXPECT_NEAR(actual[r], expected[r], 5e-5f + 0.008f * std::fabs(expected[r]));
    }
  }
}

TEST(ImportedLinearTest, DynamicFp8QuantizationHandlesZeroTinyTiesAndTail) {
  auto executor = NewExecutor();
  constexpr int kWidth = 389;
  std::vector<float> input(kWidth, 0.0f);
  // Zero group, exact-unit scale with midpoint ties, tiny group testing the
  // divisor floor, and a final partial group.
  for (int i = 128; i < 256; ++i) input[i] = ((i % 31) - 15) * 0.0625f;
  input[128] = 448;
  input[129] = -448;
  input[130] = 1.0625f;
  input[131] = 1.1875f;
  for (int i = 256; i < 384; ++i) input[i] = pluto_oracle_bf16_round((i % 5 - 2) * 1e-14f);
  for (int i = 384; i < kWidth; ++i) input[i] = pluto_oracle_bf16_round((i - 386) * 25.3f);
  // An identity matrix exposes every quantized input through the layer API.
  std::vector<uint8_t> identity(static_cast<size_t>(kWidth) * kWidth,
                                pluto_oracle_f32_to_fp8_e4m3(0.0f));
  for (int i = 0; i < kWidth; ++i)
    identity[static_cast<size_t>(i) * kWidth + i] = pluto_oracle_f32_to_fp8_e4m3(1.0f);
  auto weights = UploadRaw<uint8_t>(*executor, identity);
  auto scales = Upload<float>(*executor, std::vector<float>(16, 1.0f));
  auto dx = Upload<BFloat16>(*executor, input);
  ASSERT_TRUE(weights.ok());
  ASSERT_TRUE(scales.ok());
  ASSERT_TRUE(dx.ok());
  auto layer = FullyConnectedLayer::Create(*executor, *weights, MatrixStorage::kFp8E4M3, kWidth,
                                           kWidth, *scales);
  ASSERT_TRUE(layer.ok());
  auto output = (*layer)->fwd(*executor, {*dx});
  ASSERT_TRUE(output.ok());
  const auto actual = Read<BFloat16>(output->outputs[0]);
  std::vector<float> expected(kWidth);
  pluto_oracle_imported_quantize(input.data(), kWidth, expected.data());
  ASSERT_EQ(actual.size(), expected.size());
  for (size_t i = 0; i < input.size(); ++i)
    EXPECT_NEAR(actual[i], pluto_oracle_bf16_round(expected[i]),
                1e-20f + 0.008f * std::fabs(expected[i]));
  EXPECT_EQ(actual[130], 1.0f);
  EXPECT_EQ(actual[131], 1.25f);
}

TEST(ImportedLinearTest, RejectsBadStorageDimensionsScalesAndExecutors) {
  auto executor = NewExecutor();
  auto other = NewExecutor();
  auto weights = Upload<float>(*executor, {1, 2, 3, 4, 5, 6});
  auto scales = Upload<float>(*executor, {1});
  auto fp8 = UploadRaw<uint8_t>(*executor, std::vector<uint8_t>(6, 0));
  auto input = Upload<BFloat16>(*executor, {1, 0, -1});
  ASSERT_TRUE(weights.ok());
  ASSERT_TRUE(scales.ok());
  ASSERT_TRUE(fp8.ok());
  ASSERT_TRUE(input.ok());
  for (int bad : {0, -1, FullyConnectedLayer::kMaximumDimension + 1}) {
    EXPECT_FALSE(
        FullyConnectedLayer::Create(*executor, *weights, MatrixStorage::kFloat32, bad, 2).ok());
    EXPECT_FALSE(
        FullyConnectedLayer::Create(*executor, *weights, MatrixStorage::kFloat32, 3, bad).ok());
  }
  // wrong element size, scales with a scale-free storage, FP8 without scales,
  // a scale buffer of the wrong size, a foreign executor
  EXPECT_FALSE(FullyConnectedLayer::Create(*executor, *weights, MatrixStorage::kBFloat16, 3, 2).ok());
  EXPECT_FALSE(
      FullyConnectedLayer::Create(*executor, *weights, MatrixStorage::kFloat32, 3, 2, *scales).ok());
  EXPECT_FALSE(FullyConnectedLayer::Create(*executor, *fp8, MatrixStorage::kFp8E4M3, 3, 2).ok());
  EXPECT_FALSE(
      FullyConnectedLayer::Create(*executor, *fp8, MatrixStorage::kFp8E4M3, 3, 2, *weights).ok());
  EXPECT_FALSE(FullyConnectedLayer::Create(*other, *weights, MatrixStorage::kFloat32, 3, 2).ok());
  auto layer = FullyConnectedLayer::Create(*executor, *weights, MatrixStorage::kFloat32, 3, 2);
  ASSERT_TRUE(layer.ok());
  EXPECT_FALSE((*layer)->fwd(*executor, {}).ok());
  EXPECT_FALSE((*layer)->fwd(*executor, {*input, *input}).ok());
  EXPECT_FALSE((*layer)->fwd(*executor, {*weights}).ok());   // not a bf16 token of 3 elements
  EXPECT_FALSE((*layer)->fwd(*other, {*input}).ok());
}

}  // namespace
}  // namespace pluto::llm
