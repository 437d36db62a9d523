// The attention block of a GPT-2 layer through the host API: QKV projection,
// causal attention, output projection (src/llm/gpt2.cc:55-68 builds the same chain from
// FullyConnectedLayer and AttentionLayer).  Forward and backward are compared
// with the same chain of CPU oracles.
#include "pluto_amd/host/attention.h"
#include "pluto_amd/host/fully_connected.h"
#include "tests/cpp/test_support.h"

namespace pluto::llm {
namespace {

using testing::BFloat16;
using testing::NewExecutor;
using testing::Read;
using testing::Upload;
using testing::Values;

double Worst(const std::vector<float>& got, const std::vector<float>& want) {
  double error = 0, scale = 1e-30;
  for (size_t i = 0; i < got.size(); ++i) {
    error = std::max(error, std::fabs(double(got[i]) - want[i]));
    scale = std::max(scale, std::fabs(double(want[i])));
  }
  return error / scale;
}

void RunBlock(DataType policy, int rows, int context, int heads, int width) {
  auto executor = NewExecutor();
  const bool bf16 = policy == DataType::BF16;
  auto qkv_layer = FullyConnectedLayer::Create(*executor, width, 3 * width, policy, context);
  auto attention = AttentionLayer::Create(*executor, context, heads, width, policy);
  auto out_layer = FullyConnectedLayer::Create(*executor, width, width, policy, context);
  ASSERT_TRUE(qkv_layer.ok());
  ASSERT_TRUE(attention.ok());
  ASSERT_TRUE(out_layer.ok());
  ASSERT_TRUE((*qkv_layer)->InitializeNormal(0.2f, 11).ok());
  ASSERT_TRUE((*out_layer)->InitializeNormal(0.2f, 12).ok());
  // the layers chain: output signature of one is the input signature of the next
  EXPECT_EQ((*qkv_layer)->output_types()[0], (*attention)->input_types()[0]);
  EXPECT_EQ((*attention)->output_types()[0], (*out_layer)->input_types()[0]);

  auto x = Values(static_cast<size_t>(rows) * width, 0.7, 0.9);
  if (bf16) x = testing::RoundedToBFloat16(x);
  const auto dy = Values(static_cast<size_t>(rows) * width, 2.3, 0.4);
  auto input = bf16 ? Upload<BFloat16>(*executor, x) : Upload<float>(*executor, x);
  auto gradient = Upload<float>(*executor, dy);
  ASSERT_TRUE(input.ok());
  ASSERT_TRUE(gradient.ok());

  auto f1 = (*qkv_layer)->fwd(*executor, {*input});
  ASSERT_TRUE(f1.ok());
  auto f2 = (*attention)->fwd(*executor, {f1->outputs[0]});
  ASSERT_TRUE(f2.ok());
  auto f3 = (*out_layer)->fwd(*executor, {f2->outputs[0]});
  ASSERT_TRUE(f3.ok());
  const auto y = bf16 ? Read<BFloat16>(f3->outputs[0]) : Read<float>(f3->outputs[0]);
  auto b3 = (*out_layer)->bwd(*executor, {*gradient}, std::move(f3->state));
  ASSERT_TRUE(b3.ok());
  auto b2 = (*attention)->bwd(*executor, {(*b3)[0]}, std::move(f2->state));
  ASSERT_TRUE(b2.ok());
  auto b1 = (*qkv_layer)->bwd(*executor, {(*b2)[0]}, std::move(f1->state));
  ASSERT_TRUE(b1.ok());
  const auto dx = Read<float>((*b1)[0]);
  const auto dw_qkv = Read<float>((*qkv_layer)->gradients()[0]);
  const auto db_qkv = Read<float>((*qkv_layer)->gradients()[1]);
  const auto dw_out = Read<float>((*out_layer)->gradients()[0]);

  // the same chain on the CPU; bf16 activations are rounded between layers
  const int dtype = bf16 ? PLUTO_ORACLE_BF16 : PLUTO_ORACLE_F32;
  const auto w_qkv = Read<float>((*qkv_layer)->weights()[0]);
  const auto w_out = Read<float>((*out_layer)->weights()[0]);
  const std::vector<float> zero_qkv(3 * width, 0.0f), zero_out(width, 0.0f);
  std::vector<float> qkv(static_cast<size_t>(rows) * 3 * width), core(x.size()), want_y(x.size());
  ASSERT_EQ(pluto_oracle_dense_forward(dtype, rows, width, 3 * width, x.data(), w_qkv.data(),
                                       zero_qkv.data(), qkv.data()), 0);
  std::vector<BFloat16> qkv_bits(qkv.size()), core_bits(core.size());
  for (size_t i = 0; i < qkv.size(); ++i) qkv_bits[i] = pluto_oracle_f32_to_bf16(qkv[i]);
  const void* attention_in = bf16 ? static_cast<const void*>(qkv_bits.data()) : qkv.data();
  void* attention_out = bf16 ? static_cast<void*>(core_bits.data()) : core.data();
  std::vector<float> maxima(static_cast<size_t>(rows) * heads), normalizers(maxima.size());
  ASSERT_EQ(pluto_oracle_mha_fwd(dtype, attention_in, rows, context, heads, width, attention_out,
                                 maxima.data(), normalizers.data(), 0, rows / context, 0, heads), 0);
  if (bf16)
    for (size_t i = 0; i < core.size(); ++i) core[i] = pluto_oracle_bf16_to_f32(core_bits[i]);
  ASSERT_EQ(pluto_oracle_dense_forward(dtype, rows, width, width, core.data(), w_out.data(),
                                       zero_out.data(), want_y.data()), 0);
  std::vector<float> d_core(core.size()), want_dw_out(w_out.size()), db_out(width),
      d_qkv(qkv.size()), want_dx(x.size()), want_dw_qkv(w_qkv.size()), want_db_qkv(3 * width);
  ASSERT_EQ(pluto_oracle_dense_backward(dtype, rows, width, width, core.data(), w_out.data(),
                                        dy.data(), d_core.data(), want_dw_out.data(),
                                        db_out.data()), 0);
  ASSERT_EQ(pluto_oracle_mha_bwd(dtype, attention_in, attention_out, d_core.data(), rows, context,
                                 heads, width, d_qkv.data(), 0, rows / context, 0, heads), 0);
  ASSERT_EQ(pluto_oracle_dense_backward(dtype, rows, width, 3 * width, x.data(), w_qkv.data(),
                                        d_qkv.data(), want_dx.data(), want_dw_qkv.data(),
                                        want_db_qkv.data()), 0);
  // bf16: the layers' outputs may differ by a rounding step, which the next
  // layer multiplies; FP32 storage differs by summation order only.
  const double tolerance = bf16 ? 3e-2 : 2e-4;
  EXPECT_LE(Worst(y, want_y), tolerance);
  EXPECT_LE(Worst(dx, want_dx), tolerance);
  EXPECT_LE(Worst(dw_qkv, want_dw_qkv), tolerance);
  // The bias gradient sums 3 * width columns of d_qkv over all rows, and the
  // query and key columns cancel almost completely (each probability row's
  // gradient sums to zero): its error is bounded by the terms, not the sums.
  double bias_error = 0, bias_terms = 1e-30;
  for (int c = 0; c < 3 * width; ++c) {
    double terms = 0;
    for (int r = 0; r < rows; ++r) terms += std::fabs(d_qkv[static_cast<size_t>(r) * 3 * width + c]);
    bias_terms = std::max(bias_terms, terms);
    bias_error = std::max(bias_error, std::fabs(double(db_qkv[c]) - want_db_qkv[c]));
  }
  EXPECT_LE(bias_error, tolerance * bias_terms);
  EXPECT_LE(Worst(dw_out, want_dw_out), tolerance);
}

TEST(AttentionBlockTest, Float32ChainMatchesTheOracleChain) {
  RunBlock(DataType::FP16, 48, 12, 3, 24);   // odd head width 8: generic kernels
}

TEST(AttentionBlockTest, BFloat16ChainOnTheMatrixCoresMatchesTheOracleChain) {
  RunBlock(DataType::BF16, 512, 256, 2, 128);  // head width 64, widths multiples of 64
}

}  // namespace
}  // namespace pluto::llm
