// BatchedDecoderStep: the step contract of Model::Step
// (src/llm/qwen/model.cc:405-428) for several sequences, and the composed
// decoder against the CPU oracle.  The oracle leg follows the shape of the
// reference's scalar decoder (qwen/model_test.cc:343-459, ReferenceStep): per
// sequence and layer, scalar projections, then the scalar delta-net step or
// the scalar cached attention step, then the output projection - here the
// oracle's restatements of those scalar specifications, chained on the host.
#include <cstdio>

#include "pluto_amd/host/decoder_step.h"
#include "tests/cpp/test_support.h"

namespace pluto::llm {
namespace {

using testing::BFloat16;
using testing::NewExecutor;
using testing::Read;
using testing::Upload;
using testing::UploadRaw;
using testing::Values;
using cached_attention_ops::DeltaNetParameters;
using cached_attention_ops::FullAttentionParameters;

// A checkpoint matrix [out, in]: on the device for the layers, and as the
// oracle reads it (bf16 bit patterns, or FP8 codes with block scales).
struct Matrix {
  std::optional<Buffer> weights;
  std::optional<Buffer> scale_buffer;
  MatrixStorage storage;
  int in, out;
  std::vector<BFloat16> bf16_bits;
  std::vector<uint8_t> fp8_codes;
  std::vector<float> scales;

  StatusOr<std::unique_ptr<FullyConnectedLayer>> Layer(hip::Executor& executor) const {
    return FullyConnectedLayer::Create(executor, *weights, storage, in, out, scale_buffer);
  }
  // One token through the oracle's projection: floats holding bf16 values.
  std::vector<float> Project(const std::vector<float>& token) const {
    std::vector<float> result(out);
    const bool fp8 = storage == MatrixStorage::kFp8E4M3;
    const int code = pluto_oracle_imported_matvec(
        fp8 ? PLUTO_ORACLE_MATRIX_FP8_E4M3 : PLUTO_ORACLE_MATRIX_BF16,
        fp8 ? static_cast<const void*>(fp8_codes.data()) : static_cast<const void*>(bf16_bits.data()),
        fp8 ? scales.data() : nullptr, token.data(), in, out, result.data());
    if (code != 0) std::abort();
    return result;
  }
};

StatusOr<Matrix> MakeMatrix(hip::Executor& executor, MatrixStorage storage, int in, int out,
                            double phase, double magnitude = 1.7) {
  Matrix m;
  m.storage = storage;
  m.in = in;
  m.out = out;
  const auto source =
      Values(static_cast<size_t>(in) * out, phase, magnitude / std::sqrt(double(in)));
  if (storage == MatrixStorage::kBFloat16) {
    for (float value : source) m.bf16_bits.push_back(pluto_oracle_f32_to_bf16(value));
    ASSIGN_OR_RETURN(auto weights, UploadRaw<BFloat16>(executor, m.bf16_bits));
    m.weights = std::move(weights);
    return m;
  }
  const int block_cols = (in + 127) / 128, block_rows = (out + 127) / 128;
  m.scales.resize(static_cast<size_t>(block_cols) * block_rows);
  for (int r = 0; r < block_rows; ++r)
    for (int c = 0; c < block_cols; ++c)
      m.scales[r * block_cols + c] = (1.0f + 0.25f * ((r + 2 * c) % 3)) / 64.0f;
  std::vector<float> scaled(source.size());
  for (int o = 0; o < out; ++o)
    for (int i = 0; i < in; ++i)
      scaled[static_cast<size_t>(o) * in + i] =
          source[static_cast<size_t>(o) * in + i] / m.scales[(o / 128) * block_cols + i / 128];
  m.fp8_codes = testing::Fp8Codes(scaled);
  ASSIGN_OR_RETURN(auto weights, UploadRaw<uint8_t>(executor, m.fp8_codes));
  m.weights = std::move(weights);
  ASSIGN_OR_RETURN(auto scale_buffer, Upload<float>(executor, m.scales));
  m.scale_buffer = std::move(scale_buffer);
  return m;
}

std::vector<float> Hidden(int batch, int width, int step) {
  auto rows = Values(static_cast<size_t>(batch) * width, 0.37 + 1.3 * step, 0.9);
  for (int s = 0; s < batch; ++s)
    for (int c = 0; c < width; ++c)
      rows[static_cast<size_t>(s) * width + c] += 0.3f * std::cos(0.11f * c + s);
  return testing::RoundedToBFloat16(rows);
}

// A caller-supplied layer between the branches: passes its rows through and
// can be told to fail, as a hook or a later layer of the reference can.
class PassThrough final : public Layer {
 public:
  PassThrough(int width, const bool* fail)
      : types_{ActivationType(DataType::BF16, {ActivationType::kBatchDimension, 1, int64_t{width}})},
        fail_(fail) {}
  std::string_view name() const override { return "PassThrough"; }
  DataType output_type() const override { return DataType::BF16; }
  Span<Buffer> weights() override { return {}; }
  Span<const ActivationType> input_types() const override { return MakeConstSpan(types_); }
  Span<const ActivationType> output_types() const override { return MakeConstSpan(types_); }

 private:
  StatusOr<FwdResult> fwd_impl(hip::Executor&, Span<const Buffer> inputs,
                               LayerHooks*) const override {
    if (*fail_) return InternalError("a later layer failed");
    FwdResult forward;
    forward.outputs.push_back(inputs[0]);
    return forward;
  }
  StatusOr<BufferVec> bwd_impl(hip::Executor&, Span<const Buffer>, BackwardState,
                               LayerHooks*) override {
    return UnimplementedError("inference only");
  }
  std::vector<ActivationType> types_;
  const bool* fail_;
};

// Layer 0 a delta-net branch, layer 1 a full-attention branch (the order of
// the reference's tiny hybrid configuration, model_test.cc:352-447), a
// pass-through between and after them.
struct Decoder {
  int batch, width;
  FullAttentionParameters attention;
  DeltaNetParameters delta;
  Matrix wqkv, wz, wa, wb, wdo;      // delta-net projections
  Matrix wq, wk, wv, wo;             // attention projections
  std::vector<float> conv, a_log, dt_bias, norm, q_norm, k_norm;
  std::unique_ptr<BatchedDecoderStep> step;
  BatchedFullAttentionBranch* attention_branch = nullptr;
  BatchedDeltaNetBranch* delta_branch = nullptr;
  bool fail = false;
};

void Build(hip::Executor& executor, int batch, int width, int capacity, MatrixStorage storage,
           double magnitude, Decoder* d) {
  d->batch = batch;
  d->width = width;
  FullAttentionParameters& p = d->attention;
  p.query_heads = 4;
  p.key_value_heads = 2;
  p.head_dim = 16;
  p.rotary_dim = 8;
  p.capacity = capacity;
  DeltaNetParameters& g = d->delta;
  g.key_heads = 2;
  g.value_heads = 4;
  g.key_head_dim = 8;
  g.value_head_dim = 12;
  g.conv_kernel_dim = 3;
  const int q = p.query_heads * p.head_dim, kv = p.key_value_heads * p.head_dim;
  const int keys = g.key_heads * g.key_head_dim, values = g.value_heads * g.value_head_dim;
  const int channels = 2 * keys + values;
  auto take = [&](Matrix* into, int in, int out, double phase) {
    auto made = MakeMatrix(executor, storage, in, out, phase, magnitude);
    ASSERT_TRUE(made.ok());
    *into = std::move(*made);
  };
  take(&d->wqkv, width, channels, 0.1);
  take(&d->wz, width, values, 0.7);
  take(&d->wa, width, g.value_heads, 1.9);
  take(&d->wb, width, g.value_heads, 2.3);
  take(&d->wdo, values, width, 2.6);
  take(&d->wq, width, 2 * q, 3.1);
  take(&d->wk, width, kv, 3.7);
  take(&d->wv, width, kv, 4.3);
  take(&d->wo, q, width, 4.9);
  d->conv = Values(static_cast<size_t>(channels) * g.conv_kernel_dim, 0.73, 0.6);
  d->a_log = Values(g.value_heads, 0.18, 0.5);
  d->dt_bias = Values(g.value_heads, -0.7, 0.3);
  d->norm = Values(g.value_head_dim, 0.5, 0.6);
  d->q_norm = Values(p.head_dim, 0.2, 0.5);
  d->k_norm = Values(p.head_dim, 0.4, 0.5);
  auto conv = Upload<float>(executor, d->conv), a_log = Upload<float>(executor, d->a_log),
       dt_bias = Upload<float>(executor, d->dt_bias), norm = Upload<float>(executor, d->norm),
       q_norm = Upload<float>(executor, d->q_norm), k_norm = Upload<float>(executor, d->k_norm);
  ASSERT_TRUE(conv.ok() && a_log.ok() && dt_bias.ok() && norm.ok() && q_norm.ok() && k_norm.ok());
  auto lqkv = d->wqkv.Layer(executor), lz = d->wz.Layer(executor), la = d->wa.Layer(executor),
       lb = d->wb.Layer(executor), ldo = d->wdo.Layer(executor);
  auto lq = d->wq.Layer(executor), lk = d->wk.Layer(executor), lv = d->wv.Layer(executor),
       lo = d->wo.Layer(executor);
  ASSERT_TRUE(lqkv.ok() && lz.ok() && la.ok() && lb.ok() && ldo.ok());
  ASSERT_TRUE(lq.ok() && lk.ok() && lv.ok() && lo.ok());
  auto delta = BatchedDeltaNetBranch::Create(executor, g, batch, std::move(*lqkv), std::move(*lz),
                                             std::move(*la), std::move(*lb), std::move(*ldo), *conv,
                                             *a_log, *dt_bias, *norm);
  auto attention = BatchedFullAttentionBranch::Create(
      executor, p, batch, std::move(*lq), std::move(*lk), std::move(*lv), std::move(*lo), *q_norm,
      *k_norm, KeyValueCache::Storage::kBFloat16HeadMajor);
  ASSERT_TRUE(delta.ok() && attention.ok());
  d->delta_branch = delta->get();
  d->attention_branch = attention->get();
  std::vector<std::unique_ptr<Layer>> layers;
  layers.push_back(std::move(*delta));
  layers.push_back(std::make_unique<PassThrough>(width, &d->fail));
  layers.push_back(std::move(*attention));
  auto step = BatchedDecoderStep::Create(executor, batch, width, capacity, std::move(layers),
                                         {d->attention_branch}, {d->delta_branch});
  ASSERT_TRUE(step.ok());
  d->step = std::move(*step);
}

// The oracle's history of one sequence.
struct OracleSequence {
  std::vector<float> conv_state;
  std::vector<double> recurrent_state;
  std::vector<float> cache_keys, cache_values;
  int position = 0;
};

std::vector<float> OracleStep(const Decoder& d, const std::vector<float>& token,
                              OracleSequence* history) {
  const FullAttentionParameters& p = d.attention;
  const DeltaNetParameters& g = d.delta;
  const int keys = g.key_heads * g.key_head_dim, values = g.value_heads * g.value_head_dim;
  const int channels = 2 * keys + values;
  if (history->conv_state.empty()) {
    history->conv_state.assign(static_cast<size_t>(channels) * g.conv_kernel_dim, 0.0f);
    history->recurrent_state.assign(
        static_cast<size_t>(g.value_heads) * g.key_head_dim * g.value_head_dim, 0.0);
    const size_t cache = static_cast<size_t>(p.capacity) * p.key_value_heads * p.head_dim;
    history->cache_keys.assign(cache, 0.0f);
    history->cache_values.assign(cache, 0.0f);
  }
  // layer 0: delta-net branch
  const pluto_oracle_delta_params delta = {g.key_heads,       g.value_heads,     g.key_head_dim,
                                           g.value_head_dim,  g.conv_kernel_dim, g.rms_norm_epsilon,
                                           g.round_to_bfloat16 ? 1 : 0};
  const auto qkv = d.wqkv.Project(token), z = d.wz.Project(token), a = d.wa.Project(token),
             b = d.wb.Project(token);
  std::vector<float> mixed(values);
  if (pluto_oracle_gdn_step(&delta, history->conv_state.data(), history->recurrent_state.data(),
                            qkv.data(), z.data(), a.data(), b.data(), d.conv.data(),
                            d.a_log.data(), d.dt_bias.data(), d.norm.data(), mixed.data()) != 0)
    std::abort();
  const auto between = d.wdo.Project(mixed);
  // layer 1: full-attention branch
  const pluto_oracle_attention_params attention = {
      p.query_heads,      p.key_value_heads, p.head_dim, p.rotary_dim, p.capacity,
      p.rms_norm_epsilon, p.rope_theta,      p.round_to_bfloat16 ? 1 : 0};
  const auto q_gate = d.wq.Project(between), k = d.wk.Project(between), v = d.wv.Project(between);
  std::vector<float> attended(static_cast<size_t>(p.query_heads) * p.head_dim);
  if (pluto_oracle_gqa_cached_step(&attention, history->cache_keys.data(),
                                   history->cache_values.data(), history->position, q_gate.data(),
                                   k.data(), v.data(), d.q_norm.data(), d.k_norm.data(),
                                   attended.data(), nullptr) != 0)
    std::abort();
  ++history->position;
  return d.wo.Project(attended);
}

void RunAgainstTheOracle(MatrixStorage storage, double magnitude, const char* what) {
  auto executor = NewExecutor();
  Decoder d;
  const int batch = 3, width = 96, capacity = 12, steps = 9;
  Build(*executor, batch, width, capacity, storage, magnitude, &d);
  ASSERT_TRUE(d.step != nullptr);
  std::vector<OracleSequence> histories(batch);
  double worst = 0;
  int compared = 0, beyond = 0;
  for (int step = 0; step < steps; ++step) {
    if (step == 4) {  // sequence 1 ended: it alone starts over
      ASSERT_TRUE(d.step->Reset(1).ok());
      histories[1] = OracleSequence();
    }
    const auto hidden = Hidden(batch, width, step);
    auto rows = Upload<BFloat16>(*executor, hidden);
    ASSERT_TRUE(rows.ok());
    ASSERT_TRUE(d.step->Step(*rows).ok());
    auto result = d.step->Hidden();
    ASSERT_TRUE(result.ok());
    const auto got = Read<BFloat16>(*result);
    for (int s = 0; s < batch; ++s) {
      const std::vector<float> token(hidden.begin() + static_cast<size_t>(s) * width,
                                     hidden.begin() + static_cast<size_t>(s + 1) * width);
      const auto want = OracleStep(d, token, &histories[s]);
      EXPECT_EQ(d.step->position(s), histories[s].position);
      double square = 0;
      for (float value : want) square += double(value) * value;
      const double rms = std::sqrt(square / want.size());
      EXPECT_GT(rms, 1e-3);  // not a comparison of zeros
      for (int c = 0; c < width; ++c) {
        const double error = std::fabs(double(got[static_cast<size_t>(s) * width + c]) - want[c]);
        // the bf16 bound of the configurations: 2e-2 of |x| + rms
        const double ratio = error / (std::fabs(want[c]) + rms);
        worst = std::max(worst, ratio);
        beyond += ratio > 2e-2;
        ++compared;
      }
    }
  }
  std::printf("decoder step (%s), 2 layers, 3 sequences, 9 steps against the oracle chain: worst "
              "%.2e of |x| + rms over %d outputs\n", what, worst, compared);
  EXPECT_EQ(beyond, 0);
  EXPECT_EQ(d.step->position(0), steps);
  EXPECT_EQ(d.step->position(1), steps - 4);
}

TEST(DecoderStepTest, TwoLayerDecoderFollowsTheOracleChain) {
  RunAgainstTheOracle(MatrixStorage::kBFloat16, 6.0, "bf16 projections");
  RunAgainstTheOracle(MatrixStorage::kFp8E4M3, 6.0, "FP8 projections");
}

TEST(DecoderStepTest, IdentityFixtureLeavesZeroRows) {
  // The reference's known-logits fixture zeroes every projection of both
  // branches (model_test.cc Fp8(): rows * columns zeros), so a block's
  // attention branch adds exactly nothing to the residual, which is what makes
  // ExpectOneHotLogits (model_test.cc:461-466) hold.  Reduced to the branches:
  // zero projections give exactly zero rows, at every step.
  auto executor = NewExecutor();
  Decoder d;
  Build(*executor, 2, 96, 4, MatrixStorage::kFp8E4M3, 0.0, &d);
  ASSERT_TRUE(d.step != nullptr);
  for (int step = 0; step < 3; ++step) {
    auto rows = Upload<BFloat16>(*executor, Hidden(2, 96, step));
    ASSERT_TRUE(rows.ok());
    ASSERT_TRUE(d.step->Step(*rows).ok());
    auto result = d.step->Hidden();
    ASSERT_TRUE(result.ok());
    for (float value : Read<BFloat16>(*result)) EXPECT_EQ(value, 0.0f);
  }
}

TEST(DecoderStepTest, StepContract) {
  auto executor = NewExecutor();
  auto elsewhere = NewExecutor();
  Decoder d;
  const int batch = 2, width = 96, capacity = 3;
  Build(*executor, batch, width, capacity, MatrixStorage::kBFloat16, 1.7, &d);
  ASSERT_TRUE(d.step != nullptr);
  auto rows = Upload<BFloat16>(*executor, Hidden(batch, width, 0));
  auto one_row = Upload<BFloat16>(*executor, Hidden(1, width, 0));
  auto foreign = Upload<BFloat16>(*elsewhere, Hidden(batch, width, 0));
  ASSERT_TRUE(rows.ok() && one_row.ok() && foreign.ok());

  // no hidden rows before the first successful step (model.cc:430-435)
  EXPECT_TRUE(IsFailedPrecondition(d.step->Hidden().status()));
  // rejected inputs run nothing and poison nothing
  EXPECT_TRUE(IsInvalidArgument(d.step->Step(*one_row)));
  EXPECT_TRUE(IsInvalidArgument(d.step->Step(*foreign)));
  EXPECT_FALSE(d.step->poisoned());
  EXPECT_EQ(d.attention_branch->cache(0).position(), 0);

  ASSERT_TRUE(d.step->Step(*rows).ok());
  auto first = d.step->Hidden();
  ASSERT_TRUE(first.ok());
  const auto first_rows = Read<BFloat16>(*first);
  EXPECT_EQ(d.step->position(0), 1);
  EXPECT_EQ(d.step->position(1), 1);

  // a layer that fails after the delta-net state advanced: poisoned until Reset
  d.fail = true;
  EXPECT_FALSE(d.step->Step(*rows).ok());
  d.fail = false;
  EXPECT_TRUE(d.step->poisoned());
  EXPECT_TRUE(IsFailedPrecondition(d.step->Step(*rows)));
  EXPECT_TRUE(IsFailedPrecondition(d.step->Hidden().status()));
  EXPECT_TRUE(IsFailedPrecondition(d.step->Reset(0)));  // one sequence is not enough
  EXPECT_EQ(d.step->position(0), 1);                   // the failed step counted for nothing
  ASSERT_TRUE(d.step->Reset().ok());
  EXPECT_FALSE(d.step->poisoned());
  EXPECT_EQ(d.step->position(0), 0);
  EXPECT_EQ(d.attention_branch->cache(1).position(), 0);
  // and the first step replays bit for bit
  ASSERT_TRUE(d.step->Step(*rows).ok());
  auto replay = d.step->Hidden();
  ASSERT_TRUE(replay.ok());
  EXPECT_TRUE(Read<BFloat16>(*replay) == first_rows);

  // capacity: three tokens fit, the fourth is refused before any work
  ASSERT_TRUE(d.step->Step(*rows).ok());
  ASSERT_TRUE(d.step->Step(*rows).ok());
  EXPECT_EQ(d.step->position(1), capacity);
  EXPECT_TRUE(IsInvalidArgument(d.step->Step(*rows)));
  EXPECT_FALSE(d.step->poisoned());
  EXPECT_EQ(d.attention_branch->cache(0).position(), capacity);
  EXPECT_TRUE(d.step->Hidden().ok());  // the last successful step's rows are still there
  // a sequence that ended is reset alone; the other one is still full
  ASSERT_TRUE(d.step->Reset(1).ok());
  EXPECT_TRUE(IsInvalidArgument(d.step->Step(*rows)));
  ASSERT_TRUE(d.step->Reset(0).ok());
  ASSERT_TRUE(d.step->Step(*rows).ok());
  EXPECT_TRUE(IsInvalidArgument(d.step->Reset(2)));
}

TEST(DecoderStepTest, CreateRejectsWhatDoesNotCompose) {
  auto executor = NewExecutor();
  Decoder d;
  Build(*executor, 2, 96, 4, MatrixStorage::kBFloat16, 1.7, &d);
  ASSERT_TRUE(d.step != nullptr);
  bool never = false;
  auto layers = [&](int width) {
    std::vector<std::unique_ptr<Layer>> list;
    list.push_back(std::make_unique<PassThrough>(width, &never));
    return list;
  };
  EXPECT_TRUE(IsInvalidArgument(
      BatchedDecoderStep::Create(*executor, 0, 96, 4, layers(96), {}, {}).status()));
  EXPECT_TRUE(IsInvalidArgument(
      BatchedDecoderStep::Create(*executor, 2, 96, 4, {}, {}, {}).status()));
  // a layer of another width
  EXPECT_TRUE(IsInvalidArgument(
      BatchedDecoderStep::Create(*executor, 2, 96, 4, layers(64), {}, {}).status()));
  // a branch of another batch, a cache smaller than the capacity asked for
  EXPECT_TRUE(IsInvalidArgument(
      BatchedDecoderStep::Create(*executor, 3, 96, 4, layers(96), {d.attention_branch}, {}).status()));
  EXPECT_TRUE(IsInvalidArgument(
      BatchedDecoderStep::Create(*executor, 2, 96, 5, layers(96), {d.attention_branch}, {}).status()));
  EXPECT_TRUE(IsInvalidArgument(
      BatchedDecoderStep::Create(*executor, 3, 96, 4, layers(96), {}, {d.delta_branch}).status()));
  EXPECT_TRUE(BatchedDecoderStep::Create(*executor, 2, 96, 4, layers(96), {d.attention_branch},
                                         {d.delta_branch}).ok());
}

}  // namespace
}  // namespace pluto::llm
