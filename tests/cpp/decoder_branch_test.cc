// The batched attention branches against the chain of batch-one layers the
// reference's model loader assembles per sequence (CreateAttentionBranch,
// src/llm/qwen/model.cc:174-274): imported FullyConnectedLayer projections,
// QwenAttentionLayer over a KeyValueCache or DeltaNetLayer, output projection.
// Those layers are checked against the CPU oracle in their own tests; here the
// composition is checked against them, with sequences of different lengths.
#include <cstdio>

#include "pluto_amd/host/decoder_branch.h"
#include "pluto_amd/host/delta_net.h"
#include "pluto_amd/host/qwen_attention.h"
#include "tests/cpp/test_support.h"

namespace pluto::llm {
namespace {

using testing::BFloat16;
using testing::NewExecutor;
using testing::Read;
using testing::Upload;
using testing::UploadRaw;
using testing::Values;

// One checkpoint matrix [out, in] in device memory, shared by the batched
// branch and by the batch-one layers (imported layers do not copy).
struct Matrix {
  Buffer weights;
  std::optional<Buffer> scales;
  MatrixStorage storage;
  int in, out;
  StatusOr<std::unique_ptr<FullyConnectedLayer>> Layer(hip::Executor& executor) const {
    return FullyConnectedLayer::Create(executor, weights, storage, in, out, scales);
  }
};

StatusOr<Matrix> MakeMatrix(hip::Executor& executor, MatrixStorage storage, int in, int out,
                            double phase) {
  // entries of order 1 / sqrt(in), so that activations stay of order one
  const auto source = Values(static_cast<size_t>(in) * out, phase, 1.7 / std::sqrt(double(in)));
  if (storage == MatrixStorage::kBFloat16) {
    ASSIGN_OR_RETURN(auto weights, Upload<BFloat16>(executor, source));
    return Matrix{std::move(weights), std::nullopt, storage, in, out};
  }
  // FP8 codes of the values scaled up by 64, with block scales that undo it
  // (and differ from block to block)
  std::vector<float> scaled(source.size());
  const int block_cols = (in + 127) / 128, block_rows = (out + 127) / 128;
  std::vector<float> scales(static_cast<size_t>(block_cols) * block_rows);
  for (int r = 0; r < block_rows; ++r)
    for (int c = 0; c < block_cols; ++c)
      scales[r * block_cols + c] = (1.0f + 0.25f * ((r + 2 * c) % 3)) / 64.0f;
  for (int o = 0; o < out; ++o)
    for (int i = 0; i < in; ++i)
      scaled[static_cast<size_t>(o) * in + i] =
          source[static_cast<size_t>(o) * in + i] / scales[(o / 128) * block_cols + i / 128];
  ASSIGN_OR_RETURN(auto weights, UploadRaw<uint8_t>(executor, testing::Fp8Codes(scaled)));
  ASSIGN_OR_RETURN(auto block_scales, Upload<float>(executor, scales));
  return Matrix{std::move(weights), std::move(block_scales), storage, in, out};
}

// Rows [batch, width] of one step's input: different for every sequence and step.
std::vector<float> Hidden(int batch, int width, int step) {
  auto rows = Values(static_cast<size_t>(batch) * width, 0.37 + 1.3 * step, 0.9);
  for (int s = 0; s < batch; ++s)
    for (int c = 0; c < width; ++c)
      rows[static_cast<size_t>(s) * width + c] += 0.3f * std::cos(0.11f * c + s);
  return testing::RoundedToBFloat16(rows);
}

struct Agreement {
  int compared = 0, differing = 0;
  double worst = 0;  // |difference| / (|expected| + rms of the row)
  void Row(const std::vector<float>& got, size_t offset, const std::vector<float>& want) {
    double square = 0;
    for (float value : want) square += double(value) * value;
    const double rms = std::sqrt(square / want.size());
    for (size_t c = 0; c < want.size(); ++c) {
      const float actual = got[offset + c];
      ++compared;
      differing += actual != want[c];
      worst = std::max(worst, std::fabs(double(actual) - want[c]) / (std::fabs(want[c]) + rms));
    }
  }
};

struct AttentionCase {
  int batch, width, query_heads, kv_heads, head_dim, rotary, capacity, steps;
  MatrixStorage storage;
  KeyValueCache::Storage cache;
};

void RunAttentionCase(const AttentionCase& c) {
  auto executor = NewExecutor();
  FullAttentionParameters p;
  p.query_heads = c.query_heads;
  p.key_value_heads = c.kv_heads;
  p.head_dim = c.head_dim;
  p.rotary_dim = c.rotary;
  p.capacity = c.capacity;
  const int q = c.query_heads * c.head_dim, kv = c.kv_heads * c.head_dim;
  auto wq = MakeMatrix(*executor, c.storage, c.width, 2 * q, 0.1);
  auto wk = MakeMatrix(*executor, c.storage, c.width, kv, 0.7);
  auto wv = MakeMatrix(*executor, c.storage, c.width, kv, 1.9);
  auto wo = MakeMatrix(*executor, c.storage, q, c.width, 2.6);
  auto q_norm = Upload<float>(*executor, Values(c.head_dim, 0.2, 0.5));
  auto k_norm = Upload<float>(*executor, Values(c.head_dim, 0.4, 0.5));
  ASSERT_TRUE(wq.ok() && wk.ok() && wv.ok() && wo.ok() && q_norm.ok() && k_norm.ok());
  auto lq = wq->Layer(*executor), lk = wk->Layer(*executor), lv = wv->Layer(*executor),
       lo = wo->Layer(*executor);
  ASSERT_TRUE(lq.ok() && lk.ok() && lv.ok() && lo.ok());
  auto branch = BatchedFullAttentionBranch::Create(*executor, p, c.batch, std::move(*lq),
                                                   std::move(*lk), std::move(*lv), std::move(*lo),
                                                   *q_norm, *k_norm, c.cache);
  ASSERT_TRUE(branch.ok());
  EXPECT_EQ((*branch)->input_types()[0],
            ActivationType(DataType::BF16, {ActivationType::kBatchDimension, 1, c.width}));

  // the reference's chain, one per sequence
  struct Chain {
    std::unique_ptr<KeyValueCache> cache;
    std::unique_ptr<FullyConnectedLayer> q, k, v, o;
    std::unique_ptr<QwenAttentionLayer> attention;
  };
  std::vector<Chain> chains(c.batch);
  for (Chain& chain : chains) {
    auto cache = KeyValueCache::Create(*executor, p.capacity, p.key_value_heads, p.head_dim, c.cache);
    auto q1 = wq->Layer(*executor), k1 = wk->Layer(*executor), v1 = wv->Layer(*executor),
         o1 = wo->Layer(*executor);
    ASSERT_TRUE(cache.ok() && q1.ok() && k1.ok() && v1.ok() && o1.ok());
    auto attention = QwenAttentionLayer::Create(*executor, p, *q_norm, *k_norm, 1, cache->get());
    ASSERT_TRUE(attention.ok());
    chain = Chain{std::move(*cache), std::move(*q1), std::move(*k1), std::move(*v1),
                  std::move(*o1), std::move(*attention)};
  }

  Agreement agreement;
  for (int step = 0; step < c.steps; ++step) {
    // sequence s starts over every s + 2 steps: lengths differ across the batch
    for (int s = 0; s < c.batch; ++s)
      if (step > 0 && step % (s + 2) == 0) {
        (*branch)->cache(s).Reset();
        chains[s].cache->Reset();
      }
    const auto hidden = Hidden(c.batch, c.width, step);
    auto rows = Upload<BFloat16>(*executor, hidden);
    ASSERT_TRUE(rows.ok());
    auto forward = (*branch)->fwd(*executor, {*rows});
    ASSERT_TRUE(forward.ok());
    const auto got = Read<BFloat16>(forward->outputs[0]);
    ASSERT_EQ(got.size(), static_cast<size_t>(c.batch) * c.width);
    for (int s = 0; s < c.batch; ++s) {
      Chain& chain = chains[s];
      auto token = Upload<BFloat16>(
          *executor, {hidden.begin() + static_cast<size_t>(s) * c.width,
                      hidden.begin() + static_cast<size_t>(s + 1) * c.width});
      ASSERT_TRUE(token.ok());
      auto pq = chain.q->fwd(*executor, {*token}), pk = chain.k->fwd(*executor, {*token}),
           pv = chain.v->fwd(*executor, {*token});
      ASSERT_TRUE(pq.ok() && pk.ok() && pv.ok());
      auto attended =
          chain.attention->fwd(*executor, {pq->outputs[0], pk->outputs[0], pv->outputs[0]});
      ASSERT_TRUE(attended.ok());
      auto projected = chain.o->fwd(*executor, {attended->outputs[0]});
      ASSERT_TRUE(projected.ok());
      agreement.Row(got, static_cast<size_t>(s) * c.width, Read<BFloat16>(projected->outputs[0]));
      EXPECT_EQ((*branch)->cache(s).position(), chain.cache->position());
    }
  }
  std::printf("attention branch, batch %d, %d/%d heads of %d, width %d: %d of %d outputs differ "
              "from the batch-one chain, worst %.2e of |x| + rms\n",
              c.batch, c.query_heads, c.kv_heads, c.head_dim, c.width, agreement.differing,
              agreement.compared, agreement.worst);
  if (c.batch <= 8)
    EXPECT_EQ(agreement.differing, 0);  // the projections share the one-token arithmetic
  else
    EXPECT_LE(agreement.worst, 2e-2);   // matrix-core projections: summation order differs
}

TEST(DecoderBranchTest, FullAttentionBranchEqualsTheChainOfBatchOneLayers) {
  for (auto cache : {KeyValueCache::Storage::kFloat32TokenMajor,
                     KeyValueCache::Storage::kBFloat16HeadMajor}) {
    RunAttentionCase({3, 96, 4, 2, 16, 8, 12, 9, MatrixStorage::kBFloat16, cache});
    RunAttentionCase({5, 256, 6, 1, 128, 64, 16, 7, MatrixStorage::kFp8E4M3, cache});
  }
}

TEST(DecoderBranchTest, FullAttentionBranchAtTheModelShape) {
  // 24 query and 4 key/value heads of 256, 64 rotary channels, FP8 projections
  // from and to a 5120-wide residual stream; 32 sequences.
  RunAttentionCase({32, 5120, 24, 4, 256, 64, 24, 6, MatrixStorage::kFp8E4M3,
                    KeyValueCache::Storage::kBFloat16HeadMajor});
}

struct DeltaCase {
  int batch, width, key_heads, value_heads, key_dim, value_dim, taps, steps;
  MatrixStorage storage;
};

void RunDeltaCase(const DeltaCase& c) {
  auto executor = NewExecutor();
  DeltaNetParameters p;
  p.key_heads = c.key_heads;
  p.value_heads = c.value_heads;
  p.key_head_dim = c.key_dim;
  p.value_head_dim = c.value_dim;
  p.conv_kernel_dim = c.taps;
  const int keys = c.key_heads * c.key_dim, values = c.value_heads * c.value_dim;
  const int channels = 2 * keys + values;
  auto wqkv = MakeMatrix(*executor, c.storage, c.width, channels, 0.1);
  auto wz = MakeMatrix(*executor, c.storage, c.width, values, 0.7);
  auto wa = MakeMatrix(*executor, c.storage, c.width, c.value_heads, 1.9);
  auto wb = MakeMatrix(*executor, c.storage, c.width, c.value_heads, 2.3);
  auto wo = MakeMatrix(*executor, c.storage, values, c.width, 2.6);
  auto conv = Upload<float>(*executor, Values(static_cast<size_t>(channels) * c.taps, 0.73, 0.6));
  auto a_log = Upload<float>(*executor, Values(c.value_heads, 0.18, 0.5));
  auto dt_bias = Upload<float>(*executor, Values(c.value_heads, -0.7, 0.3));
  auto norm = Upload<float>(*executor, Values(c.value_dim, 0.5, 0.6));
  ASSERT_TRUE(wqkv.ok() && wz.ok() && wa.ok() && wb.ok() && wo.ok());
  ASSERT_TRUE(conv.ok() && a_log.ok() && dt_bias.ok() && norm.ok());
  auto lqkv = wqkv->Layer(*executor), lz = wz->Layer(*executor), la = wa->Layer(*executor),
       lb = wb->Layer(*executor), lo = wo->Layer(*executor);
  ASSERT_TRUE(lqkv.ok() && lz.ok() && la.ok() && lb.ok() && lo.ok());
  auto branch = BatchedDeltaNetBranch::Create(*executor, p, c.batch, std::move(*lqkv),
                                              std::move(*lz), std::move(*la), std::move(*lb),
                                              std::move(*lo), *conv, *a_log, *dt_bias, *norm);
  ASSERT_TRUE(branch.ok());

  struct Chain {
    std::unique_ptr<FullyConnectedLayer> qkv, z, a, b, o;
    std::unique_ptr<DeltaNetLayer> mixer;
  };
  std::vector<Chain> chains(c.batch);
  for (Chain& chain : chains) {
    auto qkv1 = wqkv->Layer(*executor), z1 = wz->Layer(*executor), a1 = wa->Layer(*executor),
         b1 = wb->Layer(*executor), o1 = wo->Layer(*executor);
    auto mixer = DeltaNetLayer::Create(*executor, p, *conv, *a_log, *dt_bias, *norm);
    ASSERT_TRUE(qkv1.ok() && z1.ok() && a1.ok() && b1.ok() && o1.ok() && mixer.ok());
    chain = Chain{std::move(*qkv1), std::move(*z1), std::move(*a1),
                  std::move(*b1),   std::move(*o1), std::move(*mixer)};
  }

  Agreement agreement;
  for (int step = 0; step < c.steps; ++step) {
    const auto hidden = Hidden(c.batch, c.width, step);
    auto rows = Upload<BFloat16>(*executor, hidden);
    ASSERT_TRUE(rows.ok());
    auto forward = (*branch)->fwd(*executor, {*rows});
    ASSERT_TRUE(forward.ok());
    const auto got = Read<BFloat16>(forward->outputs[0]);
    for (int s = 0; s < c.batch; ++s) {
      Chain& chain = chains[s];
      auto token = Upload<BFloat16>(
          *executor, {hidden.begin() + static_cast<size_t>(s) * c.width,
                      hidden.begin() + static_cast<size_t>(s + 1) * c.width});
      ASSERT_TRUE(token.ok());
      auto pqkv = chain.qkv->fwd(*executor, {*token}), pz = chain.z->fwd(*executor, {*token}),
           pa = chain.a->fwd(*executor, {*token}), pb = chain.b->fwd(*executor, {*token});
      ASSERT_TRUE(pqkv.ok() && pz.ok() && pa.ok() && pb.ok());
      auto mixed = chain.mixer->fwd(
          *executor, {pqkv->outputs[0], pz->outputs[0], pa->outputs[0], pb->outputs[0]});
      ASSERT_TRUE(mixed.ok());
      auto projected = chain.o->fwd(*executor, {mixed->outputs[0]});
      ASSERT_TRUE(projected.ok());
      agreement.Row(got, static_cast<size_t>(s) * c.width, Read<BFloat16>(projected->outputs[0]));
    }
  }
  std::printf("delta-net branch, batch %d, %d/%d heads of %d x %d, width %d: %d of %d outputs "
              "differ from the batch-one chain, worst %.2e of |x| + rms\n",
              c.batch, c.key_heads, c.value_heads, c.key_dim, c.value_dim, c.width,
              agreement.differing, agreement.compared, agreement.worst);
  if (c.batch <= 8)
    EXPECT_EQ(agreement.differing, 0);
  else
    EXPECT_LE(agreement.worst, 2e-2);
  // Reset: the first step replays
  const auto hidden = Hidden(c.batch, c.width, 0);
  auto rows = Upload<BFloat16>(*executor, hidden);
  ASSERT_TRUE(rows.ok());
  ASSERT_TRUE((*branch)->Reset().ok());
  auto once = (*branch)->fwd(*executor, {*rows});
  ASSERT_TRUE((*branch)->Reset().ok());
  auto again = (*branch)->fwd(*executor, {*rows});
  ASSERT_TRUE(once.ok() && again.ok());
  EXPECT_TRUE(Read<BFloat16>(once->outputs[0]) == Read<BFloat16>(again->outputs[0]));
}

TEST(DecoderBranchTest, DeltaNetBranchEqualsTheChainOfBatchOneLayers) {
  RunDeltaCase({3, 96, 2, 6, 5, 7, 3, 6, MatrixStorage::kBFloat16});
  RunDeltaCase({5, 256, 2, 4, 128, 128, 4, 6, MatrixStorage::kFp8E4M3});
}

TEST(DecoderBranchTest, DeltaNetBranchAtTheModelShape) {
  // 16 key and 48 value heads of 128 x 128, four taps, FP8 projections from and
  // to a 5120-wide residual stream; 32 sequences.
  RunDeltaCase({32, 5120, 16, 48, 128, 128, 4, 5, MatrixStorage::kFp8E4M3});
}

TEST(DecoderBranchTest, RejectsMismatchedProjectionsInputsAndFullCaches) {
  auto executor = NewExecutor();
  auto elsewhere = NewExecutor();
  FullAttentionParameters p;
  p.query_heads = 4;
  p.key_value_heads = 2;
  p.head_dim = 16;
  p.rotary_dim = 8;
  p.capacity = 2;
  const int width = 96, q = 64, kv = 32;
  auto wq = MakeMatrix(*executor, MatrixStorage::kBFloat16, width, 2 * q, 0.1);
  auto wk = MakeMatrix(*executor, MatrixStorage::kBFloat16, width, kv, 0.7);
  auto wo = MakeMatrix(*executor, MatrixStorage::kBFloat16, q, width, 2.6);
  auto foreign = MakeMatrix(*elsewhere, MatrixStorage::kBFloat16, width, kv, 0.7);
  auto norm = Upload<float>(*executor, Values(16, 0.2));
  auto short_norm = Upload<float>(*executor, Values(15, 0.2));
  ASSERT_TRUE(wq.ok() && wk.ok() && wo.ok() && foreign.ok() && norm.ok() && short_norm.ok());
  auto make = [&](const Matrix& query, const Matrix& key, const Matrix& value, const Matrix& out,
                  const Buffer& q_norm, int batch) {
    auto lq = query.Layer(query.weights.executor()), lk = key.Layer(key.weights.executor()),
         lv = value.Layer(value.weights.executor()), lo = out.Layer(out.weights.executor());
    return BatchedFullAttentionBranch::Create(*executor, p, batch, std::move(*lq), std::move(*lk),
                                              std::move(*lv), std::move(*lo), q_norm, *norm);
  };
  EXPECT_TRUE(IsInvalidArgument(make(*wq, *wk, *wk, *wo, *norm, 0).status()));
  EXPECT_TRUE(IsInvalidArgument(make(*wk, *wk, *wk, *wo, *norm, 2).status()));   // query|gate width
  EXPECT_TRUE(IsInvalidArgument(make(*wq, *wq, *wk, *wo, *norm, 2).status()));   // key width
  EXPECT_TRUE(IsInvalidArgument(make(*wq, *wk, *wk, *wk, *norm, 2).status()));   // output input
  EXPECT_TRUE(IsInvalidArgument(make(*wq, *wk, *foreign, *wo, *norm, 2).status()));
  EXPECT_TRUE(IsInvalidArgument(make(*wq, *wk, *wk, *wo, *short_norm, 2).status()));
  auto trainable = FullyConnectedLayer::Create(*executor, width, kv, DataType::BF16);
  auto lq = wq->Layer(*executor), lk = wk->Layer(*executor), lo = wo->Layer(*executor);
  ASSERT_TRUE(trainable.ok() && lq.ok() && lk.ok() && lo.ok());
  EXPECT_TRUE(IsInvalidArgument(
      BatchedFullAttentionBranch::Create(*executor, p, 2, std::move(*lq), std::move(*lk),
                                         std::move(*trainable), std::move(*lo), *norm, *norm)
          .status()));

  auto branch = make(*wq, *wk, *wk, *wo, *norm, 2);
  ASSERT_TRUE(branch.ok());
  auto rows = Upload<BFloat16>(*executor, Hidden(2, width, 0));
  auto one_row = Upload<BFloat16>(*executor, Hidden(1, width, 0));
  ASSERT_TRUE(rows.ok() && one_row.ok());
  EXPECT_TRUE(IsInvalidArgument((*branch)->fwd(*executor, {*one_row}).status()));
  EXPECT_TRUE(IsInvalidArgument((*branch)->fwd(*executor, {*rows, *rows}).status()));
  EXPECT_TRUE(IsInvalidArgument((*branch)->fwd(*elsewhere, {*rows}).status()));
  EXPECT_EQ((*branch)->cache(0).position(), 0);
  ASSERT_TRUE((*branch)->fwd(*executor, {*rows}).ok());
  (*branch)->cache(1).Reset();
  ASSERT_TRUE((*branch)->fwd(*executor, {*rows}).ok());
  EXPECT_EQ((*branch)->cache(0).position(), 2);
  EXPECT_EQ((*branch)->cache(1).position(), 1);
  // sequence 0 is full: nothing runs and no cache moves
  EXPECT_TRUE(IsResourceExhausted((*branch)->fwd(*executor, {*rows}).status()));
  EXPECT_EQ((*branch)->cache(1).position(), 1);
  (*branch)->Reset();
  auto forward = (*branch)->fwd(*executor, {*rows});
  ASSERT_TRUE(forward.ok());
  EXPECT_TRUE(IsUnimplemented(
      (*branch)->bwd(*executor, {forward->outputs[0]}, std::move(forward->state)).status()));
}

}  // namespace
}  // namespace pluto::llm
