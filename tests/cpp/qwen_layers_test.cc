// Cached attention ops, QwenAttentionLayer, DeltaNetLayer and
// SequenceDeltaNetLayer through the host API; cases follow
// src/llm/layers/util/cached_attention_ops_test.cc, cached_attention_test.cc,
// qwen_attention_test.cc and sequence_delta_net_test.cc.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>

#include "pluto_amd/host/delta_net.h"
#include "pluto_amd/host/layer_hooks.h"
#include "pluto_amd/host/qwen_attention.h"
#include "pluto_amd/host/sequence_delta_net.h"
#include "tests/cpp/test_support.h"

namespace pluto::llm {
namespace {

using cached_attention_ops::CachedAttentionStep;
using cached_attention_ops::DeltaNetState;
using cached_attention_ops::ValidateCachedAttention;
using testing::BFloat16;
using testing::NewExecutor;
using testing::Read;
using testing::RoundedToBFloat16;
using testing::Upload;
using testing::Values;

float* Data(const hip::Buffer& buffer) { return static_cast<float*>(buffer.data()); }

FullAttentionParameters Small() {
  FullAttentionParameters p;
  p.query_heads = 2;
  p.key_value_heads = 1;
  p.head_dim = 4;
  p.rotary_dim = 2;
  p.capacity = 2;
  return p;
}

const KeyValueCache::Storage kStorages[] = {KeyValueCache::Storage::kFloat32TokenMajor,
                                            KeyValueCache::Storage::kBFloat16HeadMajor};

TEST(AttentionOpsTest, KnownAnswersCapacityAndReset) {
  // cached_attention_test.cc:108-156 through CachedAttentionStep
  for (auto storage : kStorages) {
    auto executor = NewExecutor();
    const auto p = Small();
    auto cache = KeyValueCache::Create(*executor, 2, 1, 4, storage);
    ASSERT_TRUE(cache.ok());
    auto zero = Upload<float>(*executor, std::vector<float>(16, 0.f));
    auto ones = Upload<float>(*executor, std::vector<float>(4, 1.f));
    auto v1 = Upload<float>(*executor, {2, 4, -2, -4});
    auto v2 = Upload<float>(*executor, {4, 8, 2, 4});
    auto output = Upload<float>(*executor, std::vector<float>(8, -1.f));
    auto probabilities = Upload<float>(*executor, std::vector<float>(4, -1.f));
    ASSERT_TRUE(CachedAttentionStep(*executor, p, **cache, Data(*zero), Data(*ones), Data(*v1),
                                    Data(*zero), Data(*zero), Data(*output), Data(*probabilities))
                    .ok());
    EXPECT_EQ((*cache)->position(), 1);
    EXPECT_TRUE(Read<float>(*output) == (std::vector<float>{1, 2, -1, -2, 1, 2, -1, -2}));
    ASSERT_TRUE(CachedAttentionStep(*executor, p, **cache, Data(*zero), Data(*ones), Data(*v2),
                                    Data(*zero), Data(*zero), Data(*output), Data(*probabilities))
                    .ok());
    EXPECT_EQ((*cache)->position(), 2);
    EXPECT_TRUE(Read<float>(*output) == (std::vector<float>{1.5, 3, 0, 0, 1.5, 3, 0, 0}));
    EXPECT_TRUE(Read<float>(*probabilities) == (std::vector<float>(4, 0.5f)));
    const Status full = CachedAttentionStep(*executor, p, **cache, Data(*zero), Data(*ones),
                                            Data(*v1), Data(*zero), Data(*zero), Data(*output));
    EXPECT_TRUE(IsResourceExhausted(full));
    EXPECT_EQ((*cache)->position(), 2);
    EXPECT_TRUE(Read<float>(*output) == (std::vector<float>{1.5, 3, 0, 0, 1.5, 3, 0, 0}));
    (*cache)->Reset();
    ASSERT_TRUE(CachedAttentionStep(*executor, p, **cache, Data(*zero), Data(*ones), Data(*v1),
                                    Data(*zero), Data(*zero), Data(*output))
                    .ok());
    EXPECT_TRUE(Read<float>(*output) == (std::vector<float>{1, 2, -1, -2, 1, 2, -1, -2}));
  }
}

TEST(AttentionOpsTest, GqaPartialRopeGatingAndCacheMatchTheOracleAcrossTiles) {
  // cached_attention_ops_test.cc:283-362: 70 tokens cross two 32-token tiles
  auto executor = NewExecutor();
  FullAttentionParameters p;
  p.query_heads = 4;
  p.key_value_heads = 2;
  p.head_dim = 6;
  p.rotary_dim = 4;
  p.capacity = 70;
  p.rope_theta = 73.f;
  const pluto_hip_attention_params abi = cached_attention_ops::ToAbi(p);
  pluto_oracle_attention_params oracle_p;
  static_assert(sizeof(oracle_p) == sizeof(abi));
  std::memcpy(&oracle_p, &abi, sizeof(abi));
  auto cache = KeyValueCache::Create(*executor, 70, 2, 6);
  ASSERT_TRUE(cache.ok());
  const auto q_norm = Values(6, 0.2, 0.3), k_norm = Values(6, 0.8, 0.4);
  auto dq = Upload<float>(*executor, q_norm), dk = Upload<float>(*executor, k_norm);
  std::vector<float> keys(70 * 12, 0.f), values(70 * 12, 0.f);
  for (int t = 0; t < 70; ++t) {
    const auto qg = RoundedToBFloat16(Values(4 * 2 * 6, 0.15 + t, 1.5));
    const auto k = RoundedToBFloat16(Values(12, 0.78 + 2 * t));
    const auto v = RoundedToBFloat16(Values(12, -0.31 + 3 * t));
    std::vector<float> want(24), want_p(4 * (t + 1));
    ASSERT_EQ(pluto_oracle_gqa_cached_step(&oracle_p, keys.data(), values.data(), t, qg.data(),
                                           k.data(), v.data(), q_norm.data(), k_norm.data(),
                                           want.data(), want_p.data()), 0);
    auto dqg = Upload<float>(*executor, qg), dkk = Upload<float>(*executor, k),
         dv = Upload<float>(*executor, v);
    auto out = hip::Buffer::Allocate(*executor, 24 * sizeof(float));
    auto probs = hip::Buffer::Allocate(*executor, want_p.size() * sizeof(float));
    ASSERT_TRUE(CachedAttentionStep(*executor, p, **cache, Data(*dqg), Data(*dkk), Data(*dv),
                                    Data(*dq), Data(*dk), Data(*out), Data(*probs)).ok());
    if (t % 23 != 0 && t != 69) continue;
    const auto got = Read<float>(*out), got_p = Read<float>(*probs);
    for (size_t i = 0; i < got.size(); ++i)
      EXPECT_NEAR(got[i], want[i], 2e-4 + 1.6e-2 * std::fabs(want[i]));
    double sum = 0;
    for (size_t i = 0; i < got_p.size(); ++i) {
      EXPECT_NEAR(got_p[i], want_p[i], 1e-5 + 1e-3 * want_p[i]);
      sum += got_p[i];
    }
    EXPECT_NEAR(sum, 4.0, 1e-5);
  }
  EXPECT_EQ((*cache)->position(), 70);
  const auto got_values = Read<float>((*cache)->values());
  EXPECT_TRUE(got_values == values);
}

TEST(AttentionOpsTest, BatchedStepEqualsTheSingleStepOfEverySequence) {
  // The decoder step of Model::Step (qwen/model.cc:405-428) lifted to several
  // sequences: three caches at different positions advance together, every
  // output row bit for bit that of CachedAttentionStep on its own.
  using cached_attention_ops::CachedAttentionStepBatch;
  for (auto storage : kStorages) {
    auto executor = NewExecutor();
    FullAttentionParameters p;
    p.query_heads = 4;
    p.key_value_heads = 2;
    p.head_dim = 8;
    p.rotary_dim = 4;
    p.capacity = 40;
    const int batch = 3, row = p.query_heads * p.head_dim, kv = p.key_value_heads * p.head_dim;
    const auto q_norm = Values(8, 0.2, 0.3), k_norm = Values(8, 0.8, 0.4);
    auto dq = Upload<float>(*executor, q_norm), dk = Upload<float>(*executor, k_norm);
    std::vector<std::unique_ptr<KeyValueCache>> together, alone;
    for (int s = 0; s < 2 * batch; ++s) {
      auto cache = KeyValueCache::Create(*executor, 40, 2, 8, storage);
      ASSERT_TRUE(cache.ok());
      (s < batch ? together : alone).push_back(std::move(*cache));
    }
    auto token = [&](int s, int t, double phase, int count) {
      return RoundedToBFloat16(Values(count, phase + 0.37 * s + 1.3 * t));
    };
    // different histories: sequence s starts with 5 s tokens of its own
    for (int s = 0; s < batch; ++s)
      for (int t = 0; t < 5 * s; ++t) {
        auto qg = Upload<float>(*executor, token(s, t, 0.1, 2 * row));
        auto k = Upload<float>(*executor, token(s, t, 0.7, kv));
        auto v = Upload<float>(*executor, token(s, t, -0.4, kv));
        auto out = hip::Buffer::Allocate(*executor, row * sizeof(float));
        for (auto* cache : {together[s].get(), alone[s].get()})
          ASSERT_TRUE(CachedAttentionStep(*executor, p, *cache, Data(*qg), Data(*k), Data(*v),
                                          Data(*dq), Data(*dk), Data(*out)).ok());
      }
    std::vector<KeyValueCache*> caches;
    for (auto& cache : together) caches.push_back(cache.get());
    for (int t = 100; t < 103; ++t) {
      std::vector<float> qg, k, v;
      for (int s = 0; s < batch; ++s) {
        const auto a = token(s, t, 0.1, 2 * row), b = token(s, t, 0.7, kv), c = token(s, t, -0.4, kv);
        qg.insert(qg.end(), a.begin(), a.end());
        k.insert(k.end(), b.begin(), b.end());
        v.insert(v.end(), c.begin(), c.end());
      }
      auto dqg = Upload<float>(*executor, qg), dkk = Upload<float>(*executor, k),
           dv = Upload<float>(*executor, v);
      auto out = hip::Buffer::Allocate(*executor, batch * row * sizeof(float));
      ASSERT_TRUE(CachedAttentionStepBatch(*executor, p, caches, Data(*dqg), Data(*dkk), Data(*dv),
                                           Data(*dq), Data(*dk), Data(*out)).ok());
      const auto got = Read<float>(*out);
      for (int s = 0; s < batch; ++s) {
        auto one = hip::Buffer::Allocate(*executor, row * sizeof(float));
        ASSERT_TRUE(CachedAttentionStep(*executor, p, *alone[s], Data(*dqg) + s * 2 * row,
                                        Data(*dkk) + s * kv, Data(*dv) + s * kv, Data(*dq),
                                        Data(*dk), Data(*one)).ok());
        const auto want = Read<float>(*one);
        EXPECT_TRUE(std::equal(want.begin(), want.end(), got.begin() + s * row));
        EXPECT_EQ(together[s]->position(), alone[s]->position());
      }
    }
    // a full cache anywhere in the batch stops the call before any cache moves
    auto full = KeyValueCache::Create(*executor, 40, 2, 8, storage);
    ASSERT_TRUE(full.ok());
    auto scratch = Upload<float>(*executor, std::vector<float>(batch * 2 * row, 0.f));
    for (int t = 0; t < 40; ++t)
      ASSERT_TRUE(CachedAttentionStep(*executor, p, **full, Data(*scratch), Data(*scratch),
                                      Data(*scratch), Data(*dq), Data(*dk), Data(*scratch)).ok());
    const int before = together[0]->position();
    std::vector<KeyValueCache*> with_full = {together[0].get(), full->get()};
    EXPECT_TRUE(IsResourceExhausted(CachedAttentionStepBatch(
        *executor, p, with_full, Data(*scratch), Data(*scratch), Data(*scratch), Data(*dq),
        Data(*dk), Data(*scratch))));
    EXPECT_EQ(together[0]->position(), before);
    std::vector<KeyValueCache*> twice = {together[0].get(), together[0].get()};
    EXPECT_TRUE(IsInvalidArgument(CachedAttentionStepBatch(
        *executor, p, twice, Data(*scratch), Data(*scratch), Data(*scratch), Data(*dq), Data(*dk),
        Data(*scratch))));
  }
}

TEST(AttentionOpsTest, BatchedDeltaNetStateEqualsIndependentStates) {
  auto executor = NewExecutor();
  cached_attention_ops::DeltaNetParameters delta;
  delta.key_heads = 2;
  delta.value_heads = 4;
  delta.key_head_dim = 16;
  delta.value_head_dim = 24;
  const int batch = 3, channels = 2 * 2 * 16 + 4 * 24, width = 4 * 24, heads = 4;
  EXPECT_TRUE(IsInvalidArgument(DeltaNetState::Create(*executor, delta, 0).status()));
  auto together = DeltaNetState::Create(*executor, delta, batch);
  ASSERT_TRUE(together.ok());
  EXPECT_EQ((*together)->batch(), batch);
  std::vector<std::unique_ptr<DeltaNetState>> alone;
  for (int s = 0; s < batch; ++s) {
    auto state = DeltaNetState::Create(*executor, delta);
    ASSERT_TRUE(state.ok());
    alone.push_back(std::move(*state));
  }
  auto conv = Upload<float>(*executor, Values(channels * 4, 0.73, 0.6));
  auto a_log = Upload<float>(*executor, Values(heads, 0.18, 0.5));
  auto dt = Upload<float>(*executor, Values(heads, -0.7, 0.3));
  auto norm = Upload<float>(*executor, Values(24, 0.5, 0.6));
  for (int t = 0; t < 4; ++t) {
    auto qkv = Upload<float>(*executor, Values(batch * channels, 0.3 + t));
    auto z = Upload<float>(*executor, Values(batch * width, -0.6 + t));
    auto a = Upload<float>(*executor, Values(batch * heads, 0.1 + t));
    auto b = Upload<float>(*executor, Values(batch * heads, -0.7 + t));
    auto out = hip::Buffer::Allocate(*executor, batch * width * sizeof(float));
    ASSERT_TRUE((*together)->Step(Data(*qkv), Data(*z), Data(*a), Data(*b), Data(*conv),
                                  Data(*a_log), Data(*dt), Data(*norm), Data(*out)).ok());
    const auto got = Read<float>(*out);
    for (int s = 0; s < batch; ++s) {
      auto one = hip::Buffer::Allocate(*executor, width * sizeof(float));
      ASSERT_TRUE(alone[s]->Step(Data(*qkv) + s * channels, Data(*z) + s * width,
                                 Data(*a) + s * heads, Data(*b) + s * heads, Data(*conv),
                                 Data(*a_log), Data(*dt), Data(*norm), Data(*one)).ok());
      const auto want = Read<float>(*one);
      EXPECT_TRUE(std::equal(want.begin(), want.end(), got.begin() + s * width));
    }
  }
}

TEST(AttentionOpsTest, CachedAttentionRejectsInvalidParametersBeforeWork) {
  auto executor = NewExecutor();
  const auto p = Small();
  auto cache = KeyValueCache::Create(*executor, p.capacity, p.key_value_heads, p.head_dim);
  auto output = Upload<float>(*executor, std::vector<float>(16, -13.f));
  ASSERT_TRUE(cache.ok());
  ASSERT_TRUE(output.ok());
  const auto check_invalid = [&](const FullAttentionParameters& invalid) {
    EXPECT_TRUE(IsInvalidArgument(ValidateCachedAttention(*executor, invalid, **cache)));
    EXPECT_TRUE(IsInvalidArgument(CachedAttentionStep(*executor, invalid, **cache, Data(*output),
                                                      Data(*output), Data(*output), Data(*output),
                                                      Data(*output), Data(*output))));
    EXPECT_EQ((*cache)->position(), 0);
  };
  const int int_max = std::numeric_limits<int>::max();
  for (int count : {0, -1, int_max}) {
    auto invalid = p;
    invalid.query_heads = count;
    check_invalid(invalid);
    invalid = p;
    invalid.key_value_heads = count;
    check_invalid(invalid);
  }
  auto invalid = p;
  invalid.query_heads = 3;
  invalid.key_value_heads = 2;
  check_invalid(invalid);
  for (int dim : {0, -1, 257, int_max}) {
    invalid = p;
    invalid.head_dim = dim;
    check_invalid(invalid);
  }
  for (int dim : {0, -1, 3, 6}) {
    invalid = p;
    invalid.rotary_dim = dim;
    check_invalid(invalid);
  }
  for (int capacity : {0, -1, int_max}) {
    invalid = p;
    invalid.capacity = capacity;
    check_invalid(invalid);
  }
  for (float value : {0.f, -1.f, std::numeric_limits<float>::infinity(),
                      std::numeric_limits<float>::quiet_NaN()}) {
    invalid = p;
    invalid.rope_theta = value;
    check_invalid(invalid);
    invalid = p;
    invalid.rms_norm_epsilon = value;
    check_invalid(invalid);
  }
  EXPECT_TRUE(Read<float>(*output) == (std::vector<float>(16, -13.f)));
}

TEST(AttentionOpsTest, CachedAttentionRejectsMismatchedCacheBeforeWork) {
  auto executor = NewExecutor();
  const auto p = Small();
  auto output = Upload<float>(*executor, std::vector<float>(16, -17.f));
  ASSERT_TRUE(output.ok());
  const int wrong_shapes[][3] = {{3, 1, 4}, {2, 2, 4}, {2, 1, 6}};
  for (const auto& shape : wrong_shapes) {
    auto cache = KeyValueCache::Create(*executor, shape[0], shape[1], shape[2]);
    ASSERT_TRUE(cache.ok());
    EXPECT_TRUE(IsInvalidArgument(ValidateCachedAttention(*executor, p, **cache)));
    EXPECT_TRUE(IsInvalidArgument(CachedAttentionStep(*executor, p, **cache, Data(*output),
                                                      Data(*output), Data(*output), Data(*output),
                                                      Data(*output), Data(*output))));
    EXPECT_EQ((*cache)->position(), 0);
  }
  auto other = NewExecutor();
  auto foreign = KeyValueCache::Create(*other, p.capacity, p.key_value_heads, p.head_dim);
  ASSERT_TRUE(foreign.ok());
  EXPECT_TRUE(IsInvalidArgument(ValidateCachedAttention(*executor, p, **foreign)));
  EXPECT_TRUE(IsInvalidArgument(CachedAttentionStep(*executor, p, **foreign, Data(*output),
                                                    Data(*output), Data(*output), Data(*output),
                                                    Data(*output), Data(*output))));
  EXPECT_EQ((*foreign)->position(), 0);
  EXPECT_TRUE(Read<float>(*output) == (std::vector<float>(16, -17.f)));
}

TEST(AttentionOpsTest, CachedAttentionRejectsNullPointersWithoutAdvancing) {
  auto executor = NewExecutor();
  const auto p = Small();
  auto cache = KeyValueCache::Create(*executor, p.capacity, p.key_value_heads, p.head_dim);
  auto output = Upload<float>(*executor, std::vector<float>(16, -19.f));
  ASSERT_TRUE(cache.ok());
  for (int missing = 0; missing < 6; ++missing) {
    float* pointers[6];
    std::fill_n(pointers, 6, Data(*output));
    pointers[missing] = nullptr;
    EXPECT_TRUE(IsInvalidArgument(CachedAttentionStep(*executor, p, **cache, pointers[0],
                                                      pointers[1], pointers[2], pointers[3],
                                                      pointers[4], pointers[5])));
    EXPECT_EQ((*cache)->position(), 0);
  }
  EXPECT_TRUE(Read<float>(*output) == (std::vector<float>(16, -19.f)));
}

TEST(AttentionOpsTest, DeltaNetRejectsUnsupportedShapesAndNullInputs) {
  auto executor = NewExecutor();
  DeltaNetParameters delta;
  delta.key_head_dim = 129;
  EXPECT_TRUE(IsInvalidArgument(DeltaNetState::Create(*executor, delta).status()));
  delta.key_head_dim = 5;
  delta.value_head_dim = 7;
  auto state = DeltaNetState::Create(*executor, delta);
  ASSERT_TRUE(state.ok());
  EXPECT_TRUE(IsInvalidArgument((*state)->Step(nullptr, nullptr, nullptr, nullptr, nullptr,
                                               nullptr, nullptr, nullptr, nullptr)));
}

StatusOr<std::shared_ptr<BlockParameter>> Parameter(hip::Executor& executor,
                                                    const std::vector<float>& values) {
  ASSIGN_OR_RETURN(auto buffer, Upload<float>(executor, values));
  return BlockParameter::Create(executor, std::move(buffer), DataType::FP32);
}

TEST(QwenAttentionTest, ForwardMatchesCachedAttentionAndCausalHook) {
  // qwen_attention_test.cc:155-228.  The reference compares the two paths bit
  // for bit.  Here the sequence path (flash tiles, bf16 probabilities) and the
  // cached path (split-K, FP32-accurate probabilities) sum in different
  // orders, so bf16(core) can land on either side of a rounding boundary and
  // the gated product bf16(bf16(core) * bf16(gate)) then moves by up to two
  // units in the last place in general.  On the reference's own cases the two
  // paths do agree bit for bit, and that is what is asserted, as in the
  // reference (the counts are printed).
  auto executor = NewExecutor();
  for (int d : {3, 256, 128}) {
    FullAttentionParameters p;
    p.query_heads = 2;
    p.key_value_heads = 1;
    p.head_dim = d;
    p.rotary_dim = d == 3 ? 2 : 64;
    p.capacity = 40;
    const int length = d == 3 ? 33 : d == 256 ? 3 : 40;
    const auto qg = Values(static_cast<size_t>(length) * 2 * p.query_heads * d, .1);
    const auto k = Values(static_cast<size_t>(length) * d, 1.2),
               v = Values(static_cast<size_t>(length) * d, 2.3);
    auto qw = Parameter(*executor, Values(d, .2)), kw = Parameter(*executor, Values(d, .4));
    ASSERT_TRUE(qw.ok());
    ASSERT_TRUE(kw.ok());
    auto layer = QwenAttentionLayer::Create(*executor, p, *qw, *kw, length);
    ASSERT_TRUE(layer.ok());
    auto qgb = Upload<BFloat16>(*executor, qg), kb = Upload<BFloat16>(*executor, k),
         vb = Upload<BFloat16>(*executor, v);
    LayerHooks hooks;
    int hook_calls = 0;
    hooks.attention_probabilities_hook = [&](hip::Executor&, std::string_view,
                                             const ActivationType& type, const Buffer& buffer) {
      EXPECT_EQ(type, ActivationType(DataType::FP32, {1, 2, length, length}));
      const auto probs = Read<float>(buffer);
      for (int h = 0; h < 2; ++h)
        for (int row = 0; row < length; ++row) {
          double sum = 0;
          for (int t = 0; t < length; ++t) {
            const float value = probs[(h * length + row) * length + t];
            if (t > row) EXPECT_EQ(value, 0.0f);
            sum += value;
          }
          EXPECT_NEAR(sum, 1, 2e-6);
        }
      ++hook_calls;
      return OkStatus();
    };
    auto fwd = (*layer)->fwd(*executor, {*qgb, *kb, *vb}, &hooks);
    ASSERT_TRUE(fwd.ok());
    EXPECT_EQ(hook_calls, 1);
    const auto actual = Read<BFloat16>(fwd->outputs[0]);
    for (auto storage : kStorages) {
      auto cache = KeyValueCache::Create(*executor, p.capacity, p.key_value_heads, p.head_dim,
                                         storage);
      ASSERT_TRUE(cache.ok());
      auto cached_layer = QwenAttentionLayer::Create(*executor, p, *qw, *kw, 1, cache->get());
      ASSERT_TRUE(cached_layer.ok());
      int differing = 0, compared = 0, worst = 0;
      for (int row = 0; row < length; ++row) {
        auto qi = Upload<BFloat16>(*executor, {qg.begin() + row * 4 * d, qg.begin() + (row + 1) * 4 * d});
        auto ki = Upload<BFloat16>(*executor, {k.begin() + row * d, k.begin() + (row + 1) * d});
        auto vi = Upload<BFloat16>(*executor, {v.begin() + row * d, v.begin() + (row + 1) * d});
        auto output = (*cached_layer)->fwd(*executor, {*qi, *ki, *vi});
        ASSERT_TRUE(output.ok());
        EXPECT_EQ((*cache)->position(), row + 1);
        const auto expected = Read<BFloat16>(output->outputs[0]);
        for (int c = 0; c < 2 * d; ++c) {
          // bf16 bit patterns as integers that count representable values
          auto ordered = [](BFloat16 bits) {
            return (bits & 0x8000) ? -static_cast<int>(bits & 0x7fff) : static_cast<int>(bits);
          };
          const int ulps = std::abs(ordered(actual[row * 2 * d + c]) - ordered(expected[c]));
          EXPECT_LE(ulps, 2) << "d=" << d << " row=" << row << " c=" << c;
          differing += ulps != 0;
          worst = std::max(worst, ulps);
          ++compared;
        }
      }
      std::printf("sequence vs cached path, d=%d: %d of %d outputs differ, by at most %d bf16 ulp\n",
                  d, differing, compared, worst);
      EXPECT_EQ(differing, 0);
    }
  }
}

TEST(QwenAttentionTest, CachedHookReportsOneQueryRowPerToken) {
  auto executor = NewExecutor();
  auto p = Small();
  p.capacity = 3;
  auto cache = KeyValueCache::Create(*executor, 3, 1, 4);
  auto qw = Upload<float>(*executor, Values(4, .2)), kw = Upload<float>(*executor, Values(4, .4));
  ASSERT_TRUE(cache.ok());
  auto layer = QwenAttentionLayer::Create(*executor, p, *qw, *kw, 1, cache->get());
  ASSERT_TRUE(layer.ok());
  auto q = Upload<BFloat16>(*executor, Values(16, .1)), k = Upload<BFloat16>(*executor, Values(4, 1.2)),
       v = Upload<BFloat16>(*executor, Values(4, 2.3));
  int calls = 0;
  LayerHooks hooks;
  hooks.attention_probabilities_hook = [&](hip::Executor&, std::string_view name,
                                           const ActivationType& type, const Buffer& buffer) {
    ++calls;
    EXPECT_EQ(name, "QwenAttentionLayer");
    EXPECT_EQ(type, ActivationType(DataType::FP32, {1, 2, 1, calls}));
    const auto probs = Read<float>(buffer);
    for (int h = 0; h < 2; ++h) {
      double sum = 0;
      for (int t = 0; t < calls; ++t) sum += probs[h * calls + t];
      EXPECT_NEAR(sum, 1, 2e-6);
    }
    return OkStatus();
  };
  for (int step = 0; step < 3; ++step) ASSERT_TRUE((*layer)->fwd(*executor, {*q, *k, *v}, &hooks).ok());
  EXPECT_EQ(calls, 3);
  // a full cache fails before any work and keeps its position
  EXPECT_TRUE(IsResourceExhausted((*layer)->fwd(*executor, {*q, *k, *v}, &hooks).status()));
  EXPECT_EQ((*cache)->position(), 3);
  EXPECT_EQ(calls, 3);
}

TEST(QwenAttentionTest, CachePointerSelectsBackwardContractAtLengthOne) {
  auto executor = NewExecutor();
  const auto p = Small();
  auto qw = Parameter(*executor, Values(4, .2)), kw = Parameter(*executor, Values(4, .4));
  auto cache = KeyValueCache::Create(*executor, p.capacity, p.key_value_heads, p.head_dim);
  ASSERT_TRUE(cache.ok());
  auto sequence = QwenAttentionLayer::Create(*executor, p, *qw, *kw, 1);
  auto cached = QwenAttentionLayer::Create(*executor, p, *qw, *kw, 1, cache->get());
  ASSERT_TRUE(sequence.ok());
  ASSERT_TRUE(cached.ok());
  EXPECT_EQ((*sequence)->input_types()[0], (*cached)->input_types()[0]);
  EXPECT_EQ((*sequence)->output_types()[0], (*cached)->output_types()[0]);
  auto q = Upload<BFloat16>(*executor, Values(16, .1));
  auto k = Upload<BFloat16>(*executor, Values(4, 1.2));
  auto v = Upload<BFloat16>(*executor, Values(4, 2.3));
  auto dy = Upload<float>(*executor, Values(8, .7));
  auto sf = (*sequence)->fwd(*executor, {*q, *k, *v});
  auto cf = (*cached)->fwd(*executor, {*q, *k, *v});
  ASSERT_TRUE(sf.ok());
  ASSERT_TRUE(cf.ok());
  EXPECT_TRUE(Read<BFloat16>(sf->outputs[0]) == Read<BFloat16>(cf->outputs[0]));
  EXPECT_EQ((*cache)->position(), 1);
  EXPECT_TRUE(IsUnimplemented((*cached)->bwd(*executor, {*dy}, std::move(cf->state)).status()));
  // qwen_attention_test.cc:394-405: the sequence contract differentiates
  auto backward = (*sequence)->bwd(*executor, {*dy}, std::move(sf->state));
  ASSERT_TRUE(backward.ok());
  ASSERT_EQ(backward->size(), 3u);
  float value_magnitude = 0;
  for (float gradient : Read<float>((*backward)[2])) {
    EXPECT_TRUE(std::isfinite(gradient));
    value_magnitude += std::fabs(gradient);
  }
  EXPECT_GT(value_magnitude, 1e-5f);
  EXPECT_EQ((*cache)->position(), 1);
}

TEST(QwenAttentionTest, FullBackwardMatchesTheOracleAndAccumulatesNormGradients) {
  // qwen_attention_test.cc:230-300.  The oracle's backward is itself checked
  // against finite differences of a frozen-rounding forward; here the layer is
  // checked against the oracle, with the reference's bound of 3e-5.
  for (bool use_bf16_rounding : {false, true}) {
    auto executor = NewExecutor();
    FullAttentionParameters p;
    p.query_heads = 2;
    p.key_value_heads = 1;
    p.head_dim = 3;
    p.rotary_dim = 2;
    p.round_to_bfloat16 = use_bf16_rounding;
    constexpr int t = 3;
    const std::vector<float> qg = RoundedToBFloat16(Values(t * 12, .1)),
                             k = RoundedToBFloat16(Values(t * 3, 1.2)),
                             v = RoundedToBFloat16(Values(t * 3, 2.3)), qn = Values(3, .2),
                             kn = Values(3, .4), upstream = Values(t * 6, .7);
    auto qw = Parameter(*executor, qn), kw = Parameter(*executor, kn);
    ASSERT_TRUE((*qw)->Activate().ok());
    ASSERT_TRUE((*kw)->Activate().ok());
    ASSERT_TRUE((*qw)->Activate().ok());  // idempotent
    auto layer = QwenAttentionLayer::Create(*executor, p, *qw, *kw, t);
    ASSERT_TRUE(layer.ok());
    auto qgb = Upload<BFloat16>(*executor, qg), kb = Upload<BFloat16>(*executor, k),
         vb = Upload<BFloat16>(*executor, v);
    auto dy = Upload<float>(*executor, upstream);
    auto fwd = (*layer)->fwd(*executor, {*qgb, *kb, *vb});
    ASSERT_TRUE(fwd.ok());
    auto backward = (*layer)->bwd(*executor, {*dy}, std::move(fwd->state));
    ASSERT_TRUE(backward.ok());
    std::vector<std::vector<float>> actual;
    for (const auto& b : *backward) actual.push_back(Read<float>(b));
    actual.push_back(Read<float>((*qw)->gradient()));
    actual.push_back(Read<float>((*kw)->gradient()));

    const pluto_hip_attention_params abi = cached_attention_ops::ToAbi(p);
    pluto_oracle_attention_params oracle_p;
    static_assert(sizeof(oracle_p) == sizeof(abi));
    std::memcpy(&oracle_p, &abi, sizeof(abi));
    std::vector<std::vector<float>> want = {std::vector<float>(t * 12), std::vector<float>(t * 3),
                                            std::vector<float>(t * 3), std::vector<float>(3, 0.f),
                                            std::vector<float>(3, 0.f)};
    ASSERT_EQ(pluto_oracle_gqa_sequence_backward(&oracle_p, t, qg.data(), k.data(), v.data(),
                                                 qn.data(), kn.data(), upstream.data(),
                                                 want[0].data(), want[1].data(), want[2].data(),
                                                 want[3].data(), want[4].data()),
              0);
    for (size_t which = 0; which < want.size(); ++which) {
      ASSERT_EQ(actual[which].size(), want[which].size());
      for (size_t i = 0; i < want[which].size(); ++i)
        EXPECT_NEAR(actual[which][i], want[which][i], 3e-5);
    }
    // Shared norm gradients accumulate across backward calls, not overwrite.
    auto second = (*layer)->fwd(*executor, {*qgb, *kb, *vb});
    ASSERT_TRUE(second.ok());
    auto repeated = (*layer)->bwd(*executor, {*dy}, std::move(second->state));
    ASSERT_TRUE(repeated.ok());
    for (size_t i = 0; i < repeated->size(); ++i)
      EXPECT_TRUE(Read<float>((*repeated)[i]) == actual[i]);
    const auto summed = Read<float>((*qw)->gradient());
    for (size_t i = 0; i < summed.size(); ++i) EXPECT_NEAR(summed[i], 2 * actual[3][i], 1e-6);
    EXPECT_TRUE((*layer)->gradients().empty());
    // a state of the wrong shape is rejected
    auto third = (*layer)->fwd(*executor, {*qgb, *kb, *vb});
    ASSERT_TRUE(third.ok());
    third->state.intermediates.pop_back();
    EXPECT_TRUE(IsInvalidArgument((*layer)->bwd(*executor, {*dy}, std::move(third->state)).status()));
    ASSERT_TRUE((*qw)->Deactivate().ok());
    EXPECT_FALSE((*qw)->active());
  }
}

TEST(QwenAttentionTest, FrozenNormsStillPropagateToEarlierTokens) {
  // qwen_attention_test.cc:303-345
  auto executor = NewExecutor();
  FullAttentionParameters p;
  p.query_heads = 2;
  p.key_value_heads = 1;
  p.head_dim = 4;
  p.rotary_dim = 2;
  auto qw = Parameter(*executor, Values(4, .2)), kw = Parameter(*executor, Values(4, .4));
  auto layer = QwenAttentionLayer::Create(*executor, p, *qw, *kw, 3);
  ASSERT_TRUE(layer.ok());
  auto q = Upload<BFloat16>(*executor, Values(48, .1)), k = Upload<BFloat16>(*executor, Values(12, 1.2)),
       v = Upload<BFloat16>(*executor, Values(12, 2.3));
  auto result = (*layer)->fwd(*executor, {*q, *k, *v});
  ASSERT_TRUE(result.ok());
  std::vector<float> grad(24, 0.f);
  for (int i = 16; i < 24; ++i) grad[i] = .5f;
  auto dy = Upload<float>(*executor, grad);
  auto backward = (*layer)->bwd(*executor, {*dy}, std::move(result->state));
  ASSERT_TRUE(backward.ok());
  const auto dk = Read<float>((*backward)[1]), dv = Read<float>((*backward)[2]);
  float key_magnitude = 0, value_magnitude = 0;
  for (int i = 0; i < 4; ++i) {
    key_magnitude += std::fabs(dk[i]);
    value_magnitude += std::fabs(dv[i]);
  }
  EXPECT_GT(key_magnitude, 1e-5f);
  EXPECT_GT(value_magnitude, 1e-5f);
  EXPECT_FALSE((*qw)->active());
  EXPECT_FALSE((*kw)->active());
  // a gradient buffer of the wrong size is rejected
  auto again = (*layer)->fwd(*executor, {*q, *k, *v});
  ASSERT_TRUE(again.ok());
  auto short_dy = Upload<float>(*executor, std::vector<float>(23, 0.f));
  EXPECT_TRUE(IsInvalidArgument((*layer)->bwd(*executor, {*short_dy}, std::move(again->state)).status()));
}

TEST(QwenAttentionTest, RejectsIncompatibleCacheAndSequenceContracts) {
  // cached_attention_test.cc:186-230
  auto executor = NewExecutor();
  auto other = NewExecutor();
  const auto p = Small();
  auto qw = Upload<float>(*executor, Values(4, .2)), kw = Upload<float>(*executor, Values(4, .4));
  auto cache = KeyValueCache::Create(*executor, 2, 1, 4);
  auto wrong = KeyValueCache::Create(*executor, 3, 1, 4);
  auto foreign = KeyValueCache::Create(*other, 2, 1, 4);
  ASSERT_TRUE(cache.ok());
  EXPECT_TRUE(IsInvalidArgument(
      QwenAttentionLayer::Create(*executor, p, *qw, *kw, 2, cache->get()).status()));
  EXPECT_TRUE(IsInvalidArgument(
      QwenAttentionLayer::Create(*executor, p, *qw, *kw, 1, wrong->get()).status()));
  EXPECT_TRUE(IsInvalidArgument(
      QwenAttentionLayer::Create(*executor, p, *qw, *kw, 1, foreign->get()).status()));
  auto short_norm = Upload<float>(*executor, Values(3, .2));
  EXPECT_TRUE(IsInvalidArgument(
      QwenAttentionLayer::Create(*executor, p, *short_norm, *kw, 1, cache->get()).status()));
  EXPECT_TRUE(IsInvalidArgument(QwenAttentionLayer::Create(*executor, p, *qw, *kw, 0).status()));
  auto bad = p;
  bad.head_dim = 257;
  EXPECT_TRUE(IsInvalidArgument(QwenAttentionLayer::Create(*executor, bad, *qw, *kw, 4).status()));
  auto layer = QwenAttentionLayer::Create(*executor, p, *qw, *kw, 1, cache->get());
  ASSERT_TRUE(layer.ok());
  auto q = Upload<BFloat16>(*executor, Values(16, .1));
  auto k = Upload<BFloat16>(*executor, Values(4, 1.2));
  auto short_k = Upload<BFloat16>(*executor, Values(3, 1.2));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*q, *k}).status()));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*q, *short_k, *k}).status()));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*other, {*q, *k, *k}).status()));
  EXPECT_EQ((*cache)->position(), 0);
}

TEST(QwenAttentionTest, NullCacheWithRawNormsRemainsStateless) {
  auto executor = NewExecutor();
  auto p = Small();
  p.capacity = 0;  // a sequence-only layer has no cache capacity to validate
  auto qw = Parameter(*executor, Values(4, .2)), kw = Parameter(*executor, Values(4, .4));
  auto reference = QwenAttentionLayer::Create(*executor, p, *qw, *kw, 3);
  auto raw = QwenAttentionLayer::Create(*executor, p, (*qw)->value(), (*kw)->value(), 3, nullptr);
  ASSERT_TRUE(reference.ok());
  ASSERT_TRUE(raw.ok());
  EXPECT_EQ((*raw)->weights()[0].data(), (*qw)->value().data());
  EXPECT_EQ((*raw)->weights()[1].data(), (*kw)->value().data());
  EXPECT_TRUE((*raw)->gradients().empty());
  auto q = Upload<BFloat16>(*executor, Values(48, .1));
  auto k = Upload<BFloat16>(*executor, Values(12, 1.2));
  auto v = Upload<BFloat16>(*executor, Values(12, 2.3));
  auto expected = (*reference)->fwd(*executor, {*q, *k, *v});
  ASSERT_TRUE(expected.ok());
  for (int repetition = 0; repetition < 2; ++repetition) {
    auto actual = (*raw)->fwd(*executor, {*q, *k, *v});
    ASSERT_TRUE(actual.ok());
    EXPECT_TRUE(Read<BFloat16>(actual->outputs[0]) == Read<BFloat16>(expected->outputs[0]));
  }
}

DeltaNetParameters SmallDelta() {
  DeltaNetParameters p;
  p.key_heads = 1;
  p.value_heads = 2;
  p.key_head_dim = 5;
  p.value_head_dim = 7;
  p.conv_kernel_dim = 4;
  return p;
}

void SequenceMatchesOracleAndCachedTokens(DeltaNetParameters p, int length) {
  // sequence_delta_net_test.cc:241-297
  auto executor = NewExecutor();
  const int channels = 2 * p.key_heads * p.key_head_dim + p.value_heads * p.value_head_dim;
  const int width = p.value_heads * p.value_head_dim;
  const auto qkv = RoundedToBFloat16(Values(static_cast<size_t>(length) * channels, .1));
  const auto z = RoundedToBFloat16(Values(static_cast<size_t>(length) * width, 1.1));
  const auto a = RoundedToBFloat16(Values(static_cast<size_t>(length) * p.value_heads, 2.1));
  const auto b = RoundedToBFloat16(Values(static_cast<size_t>(length) * p.value_heads, 3.1));
  const auto conv = Values(static_cast<size_t>(channels) * p.conv_kernel_dim, .3, .5);
  const auto a_log = Values(p.value_heads, .5, .4), dt_bias = Values(p.value_heads, .7, .3);
  auto norm = Values(p.value_head_dim, .9, .2);
  for (float& value : norm) value += 1.0f;
  const pluto_hip_delta_params abi = cached_attention_ops::ToAbi(p);
  pluto_oracle_delta_params oracle_p;
  static_assert(sizeof(oracle_p) == sizeof(abi));
  std::memcpy(&oracle_p, &abi, sizeof(abi));
  std::vector<float> want(static_cast<size_t>(length) * width);
  ASSERT_EQ(pluto_oracle_gdn_sequence(&oracle_p, length, qkv.data(), z.data(), a.data(), b.data(),
                                      conv.data(), a_log.data(), dt_bias.data(), norm.data(),
                                      want.data(), nullptr, nullptr), 0);
  std::shared_ptr<BlockParameter> parameters[4];
  const std::vector<float>* weights[] = {&conv, &a_log, &dt_bias, &norm};
  for (int i = 0; i < 4; ++i) {
    auto parameter = Parameter(*executor, *weights[i]);
    ASSERT_TRUE(parameter.ok());
    parameters[i] = *parameter;
  }
  auto sequence = SequenceDeltaNetLayer::Create(*executor, p, parameters[0], parameters[1],
                                                parameters[2], parameters[3], length);
  ASSERT_TRUE(sequence.ok());
  auto dqkv = Upload<BFloat16>(*executor, qkv), dz = Upload<BFloat16>(*executor, z),
       da = Upload<BFloat16>(*executor, a), db = Upload<BFloat16>(*executor, b);
  std::vector<float> first;
  for (int repetition = 0; repetition < 2; ++repetition) {  // stateless: repeats agree
    auto forward = (*sequence)->fwd(*executor, {*dqkv, *dz, *da, *db});
    ASSERT_TRUE(forward.ok());
    const auto got = Read<BFloat16>(forward->outputs[0]);
    if (repetition == 0) first = got;
    EXPECT_TRUE(got == first);
    // a gradient of the wrong type/size is rejected before any work
    EXPECT_TRUE(IsInvalidArgument(
        (*sequence)->bwd(*executor, {*dz}, std::move(forward->state)).status()));
  }
  double scale = 0;
  for (float value : want) scale = std::max(scale, std::fabs(double(value)));
  for (size_t i = 0; i < want.size(); ++i)
    EXPECT_NEAR(first[i], want[i], 2e-2 * scale);

  auto cached = DeltaNetLayer::Create(*executor, p, parameters[0]->value(), parameters[1]->value(),
                                      parameters[2]->value(), parameters[3]->value());
  ASSERT_TRUE(cached.ok());
  for (int pass = 0; pass < 2; ++pass) {  // Reset starts the same sequence again
    for (int t = 0; t < length; ++t) {
      auto row = [&](const std::vector<float>& all, int columns) {
        return Upload<BFloat16>(*executor, {all.begin() + t * columns, all.begin() + (t + 1) * columns});
      };
      auto q1 = row(qkv, channels), z1 = row(z, width), a1 = row(a, p.value_heads),
           b1 = row(b, p.value_heads);
      auto step = (*cached)->fwd(*executor, {*q1, *z1, *a1, *b1});
      ASSERT_TRUE(step.ok());
      const auto got = Read<BFloat16>(step->outputs[0]);
      for (int c = 0; c < width; ++c)
        EXPECT_NEAR(got[c], want[static_cast<size_t>(t) * width + c], 2e-2 * scale);
    }
    ASSERT_TRUE((*cached)->Reset().ok());
  }
}

void BackwardMatchesOracle(DeltaNetParameters p, int length, bool rounding) {
  // sequence_delta_net_test.cc:299-380: every input and parameter gradient; the
  // oracle's backward is itself pinned by finite differences.
  p.round_to_bfloat16 = rounding;
  auto executor = NewExecutor();
  const int channels = 2 * p.key_heads * p.key_head_dim + p.value_heads * p.value_head_dim;
  const int width = p.value_heads * p.value_head_dim;
  const auto qkv = RoundedToBFloat16(Values(static_cast<size_t>(length) * channels, .1));
  const auto z = RoundedToBFloat16(Values(static_cast<size_t>(length) * width, 1.1));
  const auto a = RoundedToBFloat16(Values(static_cast<size_t>(length) * p.value_heads, 2.1));
  const auto b = RoundedToBFloat16(Values(static_cast<size_t>(length) * p.value_heads, 3.1));
  const auto conv = Values(static_cast<size_t>(channels) * p.conv_kernel_dim, .3, .5);
  const auto a_log = Values(p.value_heads, .5, .4), dt_bias = Values(p.value_heads, .7, .3);
  auto norm = Values(p.value_head_dim, .9, .2);
  for (float& value : norm) value += 1.0f;
  const auto upstream = Values(static_cast<size_t>(length) * width, .7);
  const pluto_hip_delta_params abi = cached_attention_ops::ToAbi(p);
  pluto_oracle_delta_params oracle_p;
  std::memcpy(&oracle_p, &abi, sizeof(abi));
  std::vector<std::vector<float>> want = {
      std::vector<float>(qkv.size()),  std::vector<float>(z.size()),
      std::vector<float>(a.size()),    std::vector<float>(b.size()),
      std::vector<float>(conv.size(), 0.f), std::vector<float>(a_log.size(), 0.f),
      std::vector<float>(dt_bias.size(), 0.f), std::vector<float>(norm.size(), 0.f)};
  ASSERT_EQ(pluto_oracle_gdn_sequence_backward(
                &oracle_p, length, qkv.data(), z.data(), a.data(), b.data(), conv.data(),
                a_log.data(), dt_bias.data(), norm.data(), upstream.data(), want[0].data(),
                want[1].data(), want[2].data(), want[3].data(), want[4].data(), want[5].data(),
                want[6].data(), want[7].data()),
            0);
  std::shared_ptr<BlockParameter> parameters[4];
  const std::vector<float>* weights[] = {&conv, &a_log, &dt_bias, &norm};
  for (int i = 0; i < 4; ++i) {
    auto parameter = Parameter(*executor, *weights[i]);
    ASSERT_TRUE(parameter.ok());
    parameters[i] = *parameter;
    ASSERT_TRUE(parameters[i]->Activate().ok());
  }
  auto layer = SequenceDeltaNetLayer::Create(*executor, p, parameters[0], parameters[1],
                                             parameters[2], parameters[3], length);
  ASSERT_TRUE(layer.ok());
  auto dqkv = Upload<BFloat16>(*executor, qkv), dz = Upload<BFloat16>(*executor, z),
       da = Upload<BFloat16>(*executor, a), db = Upload<BFloat16>(*executor, b);
  auto dy = Upload<float>(*executor, upstream);
  std::vector<std::vector<float>> first;
  for (int call = 0; call < 2; ++call) {
    auto forward = (*layer)->fwd(*executor, {*dqkv, *dz, *da, *db});
    ASSERT_TRUE(forward.ok());
    auto backward = (*layer)->bwd(*executor, {*dy}, std::move(forward->state));
    ASSERT_TRUE(backward.ok());
    ASSERT_EQ(backward->size(), 4u);
    std::vector<std::vector<float>> actual;
    for (const auto& gradient : *backward) actual.push_back(Read<float>(gradient));
    for (int i = 0; i < 4; ++i) actual.push_back(Read<float>(parameters[i]->gradient()));
    if (call == 0) {
      first = actual;
      for (size_t which = 0; which < want.size(); ++which) {
        ASSERT_EQ(actual[which].size(), want[which].size());
        double scale = 0;
        for (float value : want[which]) scale = std::max(scale, std::fabs(double(value)));
        // FP32 token-serial arithmetic against the double-precision oracle; with
        // rounding, operands that straddle a bf16 tie differ by one ulp
        const double bound = (rounding ? 1e-2 : 2e-4) * scale + 1e-6;
        for (size_t i = 0; i < want[which].size(); ++i)
          EXPECT_NEAR(actual[which][i], want[which][i], bound);
      }
    } else {
      // activation gradients repeat bit for bit, parameter gradients accumulate
      for (int which = 0; which < 4; ++which) EXPECT_TRUE(actual[which] == first[which]);
      for (int which = 4; which < 8; ++which)
        for (size_t i = 0; i < actual[which].size(); ++i)
          EXPECT_NEAR(actual[which][i], 2 * first[which][i], 1e-5 * (1 + std::fabs(first[which][i])));
    }
  }
  // frozen parameters: the activation gradients are the same, nothing accumulates
  for (auto& parameter : parameters) ASSERT_TRUE(parameter->Deactivate().ok());
  auto forward = (*layer)->fwd(*executor, {*dqkv, *dz, *da, *db});
  ASSERT_TRUE(forward.ok());
  auto state_copy = forward->state;
  auto backward = (*layer)->bwd(*executor, {*dy}, std::move(forward->state));
  ASSERT_TRUE(backward.ok());
  for (int which = 0; which < 4; ++which)
    EXPECT_TRUE(Read<float>((*backward)[which]) == first[which]);
  state_copy.intermediates.pop_back();
  EXPECT_TRUE(IsInvalidArgument((*layer)->bwd(*executor, {*dy}, std::move(state_copy)).status()));
}

TEST(SequenceDeltaNetTest, BackwardMatchesOracleOnSmallOddShape) {
  for (bool rounding : {false, true}) BackwardMatchesOracle(SmallDelta(), 9, rounding);
}

TEST(SequenceDeltaNetTest, BackwardMatchesOracleOnFullWidthHeads) {
  DeltaNetParameters p;
  p.key_heads = 1;
  p.value_heads = 2;
  p.key_head_dim = 128;
  p.value_head_dim = 128;
  BackwardMatchesOracle(p, 70, true);
}

TEST(SequenceDeltaNetTest, SmallOddShapeMatchesOracleAndCachedTokenInference) {
  SequenceMatchesOracleAndCachedTokens(SmallDelta(), 9);
}

TEST(SequenceDeltaNetTest, ChunkedMatrixCoreScanMatchesOracleAndCachedTokenInference) {
  DeltaNetParameters p;
  p.key_heads = 1;
  p.value_heads = 2;
  p.key_head_dim = 128;
  p.value_head_dim = 128;
  SequenceMatchesOracleAndCachedTokens(p, 150);  // two full 64-token chunks and a ragged tail
}

TEST(SequenceDeltaNetTest, RejectsBadShapesAndPreservesTypedSignatures) {
  // sequence_delta_net_test.cc:406-450
  auto executor = NewExecutor();
  const auto p = SmallDelta();
  const int channels = 2 * 5 + 14;
  auto conv = Parameter(*executor, Values(channels * 4, .3));
  auto a_log = Parameter(*executor, Values(2, .5)), dt_bias = Parameter(*executor, Values(2, .7));
  auto norm = Parameter(*executor, Values(7, .9));
  auto layer = SequenceDeltaNetLayer::Create(*executor, p, *conv, *a_log, *dt_bias, *norm, 3);
  ASSERT_TRUE(layer.ok());
  EXPECT_EQ((*layer)->input_types().size(), 4u);
  EXPECT_EQ((*layer)->input_types()[0], ActivationType(DataType::BF16, {-2, 3, channels}));
  EXPECT_EQ((*layer)->input_types()[3], ActivationType(DataType::BF16, {-2, 3, 2}));
  EXPECT_EQ((*layer)->output_types()[0], ActivationType(DataType::BF16, {-2, 3, 14}));
  EXPECT_EQ((*layer)->weights().size(), 4u);
  EXPECT_TRUE(IsInvalidArgument(
      SequenceDeltaNetLayer::Create(*executor, p, *conv, *a_log, *dt_bias, *norm, 0).status()));
  EXPECT_TRUE(IsInvalidArgument(
      SequenceDeltaNetLayer::Create(*executor, p, *a_log, *a_log, *dt_bias, *norm, 3).status()));
  EXPECT_TRUE(IsInvalidArgument(
      SequenceDeltaNetLayer::Create(*executor, p, nullptr, *a_log, *dt_bias, *norm, 3).status()));
  auto bad = p;
  bad.key_heads = 3;  // value_heads not a multiple
  EXPECT_TRUE(IsInvalidArgument(
      SequenceDeltaNetLayer::Create(*executor, bad, *conv, *a_log, *dt_bias, *norm, 3).status()));
  auto qkv = Upload<BFloat16>(*executor, Values(3 * channels, .1));
  auto z = Upload<BFloat16>(*executor, Values(3 * 14, .1));
  auto ab = Upload<BFloat16>(*executor, Values(3 * 2, .1));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*qkv, *z, *ab}).status()));
  EXPECT_TRUE(IsInvalidArgument((*layer)->fwd(*executor, {*qkv, *ab, *ab, *ab}).status()));
  EXPECT_TRUE((*layer)->fwd(*executor, {*qkv, *z, *ab, *ab}).ok());
  // the cached layer checks weights before allocating state
  EXPECT_TRUE(IsInvalidArgument(DeltaNetLayer::Create(*executor, p, (*a_log)->value(),
                                                      (*a_log)->value(), (*dt_bias)->value(),
                                                      (*norm)->value()).status()));
}

}  // namespace
}  // namespace pluto::llm
