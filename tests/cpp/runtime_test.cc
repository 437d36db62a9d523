// Status/Span/ActivationType (CPU) and executor, buffer, pinned memory and KV
// cache contracts (GPU); cases follow src/llm/activation_type_test.cc,
// src/cuda/{executor,buffer,page_locked_host_buffer}_test.cc and
// src/llm/key_value_cache_test.cc.
#include <limits>

#include "pluto_amd/host/key_value_cache.h"
#include "tests/cpp/test_support.h"

namespace pluto {
namespace {

using llm::ActivationType;
using llm::DataType;
using llm::KeyValueCache;
using testing::NewExecutor;

Status FailsThenPropagates(int* reached) {
  RETURN_IF_ERROR(InvalidArgumentError("first"));
  ++*reached;
  return OkStatus();
}

StatusOr<int> Doubles(StatusOr<int> input) {
  ASSIGN_OR_RETURN(int value, std::move(input));
  return 2 * value;
}

TEST(StatusCpu, MacrosPropagateErrorsAndValues) {
  int reached = 0;
  const Status status = FailsThenPropagates(&reached);
  EXPECT_TRUE(IsInvalidArgument(status));
  EXPECT_EQ(status.message(), "first");
  EXPECT_EQ(reached, 0);
  EXPECT_EQ(*Doubles(21), 42);
  EXPECT_TRUE(IsResourceExhausted(Doubles(ResourceExhaustedError("full")).status()));
  EXPECT_EQ(Status().ToString(), "OK");
  EXPECT_EQ(UnimplementedError("x").ToString(), "UNIMPLEMENTED: x");
  EXPECT_EQ(StrCat("a", 3, "b", size_t{4}), "a3b4");
}

TEST(StatusCpu, SpanViewsVectorsArraysAndLists) {
  std::vector<int> values = {1, 2, 3};
  Span<int> writable(values);
  writable[1] = 5;
  Span<const int> readable = writable;
  EXPECT_EQ(readable.size(), 3u);
  EXPECT_EQ(readable[1], 5);
  const int array[] = {7, 8};
  EXPECT_EQ(Span<const int>(array).size(), 2u);
  EXPECT_TRUE(Span<const int>().empty());
}

TEST(ActivationTypeCpu, BatchMatchesOnlyTheSameBatchSymbol) {
  const ActivationType batch(DataType::FP32, {ActivationType::kBatchDimension, 4});
  EXPECT_EQ(batch, ActivationType(DataType::FP32, {ActivationType::kBatchDimension, 4}));
  EXPECT_NE(batch, ActivationType(DataType::FP32, {1, 4}));
  EXPECT_NE(batch, ActivationType(DataType::FP32, {2, 4}));
}

TEST(ActivationTypeCpu, EqualityIncludesDataTypeRankAndEveryExtent) {
  const ActivationType base(DataType::BF16, {2, 3, 4});
  EXPECT_EQ(base, ActivationType(DataType::BF16, {2, 3, 4}));
  EXPECT_NE(base, ActivationType(DataType::FP32, {2, 3, 4}));
  EXPECT_NE(base, ActivationType(DataType::BF16, {2, 3}));
  EXPECT_NE(base, ActivationType(DataType::BF16, {2, 3, 5}));
  EXPECT_NE(base, ActivationType(DataType::BF16, {6, 4}));      // no flattening
  EXPECT_NE(base, ActivationType(DataType::BF16, {1, 2, 3, 4}));  // no broadcasting
}

TEST(ActivationTypeCpu, RejectsNonpositiveDimensionsOtherThanLeadingBatch) {
  EXPECT_TRUE(ActivationType(DataType::FP32, {}).Validate().ok());
  EXPECT_TRUE(ActivationType(DataType::FP32, {ActivationType::kBatchDimension, 3}).Validate().ok());
  EXPECT_TRUE(IsInvalidArgument(ActivationType(DataType::FP32, {0}).Validate()));
  EXPECT_TRUE(IsInvalidArgument(ActivationType(DataType::FP32, {-1, 3}).Validate()));
  EXPECT_TRUE(IsInvalidArgument(
      ActivationType(DataType::FP32, {3, ActivationType::kBatchDimension}).Validate()));
}

TEST(ActivationTypeCpu, LegacyComputePolicyDoesNotMislabelPhysicalStorage) {
  EXPECT_TRUE(llm::ActivationDataType(DataType::FP16) == DataType::FP32);
  EXPECT_TRUE(llm::ActivationDataType(DataType::BF16) == DataType::BF16);
}

TEST(ExecutorTest, ConvertsRuntimeErrorsToStatus) {
  EXPECT_TRUE(hip::HipStatus(0, "nothing").ok());
  const Status invalid = hip::HipStatus(1, "probe");  // hipErrorInvalidValue
  EXPECT_TRUE(invalid.code() == StatusCode::kInternal);
  EXPECT_TRUE(testing::Contains(invalid.message(), "probe failed: "));
  EXPECT_TRUE(IsResourceExhausted(hip::HipStatus(2, "allocation")));  // out of memory
  EXPECT_TRUE(IsInvalidArgument(hip::HipStatus(PLUTO_HIP_EINVAL, "argument")));
  EXPECT_TRUE(IsResourceExhausted(hip::HipStatus(PLUTO_HIP_ERANGE, "capacity")));
  EXPECT_TRUE(IsUnimplemented(hip::HipStatus(PLUTO_HIP_EUNSUPPORTED, "shape")));
}

TEST(ExecutorTest, OwnsTwoIndependentStreamsAndSynchronizes) {
  auto executor = NewExecutor();
  EXPECT_NE(executor->stream(), nullptr);
  EXPECT_NE(executor->immediate_stream(), nullptr);
  EXPECT_NE(executor->stream(), executor->immediate_stream());
  EXPECT_TRUE(executor->Synchronize().ok());
}

TEST(BufferTest, CopiesShareStorageUntilTheLastReferenceIsDestroyed) {
  auto executor = NewExecutor();
  auto original = hip::Buffer::Allocate(*executor, 64);
  ASSERT_TRUE(original.ok());
  void* address = original->data();
  EXPECT_NE(address, nullptr);
  EXPECT_EQ(original->size_bytes(), 64u);
  EXPECT_EQ(&original->executor(), executor.get());
  {
    hip::Buffer copy = *original;
    EXPECT_EQ(copy.data(), address);
    std::vector<hip::Buffer> more(3, copy);
    EXPECT_EQ(more[2].data(), address);
  }
  // the surviving handle still names live storage: a round trip works
  auto host = hip::PageLockedHostArray<int>::Allocate(*executor, 16);
  ASSERT_TRUE(host.ok());
  for (int i = 0; i < 16; ++i) (*host)[i] = i * i;
  EXPECT_EQ(pluto_hip_memcpy_async(executor->stream(), address, host->data(), 64, 1), 0);
  auto back = hip::PageLockedHostArray<int>::Allocate(*executor, 16);
  ASSERT_TRUE(back.ok());
  EXPECT_EQ(pluto_hip_memcpy_async(executor->stream(), back->data(), address, 64, 2), 0);
  EXPECT_TRUE(executor->Synchronize().ok());
  for (int i = 0; i < 16; ++i) EXPECT_EQ((*back)[i], i * i);
}

TEST(BufferTest, ZeroByteBufferRetainsItsExecutorWithoutAllocatingStorage) {
  auto executor = NewExecutor();
  auto empty = hip::Buffer::Allocate(*executor, 0);
  ASSERT_TRUE(empty.ok());
  EXPECT_EQ(empty->data(), nullptr);
  EXPECT_EQ(empty->size_bytes(), 0u);
  EXPECT_EQ(&empty->executor(), executor.get());
}

TEST(PageLockedHostArrayTest, TypedPinnedStorageIsImmediatelyCpuAccessible) {
  auto executor = NewExecutor();
  const std::vector<float> values = {1.5f, -2.f, 3.25f};
  auto array = hip::PageLockedHostArray<float>::CopyFrom(*executor, MakeConstSpan(values));
  ASSERT_TRUE(array.ok());
  EXPECT_EQ(array->size(), 3u);
  EXPECT_EQ(array->size_bytes(), 12u);
  EXPECT_EQ((*array)[2], 3.25f);
  hip::PageLockedHostArray<float> defaulted;
  EXPECT_EQ(defaulted.size(), 0u);
  EXPECT_EQ(defaulted.data(), nullptr);
  auto empty = hip::PageLockedHostArray<float>::Allocate(*executor, 0);
  ASSERT_TRUE(empty.ok());
  EXPECT_EQ(empty->data(), nullptr);
  EXPECT_EQ(&empty->executor(), executor.get());
  EXPECT_TRUE(IsInvalidArgument(
      hip::PageLockedHostArray<double>::Allocate(*executor, std::numeric_limits<size_t>::max() / 4)
          .status()));
}

TEST(PageLockedHostArrayTest, PendingUploadsOutliveTheirLastHostOwner) {
  // page_locked_host_buffer_test.cc:187-224: releasing the host array right
  // after queueing the copy must not corrupt the upload.
  auto executor = NewExecutor();
  constexpr size_t kCount = 1 << 20;
  auto device = hip::Buffer::Allocate(*executor, kCount * sizeof(int));
  ASSERT_TRUE(device.ok());
  for (int round = 0; round < 3; ++round) {
    auto host = hip::PageLockedHostArray<int>::Allocate(*executor, kCount);
    ASSERT_TRUE(host.ok());
    for (size_t i = 0; i < kCount; ++i) (*host)[i] = static_cast<int>(i) + round;
    EXPECT_EQ(pluto_hip_memcpy_async(executor->stream(), device->data(), host->data(),
                                     host->size_bytes(), 1), 0);
  }
  auto back = hip::PageLockedHostArray<int>::Allocate(*executor, kCount);
  ASSERT_TRUE(back.ok());
  EXPECT_EQ(pluto_hip_memcpy_async(executor->stream(), back->data(), device->data(),
                                   back->size_bytes(), 2), 0);
  EXPECT_TRUE(executor->Synchronize().ok());
  size_t wrong = 0;
  for (size_t i = 0; i < kCount; ++i) wrong += (*back)[i] != static_cast<int>(i) + 2;
  EXPECT_EQ(wrong, 0u);
}

TEST(KeyValueCacheTest, OwnsSeparateBuffersWithRequestedShapeAndExecutor) {
  auto executor = NewExecutor();
  auto cache = KeyValueCache::Create(*executor, 5, 2, 8);
  ASSERT_TRUE(cache.ok());
  EXPECT_EQ((*cache)->capacity(), 5);
  EXPECT_EQ((*cache)->key_value_heads(), 2);
  EXPECT_EQ((*cache)->head_dim(), 8);
  EXPECT_EQ((*cache)->position(), 0);
  EXPECT_EQ((*cache)->keys().size_bytes(), 5u * 2 * 8 * sizeof(float));
  EXPECT_EQ((*cache)->values().size_bytes(), 5u * 2 * 8 * sizeof(float));
  EXPECT_NE((*cache)->keys().data(), (*cache)->values().data());
  EXPECT_EQ(&(*cache)->executor(), executor.get());
  auto native = KeyValueCache::Create(*executor, 5, 2, 8, KeyValueCache::Storage::kBFloat16HeadMajor);
  ASSERT_TRUE(native.ok());
  EXPECT_EQ((*native)->keys().size_bytes(), 5u * 2 * 8 * 2);
  const pluto_hip_kv_cache_view view = (*native)->view();
  EXPECT_EQ(view.dtype, PLUTO_HIP_BF16);
  EXPECT_EQ(view.token_stride, 8);
  EXPECT_EQ(view.head_stride, 40);
}

TEST(KeyValueCacheTest, AdvancesUpToCapacityAndCanStartAnotherSequence) {
  auto executor = NewExecutor();
  auto cache = KeyValueCache::Create(*executor, 2, 1, 4);
  ASSERT_TRUE(cache.ok());
  EXPECT_TRUE((*cache)->Advance().ok());
  EXPECT_TRUE((*cache)->Advance().ok());
  EXPECT_TRUE(IsResourceExhausted((*cache)->Advance()));
  EXPECT_EQ((*cache)->position(), 2);
  void* keys = (*cache)->keys().data();
  (*cache)->Reset();
  EXPECT_EQ((*cache)->position(), 0);
  EXPECT_EQ((*cache)->keys().data(), keys);
  EXPECT_TRUE((*cache)->Advance().ok());
}

TEST(KeyValueCacheTest, RejectsNonpositiveDimensionsAndByteSizeOverflowBeforeAllocation) {
  auto executor = NewExecutor();
  const int invalid[][3] = {{0, 1, 1}, {1, 0, 1}, {1, 1, 0}, {-1, 1, 1}};
  for (const auto& shape : invalid)
    EXPECT_TRUE(IsInvalidArgument(
        KeyValueCache::Create(*executor, shape[0], shape[1], shape[2]).status()));
  const int huge = std::numeric_limits<int>::max();
  EXPECT_TRUE(IsInvalidArgument(KeyValueCache::Create(*executor, huge, huge, huge).status()));
}

}  // namespace
}  // namespace pluto
