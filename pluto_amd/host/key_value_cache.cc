#include "pluto_amd/host/key_value_cache.h"

#include <limits>

namespace pluto::llm {

// src/llm/key_value_cache.cc:20-46
StatusOr<std::unique_ptr<KeyValueCache>> KeyValueCache::Create(hip::Executor& executor,
                                                               int capacity, int key_value_heads,
                                                               int head_dim, Storage storage) {
  if (capacity <= 0 || key_value_heads <= 0 || head_dim <= 0)
    return InvalidArgumentError("KV cache dimensions must be positive");
  size_t bytes = storage == Storage::kFloat32TokenMajor ? sizeof(float) : 2;
  for (int dimension : {capacity, key_value_heads, head_dim}) {
    if (static_cast<size_t>(dimension) > std::numeric_limits<size_t>::max() / bytes)
      return InvalidArgumentError("KV cache byte size overflows size_t");
    bytes *= static_cast<size_t>(dimension);
  }
  ASSIGN_OR_RETURN(auto keys, hip::Buffer::Allocate(executor, bytes));
  ASSIGN_OR_RETURN(auto values, hip::Buffer::Allocate(executor, bytes));
  return std::unique_ptr<KeyValueCache>(new KeyValueCache(
      capacity, key_value_heads, head_dim, storage, std::move(keys), std::move(values)));
}

Status KeyValueCache::Advance() {
  if (position_ == capacity_) return ResourceExhaustedError("KV cache is full");
  ++position_;
  return OkStatus();
}

pluto_hip_kv_cache_view KeyValueCache::view() const {
  pluto_hip_kv_cache_view v{};
  v.keys = keys_.data();
  v.values = values_.data();
  if (storage_ == Storage::kFloat32TokenMajor) {
    v.dtype = PLUTO_HIP_F32;
    v.token_stride = 1LL * key_value_heads_ * head_dim_;
    v.head_stride = head_dim_;
  } else {
    v.dtype = PLUTO_HIP_BF16;
    v.token_stride = head_dim_;
    v.head_stride = 1LL * capacity_ * head_dim_;
  }
  return v;
}

}  // namespace pluto::llm
