// Storage and position bookkeeping of one sequence's causal attention cache:
// KeyValueCache of src/llm/key_value_cache.h:25-57.  Position is the next row
// to write (= the valid prefix length).  Reset() does not clear storage.
#pragma once

#include <memory>

#include "pluto_amd/host/executor.h"
#include "pluto_hip.h"

namespace pluto::llm {

class KeyValueCache final {
 public:
  // kFloat32TokenMajor is the reference's layout, FP32 [capacity, kv_heads,
  // head_dim]; kBFloat16HeadMajor is the layout the MI355X decode kernel
  // streams, bf16 [kv_heads, capacity, head_dim] (lossless while the attention
  // parameters round to bf16).
  enum class Storage { kFloat32TokenMajor, kBFloat16HeadMajor };

  static StatusOr<std::unique_ptr<KeyValueCache>> Create(
      hip::Executor& executor, int capacity, int key_value_heads, int head_dim,
      Storage storage = Storage::kFloat32TokenMajor);
  KeyValueCache(const KeyValueCache&) = delete;
  KeyValueCache& operator=(const KeyValueCache&) = delete;

  const hip::Buffer& keys() const { return keys_; }
  const hip::Buffer& values() const { return values_; }
  hip::Executor& executor() const { return keys_.executor(); }
  int capacity() const { return capacity_; }
  int key_value_heads() const { return key_value_heads_; }
  int head_dim() const { return head_dim_; }
  int position() const { return position_; }
  Storage storage() const { return storage_; }
  // The addressing the C ABI needs for this cache.
  pluto_hip_kv_cache_view view() const;

  // A full cache returns ResourceExhausted and keeps its position.
  Status Advance();
  void Reset() { position_ = 0; }

 private:
  KeyValueCache(int capacity, int key_value_heads, int head_dim, Storage storage,
                hip::Buffer keys, hip::Buffer values)
      : capacity_(capacity), key_value_heads_(key_value_heads), head_dim_(head_dim),
        storage_(storage), keys_(std::move(keys)), values_(std::move(values)) {}
  int capacity_, key_value_heads_, head_dim_;
  Storage storage_;
  hip::Buffer keys_, values_;
  int position_ = 0;
};

}  // namespace pluto::llm
