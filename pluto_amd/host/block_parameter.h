// Resident weight handle of src/llm/block_parameter.h.  The attention path
// only reads value(), storage(), elements() and active(); the FP32
// master/gradient copies of block-coordinate training belong to the optimizer,
// which is outside this path, so Activate() reports Unimplemented and
// active() is always false.
#pragma once

#include <memory>

#include "pluto_amd/host/layer.h"

namespace pluto::llm {

class BlockParameter final {
 public:
  static StatusOr<std::shared_ptr<BlockParameter>> Create(hip::Executor& executor, Buffer value,
                                                         DataType storage) {
    if (&value.executor() != &executor)
      return InvalidArgumentError("block parameter belongs to a different Executor");
    const size_t element = storage == DataType::FP32 ? 4 : storage == DataType::BF16 ? 2 : 0;
    if (element == 0) return InvalidArgumentError("block parameters are stored as FP32 or BF16");
    if (value.size_bytes() == 0 || value.size_bytes() % element != 0)
      return InvalidArgumentError("block parameter has an invalid byte size");
    const size_t elements = value.size_bytes() / element;
    return std::shared_ptr<BlockParameter>(new BlockParameter(std::move(value), storage, elements));
  }
  Status Activate() {
    return UnimplementedError("block-coordinate training state is outside the attention path");
  }
  bool active() const { return false; }
  const Buffer& value() const { return value_; }
  size_t elements() const { return elements_; }
  DataType storage() const { return storage_; }

 private:
  BlockParameter(Buffer value, DataType storage, size_t elements)
      : value_(std::move(value)), storage_(storage), elements_(elements) {}
  Buffer value_;
  DataType storage_;
  size_t elements_;
};

}  // namespace pluto::llm
