// Resident weight handle of src/llm/block_parameter.h: a stable resident value
// plus, while the parameter is the one being optimised, FP32 master and
// gradient buffers.  The attention path reads value(), storage(), elements()
// and active(), and accumulates norm-weight gradients into gradient().
#pragma once

#include <memory>
#include <optional>

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

  // block_parameter.cc:39-64.  All work is ordered on value's executor.
  // Idempotent; the first activation zeros the gradient.
  Status Activate() {
    if (active()) return OkStatus();
    hip::Executor& executor = value_.executor();
    ASSIGN_OR_RETURN(auto master, Buffer::Allocate(executor, elements_ * 4));
    ASSIGN_OR_RETURN(auto gradient, Buffer::Allocate(executor, elements_ * 4));
    if (storage_ == DataType::BF16) {
      RETURN_IF_ERROR(hip::HipStatus(
          pluto_hip_cast_bf16_to_f32(executor.stream(), value_.data(),
                                     static_cast<float*>(master.data()), elements_),
          "activate block weight"));
    } else {
      RETURN_IF_ERROR(hip::HipStatus(
          pluto_hip_memcpy_async(executor.stream(), master.data(), value_.data(),
                                 value_.size_bytes(), 3),
          "activate FP32 block weight"));
    }
    RETURN_IF_ERROR(hip::HipStatus(
        pluto_hip_memset_async(executor.stream(), gradient.data(), 0, gradient.size_bytes()),
        "zero block gradient"));
    master_ = std::move(master);
    gradient_ = std::move(gradient);
    return OkStatus();
  }

  // block_parameter.cc:66-81: the resident allocation keeps its address.
  Status Publish() {
    if (!active()) return OkStatus();
    hip::Executor& executor = value_.executor();
    if (storage_ == DataType::BF16)
      return hip::HipStatus(
          pluto_hip_cast_f32_to_bf16(executor.stream(), static_cast<const float*>(master_->data()),
                                     value_.data(), elements_),
          "publish block weight");
    return hip::HipStatus(pluto_hip_memcpy_async(executor.stream(), value_.data(), master_->data(),
                                                 value_.size_bytes(), 3),
                          "publish FP32 block weight");
  }

  // block_parameter.cc:83-87: releases the FP32 working set, launches nothing.
  Status Deactivate() {
    master_.reset();
    gradient_.reset();
    return OkStatus();
  }

  bool active() const { return master_.has_value(); }
  const Buffer& value() const { return value_; }
  // These accessors require active(); inactive parameters own neither buffer.
  const Buffer& master() const { return master_.value(); }
  const Buffer& gradient() const { return gradient_.value(); }
  size_t elements() const { return elements_; }
  DataType storage() const { return storage_; }

 private:
  BlockParameter(Buffer value, DataType storage, size_t elements)
      : value_(std::move(value)), storage_(storage), elements_(elements) {}
  Buffer value_;
  DataType storage_;
  size_t elements_;
  std::optional<Buffer> master_;
  std::optional<Buffer> gradient_;
};

}  // namespace pluto::llm
