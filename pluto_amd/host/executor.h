// Stream owner for the attention path on HIP: the role of cuda::Executor
// (src/cuda/executor.h:16-59), implemented over the C ABI of pluto_hip.h.
#pragma once

#include <memory>

#include "pluto_amd/host/status.h"
#include "pluto_hip.h"

namespace pluto::hip {

// Converts a pluto_hip_* return value: 0 -> OK, HIP runtime errors -> Internal
// "<operation> failed: <name>: <text>" (src/cuda/executor.cc:15-21), out of
// memory -> ResourceExhausted (src/cuda/buffer.cc:16-23), library argument
// codes -> their canonical status codes.
Status HipStatus(int code, const char* operation);

// One non-blocking compute stream, one non-blocking immediate stream and a
// cache of pinned host blocks.  Must outlive every buffer created on it.
// Calls on one executor must be serialised by the caller.
class Executor final {
 public:
  static StatusOr<std::unique_ptr<Executor>> Create();
  Executor(const Executor&) = delete;
  Executor& operator=(const Executor&) = delete;
  ~Executor();

  // Waits for the compute stream only.
  Status Synchronize() const;
  void* stream() const { return pluto_hip_executor_stream(handle_); }
  void* immediate_stream() const { return pluto_hip_executor_immediate_stream(handle_); }
  pluto_hip_executor* handle() const { return handle_; }

 private:
  Executor() = default;
  pluto_hip_executor* handle_ = nullptr;
};

// Stream-ordered device allocation shared by copyable handles; the last copy
// queues the free on the owning executor's compute stream
// (cuda::Buffer, src/cuda/buffer.h:19-40).  A zero-byte buffer has a null
// data() but still names its executor.
class Buffer final {
 public:
  static StatusOr<Buffer> Allocate(Executor& executor, size_t size_bytes);
  void* data() const;
  size_t size_bytes() const;
  Executor& executor() const;

 private:
  struct Allocation;
  explicit Buffer(std::shared_ptr<Allocation> allocation) : allocation_(std::move(allocation)) {}
  std::shared_ptr<Allocation> allocation_;
};

// Pinned host storage, usable by the CPU as soon as Allocate returns; the
// release is ordered after the compute-stream work queued so far
// (cuda::PageLockedHostBuffer, src/cuda/page_locked_host_buffer.h).
class PageLockedHostBuffer final {
 public:
  PageLockedHostBuffer() = default;
  static StatusOr<PageLockedHostBuffer> Allocate(Executor& executor, size_t size_bytes);
  void* data();
  const void* data() const;
  size_t size_bytes() const;
  Executor& executor() const;

 private:
  struct Allocation;
  explicit PageLockedHostBuffer(std::shared_ptr<Allocation> allocation)
      : allocation_(std::move(allocation)) {}
  std::shared_ptr<Allocation> allocation_;
};

// Typed view over a PageLockedHostBuffer
// (cuda::PageLockedHostArray, src/cuda/page_locked_host_array.h).
template <class T>
class PageLockedHostArray final {
 public:
  static_assert(std::is_trivially_copyable_v<T>);
  PageLockedHostArray() = default;
  static StatusOr<PageLockedHostArray> Allocate(Executor& executor, size_t size) {
    if (size > static_cast<size_t>(-1) / sizeof(T))
      return InvalidArgumentError("page-locked host array byte size overflows size_t");
    ASSIGN_OR_RETURN(auto buffer, PageLockedHostBuffer::Allocate(executor, size * sizeof(T)));
    return PageLockedHostArray(std::move(buffer), size);
  }
  static StatusOr<PageLockedHostArray> CopyFrom(Executor& executor, Span<const T> values) {
    ASSIGN_OR_RETURN(auto result, Allocate(executor, values.size()));
    for (size_t i = 0; i < values.size(); ++i) result[i] = values[i];
    return result;
  }
  T* data() { return static_cast<T*>(buffer_.data()); }
  const T* data() const { return static_cast<const T*>(buffer_.data()); }
  size_t size() const { return size_; }
  size_t size_bytes() const { return buffer_.size_bytes(); }
  T& operator[](size_t i) { return data()[i]; }
  const T& operator[](size_t i) const { return data()[i]; }
  T* begin() { return data(); }
  T* end() { return data() + size_; }
  const T* begin() const { return data(); }
  const T* end() const { return data() + size_; }
  Executor& executor() const { return buffer_.executor(); }

 private:
  PageLockedHostArray(PageLockedHostBuffer buffer, size_t size)
      : buffer_(std::move(buffer)), size_(size) {}
  PageLockedHostBuffer buffer_;
  size_t size_ = 0;
};

}  // namespace pluto::hip
