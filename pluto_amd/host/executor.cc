#include "pluto_amd/host/executor.h"

#include <cstdio>

namespace pluto::hip {

namespace {
constexpr int kHipErrorOutOfMemory = 2;
}

Status HipStatus(int code, const char* operation) {
  if (code == 0) return OkStatus();
  std::string text = StrCat(operation, " failed: ", pluto_hip_error_name(code), ": ",
                            pluto_hip_error_string(code));
  switch (code) {
    case PLUTO_HIP_EINVAL: return InvalidArgumentError(std::move(text));
    case PLUTO_HIP_ERANGE: return ResourceExhaustedError(std::move(text));
    case PLUTO_HIP_EUNSUPPORTED: return UnimplementedError(std::move(text));
    case PLUTO_HIP_EWORKSPACE: return InternalError(std::move(text));
    case kHipErrorOutOfMemory: return ResourceExhaustedError(std::move(text));
    default: return InternalError(std::move(text));
  }
}

StatusOr<std::unique_ptr<Executor>> Executor::Create() {
  std::unique_ptr<Executor> executor(new Executor());
  RETURN_IF_ERROR(HipStatus(pluto_hip_executor_create(&executor->handle_), "executor creation"));
  return executor;
}

Executor::~Executor() {
  if (handle_ == nullptr) return;
  const int code = pluto_hip_executor_destroy(handle_);
  if (code != 0)
    std::fprintf(stderr, "executor destruction failed: %s: %s\n", pluto_hip_error_name(code),
                 pluto_hip_error_string(code));
}

Status Executor::Synchronize() const {
  return HipStatus(pluto_hip_executor_synchronize(handle_), "stream synchronization");
}

struct Buffer::Allocation {
  Allocation(Executor& executor, size_t size_bytes) : size_bytes(size_bytes), executor(executor) {}
  ~Allocation() {
    if (data == nullptr) return;
    const int code = pluto_hip_free_async(executor.handle(), data);
    if (code != 0)
      std::fprintf(stderr, "stream-ordered free(%p) failed: %s: %s\n", data,
                   pluto_hip_error_name(code), pluto_hip_error_string(code));
  }
  void* data = nullptr;
  size_t size_bytes;
  Executor& executor;
};

StatusOr<Buffer> Buffer::Allocate(Executor& executor, size_t size_bytes) {
  auto allocation = std::make_shared<Allocation>(executor, size_bytes);
  if (size_bytes == 0) return Buffer(std::move(allocation));
  const std::string operation = StrCat("stream-ordered allocation(", size_bytes, ")");
  RETURN_IF_ERROR(HipStatus(pluto_hip_malloc_async(executor.handle(), size_bytes, &allocation->data),
                            operation.c_str()));
  return Buffer(std::move(allocation));
}

void* Buffer::data() const { return allocation_->data; }
size_t Buffer::size_bytes() const { return allocation_->size_bytes; }
Executor& Buffer::executor() const { return allocation_->executor; }

struct PageLockedHostBuffer::Allocation {
  Allocation(Executor& executor, size_t size_bytes) : size_bytes(size_bytes), executor(executor) {}
  ~Allocation() {
    if (data == nullptr) return;
    const int code = pluto_hip_host_free_async(executor.handle(), data);
    if (code != 0)
      std::fprintf(stderr, "pinned host release(%p) failed: %s: %s\n", data,
                   pluto_hip_error_name(code), pluto_hip_error_string(code));
  }
  void* data = nullptr;
  size_t size_bytes;
  Executor& executor;
};

StatusOr<PageLockedHostBuffer> PageLockedHostBuffer::Allocate(Executor& executor,
                                                              size_t size_bytes) {
  auto allocation = std::make_shared<Allocation>(executor, size_bytes);
  if (size_bytes == 0) return PageLockedHostBuffer(std::move(allocation));
  const std::string operation = StrCat("pinned host allocation(", size_bytes, ")");
  RETURN_IF_ERROR(HipStatus(pluto_hip_host_alloc(executor.handle(), size_bytes, &allocation->data),
                            operation.c_str()));
  return PageLockedHostBuffer(std::move(allocation));
}

void* PageLockedHostBuffer::data() { return allocation_ ? allocation_->data : nullptr; }
const void* PageLockedHostBuffer::data() const { return allocation_ ? allocation_->data : nullptr; }
size_t PageLockedHostBuffer::size_bytes() const { return allocation_ ? allocation_->size_bytes : 0; }
Executor& PageLockedHostBuffer::executor() const { return allocation_->executor; }

}  // namespace pluto::hip
