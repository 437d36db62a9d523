// Stream/buffer runtime behind the C ABI: the pieces of the reference's
// src/cuda (executor, device buffer, page-locked host buffer) that the
// attention path needs, written for HIP.
#include <hip/hip_runtime.h>

#include <mutex>
#include <new>
#include <vector>

#include "common.h"

namespace {

struct PinnedBlock {
  void* data;
  size_t bytes;
  hipEvent_t released;  // recorded on the compute stream when handed back
  bool in_use;
};

}  // namespace

// Pinned host memory is served from a per-executor cache of hipHostMalloc
// blocks.  A released block is reused only once the event recorded on the
// compute stream at release time has completed, so handing out memory never
// waits for compute (src/cuda/executor.cc:72-88 states the same policy for
// the reference's host memory pool).
struct pluto_hip_executor {
  int device = 0;
  hipStream_t stream = nullptr;
  hipStream_t immediate_stream = nullptr;
  std::mutex mutex;
  std::vector<PinnedBlock> pinned;
  size_t cached_bytes = 0;
};

namespace {

constexpr size_t kPinnedCacheLimit = 64ull << 20;  // executor.cc:90-95

const char* const kNegativeNames[] = {"PLUTO_HIP_OK", "PLUTO_HIP_EINVAL",
                                      "PLUTO_HIP_ERANGE",
                                      "PLUTO_HIP_EUNSUPPORTED",
                                      "PLUTO_HIP_EWORKSPACE", "PLUTO_HIP_ELIMIT"};
const char* const kNegativeStrings[] = {
    "success", "invalid argument", "capacity exhausted",
    "unsupported configuration", "workspace missing or too small",
    "request larger than the fixed scratch of this entry point"};

}  // namespace

extern "C" {

const char* pluto_hip_error_name(int code) {
  if (code <= 0 && code >= -5) return kNegativeNames[-code];
  if (code > 0) return hipGetErrorName(static_cast<hipError_t>(code));
  return "PLUTO_HIP_EUNKNOWN";
}

const char* pluto_hip_error_string(int code) {
  if (code <= 0 && code >= -5) return kNegativeStrings[-code];
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error code";
}

int pluto_hip_abi_version(void) { return PLUTO_HIP_ABI_VERSION; }
const char* pluto_hip_target_arch(void) { return "gfx950"; }

int pluto_hip_executor_create(pluto_hip_executor** out) {
  if (!out) return PLUTO_HIP_EINVAL;
  *out = nullptr;
  auto* executor = new (std::nothrow) pluto_hip_executor();
  if (!executor) return static_cast<int>(hipErrorOutOfMemory);
  hipError_t error = hipGetDevice(&executor->device);
  if (error == hipSuccess)
    error = hipStreamCreateWithFlags(&executor->stream, hipStreamNonBlocking);
  if (error == hipSuccess)
    error = hipStreamCreateWithFlags(&executor->immediate_stream,
                                     hipStreamNonBlocking);
  if (error != hipSuccess) {
    if (executor->immediate_stream)
      (void)hipStreamDestroy(executor->immediate_stream);
    if (executor->stream) (void)hipStreamDestroy(executor->stream);
    delete executor;
    return static_cast<int>(error);
  }
  *out = executor;
  return 0;
}

int pluto_hip_executor_destroy(pluto_hip_executor* executor) {
  if (!executor) return PLUTO_HIP_EINVAL;
  int first = 0;
  auto note = [&first](hipError_t e) {
    if (e != hipSuccess && first == 0) first = static_cast<int>(e);
  };
  note(hipStreamSynchronize(executor->stream));
  note(hipStreamSynchronize(executor->immediate_stream));
  for (auto& block : executor->pinned) {
    note(hipEventDestroy(block.released));
    note(hipHostFree(block.data));
  }
  note(hipStreamDestroy(executor->immediate_stream));
  note(hipStreamDestroy(executor->stream));
  delete executor;
  return first;
}

int pluto_hip_executor_synchronize(pluto_hip_executor* executor) {
  if (!executor) return PLUTO_HIP_EINVAL;
  return static_cast<int>(hipStreamSynchronize(executor->stream));
}

void* pluto_hip_executor_stream(pluto_hip_executor* executor) {
  return executor ? executor->stream : nullptr;
}

void* pluto_hip_executor_immediate_stream(pluto_hip_executor* executor) {
  return executor ? executor->immediate_stream : nullptr;
}

int pluto_hip_malloc_async(pluto_hip_executor* executor, size_t bytes,
                           void** data) {
  if (!executor || !data) return PLUTO_HIP_EINVAL;
  *data = nullptr;
  if (bytes == 0) return 0;  // buffer.cc:58-61: no storage, still a buffer
  return static_cast<int>(hipMallocAsync(data, bytes, executor->stream));
}

int pluto_hip_free_async(pluto_hip_executor* executor, void* data) {
  if (!executor) return PLUTO_HIP_EINVAL;
  if (!data) return 0;
  return static_cast<int>(hipFreeAsync(data, executor->stream));
}

int pluto_hip_host_alloc(pluto_hip_executor* executor, size_t bytes,
                         void** data) {
  if (!executor || !data) return PLUTO_HIP_EINVAL;
  *data = nullptr;
  if (bytes == 0) return 0;
  {
    std::lock_guard<std::mutex> lock(executor->mutex);
    PinnedBlock* best = nullptr;
    for (auto& block : executor->pinned) {
      if (block.in_use || block.bytes < bytes) continue;
      if (best && best->bytes <= block.bytes) continue;
      // Only blocks whose release point has already passed: never wait.
      if (hipEventQuery(block.released) != hipSuccess) continue;
      best = &block;
    }
    if (best && best->bytes <= 2 * bytes + 4096) {
      best->in_use = true;
      *data = best->data;
      return 0;
    }
  }
  PinnedBlock block{};
  hipError_t error = hipHostMalloc(&block.data, bytes, hipHostMallocDefault);
  if (error != hipSuccess) return static_cast<int>(error);
  error = hipEventCreateWithFlags(&block.released, hipEventDisableTiming);
  if (error != hipSuccess) {
    (void)hipHostFree(block.data);
    return static_cast<int>(error);
  }
  block.bytes = bytes;
  block.in_use = true;
  std::lock_guard<std::mutex> lock(executor->mutex);
  executor->pinned.push_back(block);
  executor->cached_bytes += bytes;
  *data = block.data;
  return 0;
}

int pluto_hip_host_free_async(pluto_hip_executor* executor, void* data) {
  if (!executor) return PLUTO_HIP_EINVAL;
  if (!data) return 0;
  std::lock_guard<std::mutex> lock(executor->mutex);
  for (size_t i = 0; i < executor->pinned.size(); ++i) {
    PinnedBlock& block = executor->pinned[i];
    if (block.data != data || !block.in_use) continue;
    hipError_t error = hipEventRecord(block.released, executor->stream);
    if (error != hipSuccess) return static_cast<int>(error);
    block.in_use = false;
    // Trim: drop completed free blocks while the cache is above its limit.
    if (executor->cached_bytes > kPinnedCacheLimit) {
      for (size_t j = 0; j < executor->pinned.size();) {
        PinnedBlock& candidate = executor->pinned[j];
        if (executor->cached_bytes > kPinnedCacheLimit && !candidate.in_use &&
            hipEventQuery(candidate.released) == hipSuccess) {
          (void)hipEventDestroy(candidate.released);
          (void)hipHostFree(candidate.data);
          executor->cached_bytes -= candidate.bytes;
          executor->pinned[j] = executor->pinned.back();
          executor->pinned.pop_back();
        } else {
          ++j;
        }
      }
    }
    return 0;
  }
  return PLUTO_HIP_EINVAL;
}

int pluto_hip_memcpy_async(void* stream, void* dst, const void* src,
                           size_t bytes, int kind) {
  if (bytes == 0) return 0;
  if (!dst || !src) return PLUTO_HIP_EINVAL;
  hipMemcpyKind k;
  switch (kind) {
    case 1: k = hipMemcpyHostToDevice; break;
    case 2: k = hipMemcpyDeviceToHost; break;
    case 3: k = hipMemcpyDeviceToDevice; break;
    default: return PLUTO_HIP_EINVAL;
  }
  return static_cast<int>(
      hipMemcpyAsync(dst, src, bytes, k, static_cast<hipStream_t>(stream)));
}

int pluto_hip_memset_async(void* stream, void* dst, int value, size_t bytes) {
  if (bytes == 0) return 0;
  if (!dst) return PLUTO_HIP_EINVAL;
  return static_cast<int>(
      hipMemsetAsync(dst, value, bytes, static_cast<hipStream_t>(stream)));
}

int pluto_hip_stream_synchronize(void* stream) {
  return static_cast<int>(
      hipStreamSynchronize(static_cast<hipStream_t>(stream)));
}

}  // extern "C"

namespace {

using namespace pluto_hip;

// 256 threads, 8 elements each; grid-stride for large tensors.
__global__ void __launch_bounds__(256)
cast_bf16_to_f32_kernel(const uint16_t* __restrict__ src,
                        float* __restrict__ dst, size_t count) {
  size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x);
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  for (; i < count; i += stride) dst[i] = bf16_bits_to_float(src[i]);
}

__global__ void __launch_bounds__(256)
cast_f32_to_bf16_kernel(const float* __restrict__ src,
                        uint16_t* __restrict__ dst, size_t count) {
  size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x);
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  for (; i < count; i += stride) dst[i] = float_to_bf16_bits(src[i]);
}

int cast_grid(size_t count) {
  size_t blocks = (count + 255) / 256;
  return static_cast<int>(blocks > 65536 ? 65536 : blocks);
}

}  // namespace

extern "C" {

int pluto_hip_cast_bf16_to_f32(void* stream, const void* src, float* dst,
                               size_t count) {
  if (count == 0) return 0;
  if (!src || !dst) return PLUTO_HIP_EINVAL;
  cast_bf16_to_f32_kernel<<<cast_grid(count), 256, 0,
                            static_cast<hipStream_t>(stream)>>>(
      static_cast<const uint16_t*>(src), dst, count);
  return launch_status();
}

int pluto_hip_cast_f32_to_bf16(void* stream, const float* src, void* dst,
                               size_t count) {
  if (count == 0) return 0;
  if (!src || !dst) return PLUTO_HIP_EINVAL;
  cast_f32_to_bf16_kernel<<<cast_grid(count), 256, 0,
                            static_cast<hipStream_t>(stream)>>>(
      src, static_cast<uint16_t*>(dst), count);
  return launch_status();
}

}  // extern "C"
