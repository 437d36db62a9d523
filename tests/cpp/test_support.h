// Upload/Read helpers and deterministic inputs shared by the host-API tests.
#pragma once

#include <cmath>
#include <cstdint>
#include <memory>
#include <vector>

#include "oracle/pluto_oracle.h"
#include "pluto_amd/host/executor.h"
#include "pluto_amd/host/layer.h"
#include "tests/cpp/mini_test.h"

namespace pluto::testing {

using BFloat16 = uint16_t;  // raw bits on the host

inline std::unique_ptr<hip::Executor> NewExecutor() {
  auto executor = hip::Executor::Create();
  if (!executor.ok()) {
    std::cout << "executor: " << executor.status() << std::endl;
    std::abort();
  }
  return std::move(*executor);
}

// sin-based values used throughout the reference's tests (e.g.
// qwen_attention_test.cc Values()).
inline std::vector<float> Values(size_t count, double phase, double scale = 1.0) {
  std::vector<float> values(count);
  for (size_t i = 0; i < count; ++i)
    values[i] = static_cast<float>(scale * std::sin(phase + 0.29 * static_cast<double>(i)));
  return values;
}

inline std::vector<float> RoundedToBFloat16(std::vector<float> values) {
  for (float& value : values) value = pluto_oracle_bf16_round(value);
  return values;
}

template <class T>
T FromFloat(float value);
template <>
inline float FromFloat<float>(float value) { return value; }
template <>
inline BFloat16 FromFloat<BFloat16>(float value) { return pluto_oracle_f32_to_bf16(value); }
inline float ToFloat(float value) { return value; }
inline float ToFloat(BFloat16 value) { return pluto_oracle_bf16_to_f32(value); }

// Copies host floats to a new device buffer of element type T and waits.
template <class T>
StatusOr<hip::Buffer> Upload(hip::Executor& executor, const std::vector<float>& values) {
  ASSIGN_OR_RETURN(auto host, hip::PageLockedHostArray<T>::Allocate(executor, values.size()));
  for (size_t i = 0; i < values.size(); ++i) host[i] = FromFloat<T>(values[i]);
  ASSIGN_OR_RETURN(auto device, hip::Buffer::Allocate(executor, values.size() * sizeof(T)));
  if (!values.empty())
    RETURN_IF_ERROR(hip::HipStatus(
        pluto_hip_memcpy_async(executor.stream(), device.data(), host.data(), host.size_bytes(), 1),
        "upload"));
  RETURN_IF_ERROR(executor.Synchronize());
  return device;
}

// Uploads raw elements of type T (bf16 bit patterns, FP8 codes) and waits.
template <class T>
StatusOr<hip::Buffer> UploadRaw(hip::Executor& executor, const std::vector<T>& values) {
  ASSIGN_OR_RETURN(auto host, hip::PageLockedHostArray<T>::Allocate(executor, values.size()));
  for (size_t i = 0; i < values.size(); ++i) host[i] = values[i];
  ASSIGN_OR_RETURN(auto device, hip::Buffer::Allocate(executor, values.size() * sizeof(T)));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_memcpy_async(executor.stream(), device.data(), host.data(), host.size_bytes(), 1),
      "upload"));
  RETURN_IF_ERROR(executor.Synchronize());
  return device;
}

// OCP FP8 E4M3 codes of the values, rounded as the oracle rounds.
inline std::vector<uint8_t> Fp8Codes(const std::vector<float>& values) {
  std::vector<uint8_t> codes(values.size());
  for (size_t i = 0; i < values.size(); ++i) codes[i] = pluto_oracle_f32_to_fp8_e4m3(values[i]);
  return codes;
}

// Reads a device buffer of element type T back as floats.
template <class T>
std::vector<float> Read(const hip::Buffer& buffer) {
  hip::Executor& executor = buffer.executor();
  const size_t count = buffer.size_bytes() / sizeof(T);
  auto host = hip::PageLockedHostArray<T>::Allocate(executor, count);
  std::vector<float> values(count);
  if (!host.ok() || count == 0) return values;
  const int code =
      pluto_hip_memcpy_async(executor.stream(), host->data(), buffer.data(), buffer.size_bytes(), 2);
  if (code != 0 || !executor.Synchronize().ok()) {
    std::cout << "device read failed" << std::endl;
    std::abort();
  }
  for (size_t i = 0; i < count; ++i) values[i] = ToFloat((*host)[i]);
  return values;
}

inline bool Contains(std::string_view text, std::string_view piece) {
  return text.find(piece) != std::string_view::npos;
}

}  // namespace pluto::testing
