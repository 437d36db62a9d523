// Buffer/shape validators and cast helpers shared by the attention layers:
// the subset of src/llm/layers/util.h:15-173 the path calls.
#pragma once

#include <limits>

#include "pluto_amd/host/layer.h"

namespace pluto::llm::internal {

inline size_t ActivationElementBytes(DataType data_type) {
  return data_type == DataType::BF16 ? 2 : sizeof(float);
}

inline Status ValidateComputeType(DataType data_type) {
  if (data_type == DataType::FP16 || data_type == DataType::BF16) return OkStatus();
  if (data_type != DataType::FP8)
    return UnimplementedError("this backend supports only FP16 and BF16 compute policies");
  return UnimplementedError(
      "FP8 requires an explicit scaling policy; this backend implements FP16 and BF16 "
      "compute with FP32 master weights");
}

inline Status ValidateExecutor(hip::Executor& expected, hip::Executor& actual, const char* name) {
  if (&actual != &expected)
    return InvalidArgumentError(StrCat(name, " was created for a different Executor"));
  return OkStatus();
}

inline StatusOr<int> RowsOf(hip::Executor& executor, const Buffer& buffer, int columns,
                            size_t element_bytes, const char* name, const char* kind) {
  if (&buffer.executor() != &executor)
    return InvalidArgumentError(StrCat(name, " belongs to a different Executor"));
  const size_t row_bytes = static_cast<size_t>(columns) * element_bytes;
  if (columns <= 0 || buffer.size_bytes() == 0 || buffer.size_bytes() % row_bytes != 0)
    return InvalidArgumentError(
        StrCat(name, " is not a non-empty ", kind, " matrix with ", columns, " columns"));
  const size_t rows = buffer.size_bytes() / row_bytes;
  if (rows > static_cast<size_t>(std::numeric_limits<int>::max()))
    return InvalidArgumentError(StrCat(name, " has too many rows"));
  return static_cast<int>(rows);
}

inline StatusOr<int> MatrixRows(hip::Executor& executor, const Buffer& buffer, int columns,
                                const char* name) {
  return RowsOf(executor, buffer, columns, sizeof(float), name, "float");
}

inline StatusOr<int> ActivationRows(hip::Executor& executor, const Buffer& buffer, int columns,
                                    DataType data_type, const char* name) {
  return RowsOf(executor, buffer, columns, ActivationElementBytes(data_type), name, "activation");
}

inline Status ValidateBuffer(hip::Executor& executor, const Buffer& buffer, size_t expected_bytes,
                             const char* name) {
  if (buffer.size_bytes() != expected_bytes)
    return InvalidArgumentError(
        StrCat(name, " has ", buffer.size_bytes(), " bytes; expected ", expected_bytes));
  if (&buffer.executor() != &executor)
    return InvalidArgumentError(StrCat(name, " belongs to a different Executor"));
  return OkStatus();
}

// Each input must be a bf16 buffer of exactly element_counts[i] elements on
// `executor` (ValidateBFloat16Inputs, src/llm/layers/util.h:26-28).
inline Status ValidateBFloat16Inputs(hip::Executor& executor, Span<const Buffer> inputs,
                                     Span<const int> element_counts) {
  if (inputs.size() != element_counts.size())
    return InvalidArgumentError(StrCat("layer expects ", element_counts.size(), " inputs; got ",
                                       inputs.size()));
  for (size_t i = 0; i < inputs.size(); ++i)
    RETURN_IF_ERROR(ValidateBuffer(executor, inputs[i],
                                   static_cast<size_t>(element_counts[i]) * 2, "bf16 layer input"));
  return OkStatus();
}

inline StatusOr<Buffer> AllocateFloatVector(hip::Executor& executor, int elements) {
  return Buffer::Allocate(executor, static_cast<size_t>(elements) * sizeof(float));
}

// CastKernel, src/llm/layers/util.cc:14-40.
inline StatusOr<Buffer> ToFloat(hip::Executor& executor, const Buffer& input, int elements) {
  ASSIGN_OR_RETURN(auto output, AllocateFloatVector(executor, elements));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_cast_bf16_to_f32(executor.stream(), input.data(),
                                 static_cast<float*>(output.data()), elements),
      "bf16 to fp32 cast"));
  return output;
}

inline StatusOr<Buffer> ToBFloat16(hip::Executor& executor, const Buffer& input, int elements) {
  ASSIGN_OR_RETURN(auto output, Buffer::Allocate(executor, static_cast<size_t>(elements) * 2));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_cast_f32_to_bf16(executor.stream(), static_cast<const float*>(input.data()),
                                 output.data(), elements),
      "fp32 to bf16 cast"));
  return output;
}

}  // namespace pluto::llm::internal
