#include "pluto_amd/host/fully_connected.h"

#include <algorithm>
#include <random>

#include "pluto_amd/host/layer_util.h"

namespace pluto::llm {
namespace {

int StorageCode(DataType type) { return type == DataType::BF16 ? PLUTO_HIP_BF16 : PLUTO_HIP_F32; }

// src/llm/layers/util.h:66-71
Status ValidatePositiveExtent(int extent, const char* name) {
  if (extent <= 0) return InvalidArgumentError(StrCat(name, " must be positive; got ", extent));
  return OkStatus();
}

int StorageCode(MatrixStorage storage) {
  switch (storage) {
    case MatrixStorage::kBFloat16: return PLUTO_HIP_MATRIX_BF16;
    case MatrixStorage::kFloat32: return PLUTO_HIP_MATRIX_F32;
    case MatrixStorage::kFp8E4M3: return PLUTO_HIP_MATRIX_FP8_E4M3;
  }
  return -1;
}

}  // namespace

// src/llm/layers/matrix_common.cc
StatusOr<size_t> MatrixElementBytes(MatrixStorage storage) {
  switch (storage) {
    case MatrixStorage::kBFloat16: return size_t{2};
    case MatrixStorage::kFloat32: return size_t{4};
    case MatrixStorage::kFp8E4M3: return size_t{1};
  }
  return InvalidArgumentError("unknown matrix storage");
}

FullyConnectedLayer::FullyConnectedLayer(hip::Executor& executor, int input_dim, int output_dim,
                                         BufferVec weights, MatrixStorage storage)
    : executor_(executor), input_dim_(input_dim), output_dim_(output_dim),
      output_type_(DataType::BF16), weights_(std::move(weights)), imported_storage_(storage) {
  input_types_.emplace_back(DataType::BF16, std::vector<int64_t>{1, 1, 1LL * input_dim});
  output_types_.emplace_back(DataType::BF16, std::vector<int64_t>{1, 1, 1LL * output_dim});
}

// src/llm/layers/fully_connected.cc:267-293
StatusOr<std::unique_ptr<FullyConnectedLayer>> FullyConnectedLayer::Create(
    hip::Executor& executor, Buffer weights, MatrixStorage storage, int input_dim, int output_dim,
    std::optional<Buffer> scales) {
  if (input_dim <= 0 || input_dim > kMaximumDimension || output_dim <= 0 ||
      output_dim > kMaximumDimension)
    return InvalidArgumentError("imported linear dimensions must be in [1, 1048576]");
  ASSIGN_OR_RETURN(size_t element_bytes, MatrixElementBytes(storage));
  RETURN_IF_ERROR(internal::ValidateBuffer(
      executor, weights, static_cast<size_t>(input_dim) * output_dim * element_bytes,
      "imported linear weights"));
  if ((storage == MatrixStorage::kFp8E4M3) != scales.has_value())
    return InvalidArgumentError("only FP8 linear weights require block scales");
  BufferVec buffers{std::move(weights)};
  if (scales) {
    RETURN_IF_ERROR(internal::ValidateBuffer(
        executor, *scales,
        static_cast<size_t>((input_dim + 127) / 128) * ((output_dim + 127) / 128) * sizeof(float),
        "imported linear block scales"));
    buffers.push_back(std::move(*scales));
  }
  return std::unique_ptr<FullyConnectedLayer>(
      new FullyConnectedLayer(executor, input_dim, output_dim, std::move(buffers), storage));
}

// src/llm/layers/fully_connected.cc:295-341; the cast of the token to FP32 and
// its FP8 quantization happen inside the library call.
StatusOr<FwdResult> FullyConnectedLayer::ImportedForward(hip::Executor& executor,
                                                         Span<const Buffer> inputs) const {
  const int counts[] = {input_dim_};
  RETURN_IF_ERROR(internal::ValidateBFloat16Inputs(executor, inputs, counts));
  ASSIGN_OR_RETURN(Buffer output,
                   Buffer::Allocate(executor, static_cast<size_t>(output_dim_) * 2));
  const size_t workspace_bytes = pluto_hip_dense_imported_workspace_bytes(input_dim_);
  ASSIGN_OR_RETURN(Buffer workspace, Buffer::Allocate(executor, workspace_bytes));
  const float* scales =
      weights_.size() == 2 ? static_cast<const float*>(weights_[1].data()) : nullptr;
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_dense_imported_forward(executor.stream(), StorageCode(*imported_storage_),
                                       weights_[0].data(), scales, inputs[0].data(), input_dim_,
                                       output_dim_, output.data(), workspace.data(),
                                       workspace_bytes),
      "imported projection launch"));
  return FwdResult{{std::move(output)}, {}};
}

FullyConnectedLayer::FullyConnectedLayer(hip::Executor& executor, int input_dim, int output_dim,
                                         DataType data_type, BufferVec weights, BufferVec gradients,
                                         int sequence_length)
    : executor_(executor), input_dim_(input_dim), output_dim_(output_dim), output_type_(data_type),
      weights_(std::move(weights)), gradients_(std::move(gradients)) {
  const DataType storage = ActivationDataType(data_type);
  input_types_.emplace_back(storage, std::vector<int64_t>{ActivationType::kBatchDimension,
                                                          sequence_length, 1LL * input_dim});
  output_types_.emplace_back(storage, std::vector<int64_t>{ActivationType::kBatchDimension,
                                                           sequence_length, 1LL * output_dim});
}

// src/llm/layers/fully_connected.cc:343-370
StatusOr<std::unique_ptr<FullyConnectedLayer>> FullyConnectedLayer::Create(
    hip::Executor& executor, int input_dim, int output_dim, DataType data_type,
    int sequence_length) {
  if (sequence_length <= 0) return InvalidArgumentError("sequence_length must be positive");
  RETURN_IF_ERROR(internal::ValidateComputeType(data_type));
  RETURN_IF_ERROR(ValidatePositiveExtent(input_dim, "input_dim"));
  RETURN_IF_ERROR(ValidatePositiveExtent(output_dim, "output_dim"));
  const size_t matrix_bytes = static_cast<size_t>(input_dim) * output_dim * sizeof(float);
  const size_t bias_bytes = static_cast<size_t>(output_dim) * sizeof(float);
  BufferVec buffers;
  for (size_t bytes : {matrix_bytes, bias_bytes, matrix_bytes, bias_bytes}) {
    ASSIGN_OR_RETURN(auto buffer, Buffer::Allocate(executor, bytes));
    RETURN_IF_ERROR(hip::HipStatus(
        pluto_hip_memset_async(executor.stream(), buffer.data(), 0, buffer.size_bytes()),
        "hipMemsetAsync(dense parameter)"));
    buffers.push_back(std::move(buffer));
  }
  return std::unique_ptr<FullyConnectedLayer>(new FullyConnectedLayer(
      executor, input_dim, output_dim, data_type, BufferVec{buffers[0], buffers[1]},
      BufferVec{buffers[2], buffers[3]}, sequence_length));
}

// src/llm/layers/fully_connected.cc:372-389
Status FullyConnectedLayer::InitializeIdentity(float scale) {
  if (imported_storage_)
    return FailedPreconditionError("cannot initialize frozen imported linear weights");
  ASSIGN_OR_RETURN(auto matrix, hip::PageLockedHostArray<float>::Allocate(
                                    executor_, static_cast<size_t>(input_dim_) * output_dim_));
  std::fill(matrix.begin(), matrix.end(), 0.0f);
  for (int index = 0; index < std::min(input_dim_, output_dim_); ++index)
    matrix[static_cast<size_t>(index) * output_dim_ + index] = scale;
  // The pinned block is released after this upload in stream order.
  return hip::HipStatus(pluto_hip_memcpy_async(executor_.stream(), weights_[0].data(),
                                               matrix.data(), weights_[0].size_bytes(), 1),
                        "hipMemcpyAsync(identity matrix)");
}

// src/llm/layers/fully_connected.cc:391-413
Status FullyConnectedLayer::InitializeNormal(float standard_deviation, uint64_t seed) {
  if (imported_storage_)
    return FailedPreconditionError("cannot initialize frozen imported linear weights");
  if (!(standard_deviation > 0.0f))
    return InvalidArgumentError("dense initialization standard deviation must be positive");
  std::mt19937_64 random(seed);
  std::normal_distribution<float> distribution(0.0f, standard_deviation);
  ASSIGN_OR_RETURN(auto matrix, hip::PageLockedHostArray<float>::Allocate(
                                    executor_, static_cast<size_t>(input_dim_) * output_dim_));
  for (float& value : matrix) value = distribution(random);
  return hip::HipStatus(pluto_hip_memcpy_async(executor_.stream(), weights_[0].data(),
                                               matrix.data(), weights_[0].size_bytes(), 1),
                        "hipMemcpyAsync(normal matrix)");
}

// src/llm/layers/fully_connected.cc:415-454
StatusOr<FwdResult> FullyConnectedLayer::fwd_impl(hip::Executor& executor,
                                                  Span<const Buffer> inputs, LayerHooks*) const {
  RETURN_IF_ERROR(internal::ValidateExecutor(executor_, executor, "FullyConnectedLayer"));
  if (imported_storage_) return ImportedForward(executor, inputs);
  if (inputs.size() != 1) return InvalidArgumentError("FullyConnectedLayer fwd expects one input");
  ASSIGN_OR_RETURN(int rows, internal::ActivationRows(executor, inputs[0], input_dim_,
                                                      output_type_, "dense input"));
  ASSIGN_OR_RETURN(auto output,
                   Buffer::Allocate(executor, static_cast<size_t>(rows) * output_dim_ *
                                                  internal::ActivationElementBytes(output_type_)));
  // 16-bit copies of the operands; the reference kernels convert tile by tile.
  const size_t workspace_bytes = pluto_hip_dense_workspace_bytes(StorageCode(output_type_), rows,
                                                                 input_dim_, output_dim_);
  ASSIGN_OR_RETURN(auto workspace, Buffer::Allocate(executor, workspace_bytes));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_dense_forward(executor.stream(), StorageCode(output_type_), inputs[0].data(),
                              static_cast<const float*>(weights_[0].data()),
                              static_cast<const float*>(weights_[1].data()), rows, input_dim_,
                              output_dim_, output.data(), workspace.data(), workspace_bytes),
      "dense forward launch"));
  BackwardState state;
  state.intermediates = {inputs[0]};
  return FwdResult{{std::move(output)}, std::move(state)};
}

// src/llm/layers/fully_connected.cc:456-530
StatusOr<BufferVec> FullyConnectedLayer::bwd_impl(hip::Executor& executor,
                                                  Span<const Buffer> output_gradients,
                                                  BackwardState state, LayerHooks*) {
  RETURN_IF_ERROR(internal::ValidateExecutor(executor_, executor, "FullyConnectedLayer"));
  if (imported_storage_)
    return UnimplementedError("imported linear weights do not support backward");
  if (output_gradients.size() != 1 || state.intermediates.size() != 1)
    return InvalidArgumentError(
        "FullyConnectedLayer bwd received an incompatible gradient or state");
  ASSIGN_OR_RETURN(int rows, internal::MatrixRows(executor, output_gradients[0], output_dim_,
                                                  "dense output gradient"));
  RETURN_IF_ERROR(internal::ValidateBuffer(
      executor, state.intermediates[0],
      static_cast<size_t>(rows) * input_dim_ * internal::ActivationElementBytes(output_type_),
      "dense saved input"));
  ASSIGN_OR_RETURN(auto input_gradient,
                   Buffer::Allocate(executor, static_cast<size_t>(rows) * input_dim_ *
                                                  sizeof(float)));
  // Holds the bias partial sums the reference allocates here
  // (fully_connected.cc:508-512) and the 16-bit operand copies.
  const size_t workspace_bytes = pluto_hip_dense_workspace_bytes(StorageCode(output_type_), rows,
                                                                 input_dim_, output_dim_);
  ASSIGN_OR_RETURN(auto workspace, Buffer::Allocate(executor, workspace_bytes));
  RETURN_IF_ERROR(hip::HipStatus(
      pluto_hip_dense_backward(executor.stream(), StorageCode(output_type_),
                               state.intermediates[0].data(),
                               static_cast<const float*>(weights_[0].data()),
                               static_cast<const float*>(output_gradients[0].data()), rows,
                               input_dim_, output_dim_, static_cast<float*>(input_gradient.data()),
                               static_cast<float*>(gradients_[0].data()),
                               static_cast<float*>(gradients_[1].data()), workspace.data(),
                               workspace_bytes),
      "dense backward launch"));
  return BufferVec{std::move(input_gradient)};
}

}  // namespace pluto::llm
