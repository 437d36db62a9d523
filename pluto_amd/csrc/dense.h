// Launchers of the FullyConnectedLayer kernels (dense.hip).
#pragma once

#include "common.h"

namespace pluto_hip {

size_t dense_workspace_bytes(int dtype, int rows, int input_dim, int output_dim);
int launch_dense_forward(hipStream_t stream, int dtype, const void* input, const float* matrix,
                         const float* bias, int rows, int input_dim, int output_dim, void* output,
                         void* workspace);
int launch_dense_backward(hipStream_t stream, int dtype, const void* input, const float* matrix,
                          const float* d_output, int rows, int input_dim, int output_dim,
                          float* d_input, float* d_matrix, float* d_bias, void* workspace);

// Imported (frozen, output-major) projection of one bf16 token (dense_imported.hip).
size_t dense_imported_workspace_bytes(int tokens, int input_dim);
int launch_dense_imported_forward(hipStream_t stream, int storage, const void* weights,
                                  const float* scales, const void* input, int tokens,
                                  int input_dim, int output_dim, void* output, void* workspace);

}  // namespace pluto_hip
