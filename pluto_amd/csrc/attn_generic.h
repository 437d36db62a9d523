// Argument blocks and launchers of the any-shape FP32-arithmetic kernels.
#pragma once

#include "common.h"

namespace pluto_hip {

// Element (seq, row, head, c) of a tensor is
// base[seq*seq_stride + row*row_stride + head*head_stride + c].
struct StridedView {
  const void* base = nullptr;
  long long seq_stride = 0;
  long long row_stride = 0;
  long long head_stride = 0;
  int dtype = PLUTO_HIP_F32;
};

struct GenericForwardArgs {
  StridedView q, k, v;
  StridedView gate;  // optional sigmoid gate logits, indexed like q
  void* out = nullptr;
  long long o_seq_stride = 0, o_row_stride = 0, o_head_stride = 0;
  int o_dtype = PLUTO_HIP_F32;
  float* maxima = nullptr;       // [(seq*QH + head)*q_rows + row]
  float* normalizers = nullptr;  // same layout
  float* lse = nullptr;          // [(seq*q_rows + row)*QH + head]
  int q_rows = 0;          // query rows per sequence
  int kv_rows = 0;         // valid key rows per sequence
  int start_position = 0;  // query row i sees keys [0, start_position + i]
  int query_heads = 0;
  int group = 1;  // query heads per key/value head
  int head_dim = 0;
  float scale = 1.0f;
  int round_to_bf16 = 0;  // rounding points of the gated output
};

struct GenericBackwardArgs {
  const void* qkv = nullptr;  // packed [rows, 3E]
  const void* out = nullptr;  // stored forward output [rows, E]
  int dtype = PLUTO_HIP_F32;
  const float* d_out = nullptr;
  const float* maxima = nullptr;
  const float* normalizers = nullptr;
  float* deltas = nullptr;
  float* d_qkv = nullptr;
  int rows = 0, context_length = 0, num_heads = 0, embedding_dim = 0;
  float scale = 1.0f;
};

int launch_generic_forward(hipStream_t stream, const GenericForwardArgs& args,
                           int sequences);
// FP32 storage, FP32 matrix-core arithmetic, head widths 32/64/128, no gate
// (attn_f32_mfma.hip).
bool f32_forward_supported(const GenericForwardArgs& args);
int launch_f32_forward(hipStream_t stream, const GenericForwardArgs& args, int sequences);
int launch_generic_probabilities(hipStream_t stream,
                                 const GenericForwardArgs& args, int sequences,
                                 float* probabilities);
int launch_generic_delta(hipStream_t stream, const GenericBackwardArgs& args);
int launch_generic_backward(hipStream_t stream, const GenericBackwardArgs& args);

}  // namespace pluto_hip
