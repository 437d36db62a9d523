// Argument block of the gated delta-net kernels and the per-chunk scratch
// layout shared by the two kernels of the chunked scan.
#pragma once

#include "common.h"

namespace pluto_hip {

// Scratch written by the chunk-parallel kernel for one 64-token chunk of one
// (sequence, head):
//   T        bf16 [6 fragments][64 lanes][8]                     6 KiB
//            (I + A)^-1 in matrix-core operand order: fragment (token tile i,
//            token block kb) for (0,0) (1,0) (2,0) (2,1) (3,0) (3,1); the other
//            two are zero, the matrix being lower triangular
//   A2       bf16 same shape: M o (Q K^T) with every factor       6 KiB
//   factors  fp32 [4][64]: beta, beta exp(c)/|k|, q_scale exp(c)/|q|,
//            exp(c_C - c)/|k| per token; then exp(c_C)            2 KiB
constexpr size_t kGdnOffsetT = 0;
constexpr size_t kGdnOffsetA2 = 6144;
constexpr size_t kGdnOffsetFactors = 12288;
constexpr size_t kGdnChunkBytes = 14336;

struct GdnArgs {
  // Row `token` (= sequence * T + t) of q starts at q + token * q_token_stride
  // elements, head h at + h * kd; likewise k and v (head h at + h * vd).
  // bf16 for the chunked scan; the recurrence kernel also reads fp32.
  const uint16_t* q = nullptr;
  const uint16_t* k = nullptr;
  const uint16_t* v = nullptr;
  long long q_token_stride = 0, k_token_stride = 0, v_token_stride = 0;
  int in_dtype = PLUTO_HIP_BF16;
  const float* log_decay = nullptr;  // [batch, T, vh]
  const float* beta = nullptr;
  float* state = nullptr;   // fp32 [batch, vh, kd, vd]
  uint16_t* out = nullptr;  // bf16 [batch, T, vh, vd] (chunked scan)
  void* out_any = nullptr;  // recurrence kernel: bf16 or fp32
  char* workspace = nullptr;
  int batch = 0, length = 0;
  int key_heads = 0, value_heads = 0, key_dim = 0, value_dim = 0;
  int normalize_qk = 0;
  int round_output = 1;
  float q_scale = 1.0f;
};

bool gdn_chunked_supported(const GdnArgs& args, int chunk);
int launch_gdn_chunked(hipStream_t stream, const GdnArgs& args);
int launch_gdn_recurrence(hipStream_t stream, const GdnArgs& args, int out_dtype);

// Layer-level pieces around the scan (gdn_layer.hip).
// Causal depthwise convolution + SiLU over whole sequences with zero history:
// ConvForward, src/llm/layers/sequence_delta_net.cc:31-51.
int launch_gdn_conv_sequence(hipStream_t stream, const void* input, int in_dtype,
                             const float* weight, int batch, int length, int channels,
                             int kernel, bool round, void* post, int post_dtype);
// One token per sequence against that sequence's [channels, kernel] shift
// register (input, output [batch, channels]; state [batch, channels, kernel]):
// ConvolutionKernel, src/llm/layers/util/cached_attention_ops.cc:180-203.
int launch_gdn_conv_step(hipStream_t stream, const void* input, int in_dtype, const float* weight,
                         int batch, int channels, int kernel, bool round, float* state,
                         float* output);
// Gates, one token of the recurrence and the output norm/gate of `batch`
// sequences in one launch, for key and value widths up to 128 (step_kernel).
bool gdn_step_fused_supported(int key_dim, int value_dim);
int launch_gdn_step_fused(hipStream_t stream, const float* convolved, const void* z,
                          const void* a, const void* b, int io_dtype, const float* a_log,
                          const float* dt_bias, const float* norm, int batch, int key_heads,
                          int value_heads, int key_dim, int value_dim, float epsilon, bool round,
                          float* state, void* out);
// g = -exp(A_log) softplus(a + dt_bias), beta = round(sigmoid(b)):
// sequence_delta_net.cc:88-96.
int launch_gdn_gates(hipStream_t stream, const void* a, const void* b, int in_dtype,
                     const float* a_log, const float* dt_bias, long long rows, int heads,
                     bool round, float* log_decay, float* beta);
// RMSNorm (plain weight) x SiLU(z): OutputForward, sequence_delta_net.cc:104-121.
int launch_gdn_output(hipStream_t stream, const void* core, int core_dtype, const void* z,
                      int z_dtype, const float* norm, long long rows, int value_dim,
                      float epsilon, bool round, void* out, int out_dtype);

// Chunked form of the recurrence part of the backward for 128 x 128 heads
// (gdn_backward_chunked.hip): `forward` leaves the outputs in `core`, `reverse`
// (after `dcore` is known) leaves dv in `dpost` and the q/k and gate gradients
// as one partial per (token, value head), in the layout the token-by-token
// kernels use with a single column tile.
struct GdnChunkedBackward {
  const float* post = nullptr;   // [T, channels] convolved, activated q | k | v
  const uint16_t* a = nullptr;   // bf16 [T, vh]
  const uint16_t* b = nullptr;
  const float* a_log = nullptr;
  const float* dt_bias = nullptr;
  const float* dcore = nullptr;  // [T, vh, 128]
  float* core = nullptr;         // [T, vh, 128]
  float* dpost = nullptr;
  float* qk_partials = nullptr;      // [T, vh, 2, 128]
  float* scalar_partials = nullptr;  // [T, vh, 3]
  float* records = nullptr;          // gdn_backward_chunked_bytes(...)
  int length = 0, key_heads = 0, value_heads = 0;
  bool round = true;
};
bool gdn_backward_chunked_supported(const pluto_hip_delta_params* p);
size_t gdn_backward_chunked_bytes(const pluto_hip_delta_params* p, int length);
int launch_gdn_backward_chunked_forward(hipStream_t stream, const GdnChunkedBackward& c);
int launch_gdn_backward_chunked_reverse(hipStream_t stream, const GdnChunkedBackward& c);

// Backward of the whole layer for one sequence (gdn_backward.hip): the forward
// pass is repeated with the states it needs kept in `workspace` (one per
// 64-token chunk for 128 x 128 heads, one per token otherwise).
constexpr int kGdnSumChunks = 512;
size_t gdn_backward_workspace_bytes(const pluto_hip_delta_params* p, int length, bool norm_grad);
int launch_gdn_backward(hipStream_t stream, const pluto_hip_delta_params* p, int length,
                        const void* qkv, const void* z, const void* a, const void* b,
                        const float* conv_weight, const float* a_log, const float* dt_bias,
                        const float* norm, const float* dy, float* dqkv, float* dz, float* da,
                        float* db, float* d_conv_weight, float* d_a_log, float* d_dt_bias,
                        float* d_norm, void* workspace);

}  // namespace pluto_hip
