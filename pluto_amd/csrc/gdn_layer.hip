// Layer-level pieces of the gated delta-net around the recurrence: causal
// depthwise convolution + SiLU, decay/beta gates, and the gated RMSNorm output.
// All are bandwidth-trivial elementwise kernels; every bf16 rounding point of
// the reference is kept (src/llm/layers/sequence_delta_net.cc:31-51,88-96,
// 104-121 and src/llm/layers/util/cached_attention_ops.cc:180-203,253-272).
#include "gdn.h"

namespace pluto_hip {
namespace {

__device__ inline float maybe_round(float x, bool round) {
  return round ? round_to_bf16(x) : x;
}

__global__ void __launch_bounds__(256)
conv_sequence_kernel(const void* input, int in_dtype, const float* __restrict__ weight,
                     int length, int channels, int kernel, bool round, void* post,
                     int post_dtype, long long total) {
  const long long i = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total) return;
  const int c = static_cast<int>(i % channels);
  const long long row = i / channels;          // sequence * length + t
  const int t = static_cast<int>(row % length);
  float sum = 0.0f;
  for (int tap = 0; tap < kernel; ++tap) {
    const int source = t + tap - kernel + 1;
    if (source >= 0)
      sum += load_element(input, (row - t + source) * channels + c, in_dtype) *
             weight[static_cast<long long>(c) * kernel + tap];
  }
  sum = maybe_round(sum, round);
  store_element(post, i, post_dtype, maybe_round(sum / (1.0f + expf(-sum)), round));
}

__global__ void __launch_bounds__(128)
conv_step_kernel(const float* __restrict__ input, const float* __restrict__ weight,
                 int channels, int kernel, bool round, float* __restrict__ state,
                 float* __restrict__ output) {
  const int c = blockIdx.x * 128 + threadIdx.x;
  if (c >= channels) return;
  float* taps = state + static_cast<long long>(c) * kernel;
  const float* w = weight + static_cast<long long>(c) * kernel;
  float sum = 0.0f;
  // each channel is owned by one thread; shifting in ascending order never
  // overwrites a source still to be read
  for (int tap = 0; tap < kernel - 1; ++tap) {
    const float previous = taps[tap + 1];
    sum += previous * w[tap];
    taps[tap] = previous;
  }
  const float current = maybe_round(input[c], round);
  taps[kernel - 1] = current;
  sum = maybe_round(sum + current * w[kernel - 1], round);
  output[c] = maybe_round(sum / (1.0f + expf(-sum)), round);
}

__global__ void __launch_bounds__(256)
gates_kernel(const void* a, const void* b, int in_dtype, const float* __restrict__ a_log,
             const float* __restrict__ dt_bias, long long rows, int heads, bool round,
             float* __restrict__ log_decay, float* __restrict__ beta) {
  const long long i = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= rows * heads) return;
  const int head = static_cast<int>(i % heads);
  const float alpha = load_element(a, i, in_dtype) + dt_bias[head];
  // stable softplus: no overflow for strongly positive time steps
  const float softplus = fmaxf(alpha, 0.0f) + log1pf(expf(-fabsf(alpha)));
  log_decay[i] = -expf(a_log[head]) * softplus;
  beta[i] = maybe_round(1.0f / (1.0f + expf(-load_element(b, i, in_dtype))), round);
}

// One wave per (token, head) row of value_dim <= 256 channels.
__global__ void __launch_bounds__(256)
output_kernel(const void* core, int core_dtype, const void* z, int z_dtype,
              const float* __restrict__ norm, long long rows, int value_dim, float epsilon,
              bool round, void* out, int out_dtype) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const long long row = static_cast<long long>(blockIdx.x) * 4 + wave;
  if (row >= rows) return;
  float x[4];
  float square = 0.0f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = lane + 64 * i;
    x[i] = c < value_dim ? load_element(core, row * value_dim + c, core_dtype) : 0.0f;
    square += x[i] * x[i];
  }
  square = wave_sum(square);
  const float inverse = rsqrtf(square / static_cast<float>(value_dim) + epsilon);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = lane + 64 * i;
    if (c >= value_dim) continue;
    const float normalized = maybe_round(x[i] * inverse, round);
    const float affine = maybe_round(normalized * norm[c], round);
    const float gate = load_element(z, row * value_dim + c, z_dtype);
    const float value = affine * (gate / (1.0f + expf(-gate)));
    // the sequence layer stores bf16; the single-token step keeps fp32 and
    // rounds only when asked to (cached_attention_ops.cc:270-271)
    store_element(out, row * value_dim + c, out_dtype,
                  out_dtype == PLUTO_HIP_BF16 ? value : maybe_round(value, round));
  }
}

}  // namespace

int launch_gdn_conv_sequence(hipStream_t stream, const void* input, int in_dtype,
                             const float* weight, int batch, int length, int channels,
                             int kernel, bool round, void* post, int post_dtype) {
  const long long total = static_cast<long long>(batch) * length * channels;
  conv_sequence_kernel<<<static_cast<unsigned>((total + 255) / 256), 256, 0, stream>>>(
      input, in_dtype, weight, length, channels, kernel, round, post, post_dtype, total);
  return launch_status();
}

int launch_gdn_conv_step(hipStream_t stream, const float* input, const float* weight,
                         int channels, int kernel, bool round, float* state, float* output) {
  conv_step_kernel<<<(channels + 127) / 128, 128, 0, stream>>>(input, weight, channels, kernel,
                                                               round, state, output);
  return launch_status();
}

int launch_gdn_gates(hipStream_t stream, const void* a, const void* b, int in_dtype,
                     const float* a_log, const float* dt_bias, long long rows, int heads,
                     bool round, float* log_decay, float* beta) {
  const long long total = rows * heads;
  gates_kernel<<<static_cast<unsigned>((total + 255) / 256), 256, 0, stream>>>(
      a, b, in_dtype, a_log, dt_bias, rows, heads, round, log_decay, beta);
  return launch_status();
}

int launch_gdn_output(hipStream_t stream, const void* core, int core_dtype, const void* z,
                      int z_dtype, const float* norm, long long rows, int value_dim,
                      float epsilon, bool round, void* out, int out_dtype) {
  output_kernel<<<static_cast<unsigned>((rows + 3) / 4), 256, 0, stream>>>(
      core, core_dtype, z, z_dtype, norm, rows, value_dim, epsilon, round, out, out_dtype);
  return launch_status();
}

}  // namespace pluto_hip
