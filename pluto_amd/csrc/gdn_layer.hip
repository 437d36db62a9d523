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
conv_step_kernel(const void* __restrict__ input, int in_dtype, const float* __restrict__ weight,
                 int channels, int kernel, bool round, float* __restrict__ state,
                 float* __restrict__ output) {
  const int c = blockIdx.x * 128 + threadIdx.x;
  if (c >= channels) return;
  // blockIdx.y: the sequence, each with its own shift registers and row
  const long long sequence = blockIdx.y;
  output += sequence * channels;
  float* taps = state + (sequence * channels + c) * kernel;
  const float* w = weight + static_cast<long long>(c) * kernel;
  float sum = 0.0f;
  // each channel is owned by one thread; shifting in ascending order never
  // overwrites a source still to be read
  for (int tap = 0; tap < kernel - 1; ++tap) {
    const float previous = taps[tap + 1];
    sum += previous * w[tap];
    taps[tap] = previous;
  }
  const float current = maybe_round(load_element(input, sequence * channels + c, in_dtype), round);
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

// One token of the gated delta rule for one (sequence, value head) with the
// gates before it and RMSNorm x SiLU(z) after it: DeltaRecurrenceKernel and
// DeltaOutputKernel (cached_attention_ops.cc:205-272) with the gate
// arithmetic of sequence_delta_net.cc:88-96 in one launch.  The state is read
// and written exactly once, every load is issued before anything is waited
// for.
struct StepArgs {
  const float* convolved = nullptr;  // [batch, channels] q | k | v after conv + SiLU
  const void* z = nullptr;           // [batch, vh * vd], fp32 or bf16 (template argument)
  const void* a = nullptr;           // [batch, vh]
  const void* b = nullptr;
  const float* a_log = nullptr;
  const float* dt_bias = nullptr;
  const float* norm = nullptr;
  float* state = nullptr;            // [batch, vh, kd, vd]
  void* out = nullptr;               // [batch, vh * vd], same type as z
  int kh = 0, vh = 0, kd = 0, vd = 0;
  float epsilon = 1e-6f;
  bool round = true;
};

// Threads per workgroup of step_kernel: thread (part, column) = (tid / 128,
// tid % 128) owns rows 16 part .. 16 part + 15 of its column.  With 64 rows a
// thread the kernel needed 272 registers, which left a compute unit four waves
// that loaded, computed and stored in turn (60 us for 32 x 48 heads); sixteen
// waves of 97 registers take 49 us.
constexpr int kStepThreads = 1024;
constexpr int kStepParts = kStepThreads / 128, kStepRows = 128 / kStepParts;

template <int IO>
__global__ void __launch_bounds__(kStepThreads)
step_kernel(StepArgs a) {
  __shared__ float ks[128], qs[128];
  __shared__ float partial[kStepParts][128];
  __shared__ float squares[2];
  const int bh = blockIdx.x, seq = bh / a.vh, head = bh % a.vh;
  const int key_head = head / (a.vh / a.kh);
  const int kd = a.kd, vd = a.vd;
  const int tid = threadIdx.x, column = tid % 128, part = tid / 128;
  const int channels = 2 * a.kh * kd + a.vh * vd;
  const float* token = a.convolved + static_cast<size_t>(seq) * channels;
  float* state = a.state + static_cast<size_t>(bh) * kd * vd;
  const bool active = column < vd;
  const int column_read = active ? column : vd - 1;
  // the state slice: rows beyond the key width read the last row and count as zero
  float s[kStepRows];
#pragma unroll
  for (int r = 0; r < kStepRows; ++r) {
    const int row = kStepRows * part + r;
    const float value = state[min(row, kd - 1) * vd + column_read];
    s[r] = (row < kd && active) ? value : 0.0f;
  }
  if (tid < 128) {
    const int d = min(tid, kd - 1);
    const float kv = token[(a.kh + key_head) * kd + d], qv = token[key_head * kd + d];
    ks[tid] = tid < kd ? kv : 0.0f;
    qs[tid] = tid < kd ? qv : 0.0f;
  }
  const float value = token[2 * a.kh * kd + head * vd + column_read];
  const float gate =
      load_element(a.z, (static_cast<long long>(seq) * a.vh + head) * vd + column_read, IO);
  const float weight = a.norm[column_read];
  const size_t scalar = static_cast<size_t>(seq) * a.vh + head;
  const float alpha = load_element(a.a, scalar, IO) + a.dt_bias[head];
  // stable softplus: no overflow for strongly positive time steps
  const float softplus = fmaxf(alpha, 0.0f) + log1pf(expf(-fabsf(alpha)));
  const float decay = __expf(-expf(a.a_log[head]) * softplus);
  const float beta = maybe_round(1.0f / (1.0f + expf(-load_element(a.b, scalar, IO))), a.round);
  __syncthreads();
  // the normalised key and the normalised, scaled query replace the raw ones
  // in LDS (1e-6 inside the root: cached_attention_ops.cc:224-228)
  float k_scaled = 0.0f, q_scaled = 0.0f;
  if (tid < 128) {
    float kk = 1e-6f, qq = 1e-6f;
    for (int d = 0; d < 128; ++d) {
      kk += ks[d] * ks[d];
      qq += qs[d] * qs[d];
    }
    k_scaled = ks[tid] * rsqrtf(kk);
    q_scaled = qs[tid] * (rsqrtf(qq) / sqrtf(static_cast<float>(kd)));
  }
  __syncthreads();
  if (tid < 128) {
    ks[tid] = k_scaled;
    qs[tid] = q_scaled;
  }
  __syncthreads();
  float prediction = 0.0f;
#pragma unroll
  for (int r = 0; r < kStepRows; ++r) {
    s[r] *= decay;
    prediction += s[r] * ks[kStepRows * part + r];
  }
  partial[part][column] = prediction;
  __syncthreads();
  float predicted = partial[0][column];
#pragma unroll
  for (int i = 1; i < kStepParts; ++i) predicted += partial[i][column];
  const float delta = (value - predicted) * beta;
  __syncthreads();
  float output = 0.0f;
#pragma unroll
  for (int r = 0; r < kStepRows; ++r) {
    s[r] += ks[kStepRows * part + r] * delta;
    output += s[r] * qs[kStepRows * part + r];
  }
#pragma unroll
  for (int r = 0; r < kStepRows; ++r) {
    const int row = kStepRows * part + r;
    if (row < kd && active) state[row * vd + column] = s[r];
  }
  partial[part][column] = output;
  __syncthreads();
  // RMSNorm over the head's columns, then the SiLU(z) gate
  float core = 0.0f;
  if (part == 0 && active) {
    core = partial[0][column];
#pragma unroll
    for (int i = 1; i < kStepParts; ++i) core += partial[i][column];
    core = maybe_round(core, a.round);
  }
  const float square = wave_sum(core * core);
  if (part == 0 && tid % 64 == 0) squares[tid / 64] = square;
  __syncthreads();
  if (part != 0 || !active) return;
  const float inverse = rsqrtf((squares[0] + squares[1]) / static_cast<float>(vd) + a.epsilon);
  const float normalized = maybe_round(core * inverse, a.round);
  const float affine = maybe_round(normalized * weight, a.round);
  const float result = affine * (gate / (1.0f + expf(-gate)));
  // a bf16 result is rounded once, by the store: the FP32 step followed by the
  // layer's cast (delta_net.cc:97-101) gives the same bits with or without the flag
  store_element(a.out, (static_cast<long long>(seq) * a.vh + head) * vd + column, IO,
                IO == PLUTO_HIP_BF16 ? result : maybe_round(result, a.round));
}

}  // namespace

bool gdn_step_fused_supported(int key_dim, int value_dim) {
  return key_dim <= 128 && value_dim <= 128;
}

int launch_gdn_step_fused(hipStream_t stream, const float* convolved, const void* z,
                          const void* a, const void* b, int io_dtype, const float* a_log,
                          const float* dt_bias, const float* norm, int batch, int key_heads,
                          int value_heads, int key_dim, int value_dim, float epsilon, bool round,
                          float* state, void* out) {
  StepArgs s;
  s.convolved = convolved;
  s.z = z;
  s.a = a;
  s.b = b;
  s.a_log = a_log;
  s.dt_bias = dt_bias;
  s.norm = norm;
  s.state = state;
  s.out = out;
  s.kh = key_heads;
  s.vh = value_heads;
  s.kd = key_dim;
  s.vd = value_dim;
  s.epsilon = epsilon;
  s.round = round;
  if (io_dtype == PLUTO_HIP_BF16)
    step_kernel<PLUTO_HIP_BF16><<<batch * value_heads, kStepThreads, 0, stream>>>(s);
  else
    step_kernel<PLUTO_HIP_F32><<<batch * value_heads, kStepThreads, 0, stream>>>(s);
  return launch_status();
}

int launch_gdn_conv_sequence(hipStream_t stream, const void* input, int in_dtype,
                             const float* weight, int batch, int length, int channels,
                             int kernel, bool round, void* post, int post_dtype) {
  const long long total = static_cast<long long>(batch) * length * channels;
  conv_sequence_kernel<<<static_cast<unsigned>((total + 255) / 256), 256, 0, stream>>>(
      input, in_dtype, weight, length, channels, kernel, round, post, post_dtype, total);
  return launch_status();
}

int launch_gdn_conv_step(hipStream_t stream, const void* input, int in_dtype, const float* weight,
                         int batch, int channels, int kernel, bool round, float* state,
                         float* output) {
  conv_step_kernel<<<dim3((channels + 127) / 128, batch), 128, 0, stream>>>(
      input, in_dtype, weight, channels, kernel, round, state, output);
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
