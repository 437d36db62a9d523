// Qwen attention input preparation: per-head RMSNorm with (1 + w), split-half
// partial RoPE, and the append of K / V to the cache.
//
// Semantics: PrepareKernel (src/llm/layers/qwen_attention.cc:30-63) and
// PrepareAttentionKernel (src/llm/layers/util/cached_attention_ops.cc:30-79),
// with every bf16 rounding point of the reference's scalar specification
// (src/llm/layers/util/cached_attention_ops_test.cc:56-78).  The normalisation
// and the rotation angle are evaluated in FP64 like that specification, so the
// rounded results agree with it except on exact rounding ties.
#include "gqa.h"

namespace pluto_hip {
namespace {

__device__ inline float maybe_round(float x, bool round) {
  return round ? round_to_bf16(x) : x;
}

__device__ inline double wave_sum_f64(double v) {
  for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
  return v;
}

// cos/sin of position * theta^(-2 i / rotary) for i < rotary/2, rounded.
__global__ void __launch_bounds__(256)
rope_table_kernel(int start_position, int length, int rotary_dim, float theta,
                  bool round, float* __restrict__ cosines, float* __restrict__ sines) {
  const int half = rotary_dim / 2;
  const long long i = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  if (i >= static_cast<long long>(length) * half) return;
  const int row = static_cast<int>(i / half), f = static_cast<int>(i % half);
  const double angle = static_cast<double>(start_position + row) *
                       pow(static_cast<double>(theta), -2.0 * f / rotary_dim);
  cosines[i] = maybe_round(static_cast<float>(cos(angle)), round);
  sines[i] = maybe_round(static_cast<float>(sin(angle)), round);
}

// Normalises and rotates one head vector held one-or-more channels per lane.
// `x` reads the raw input, cos_row/sin_row hold rotary/2 rounded values.
struct HeadInput {
  const void* base;
  long long offset;
  int dtype;
  __device__ float operator()(int c) const { return load_element(base, offset + c, dtype); }
};

template <class Sink>
__device__ inline void normalize_rotate(const HeadInput& x, const float* weight,
                                        int dim, int rotary_dim, float epsilon,
                                        bool round, const float* cos_row,
                                        const float* sin_row, Sink sink) {
  const int lane = threadIdx.x % 64;
  double square = 0.0;
  for (int c = lane; c < dim; c += 64) {
    const float v = x(c);
    square += static_cast<double>(v * v);
  }
  square = wave_sum_f64(square);
  const double inverse = 1.0 / sqrt(square / dim + static_cast<double>(epsilon));
  const int half = rotary_dim / 2;
  for (int c = lane; c < dim; c += 64) {
    const float n = maybe_round(
        static_cast<float>(x(c) * inverse * (1.0 + static_cast<double>(weight[c]))), round);
    float result = n;
    if (c < rotary_dim) {
      const int partner = c < half ? c + half : c - half;
      const int f = c < half ? c : c - half;
      const float np = maybe_round(
          static_cast<float>(x(partner) * inverse *
                             (1.0 + static_cast<double>(weight[partner]))),
          round);
      const float cosine = cos_row[f], sine = sin_row[f];
      const float a = maybe_round(n * cosine, round);
      const float b = maybe_round(np * sine, round);
      result = maybe_round(c < half ? a - b : a + b, round);
    }
    sink(c, result);
  }
}

// One wave per (row, head); heads [0, qh) are queries, [qh, qh + kh) keys
// (the key wave also stores the value row).
__global__ void __launch_bounds__(256)
prefill_prepare_kernel(PrefillPrepareArgs a) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int heads = a.query_heads + a.key_value_heads;
  const long long unit = static_cast<long long>(blockIdx.x) * 4 + wave;
  if (unit >= static_cast<long long>(a.length) * heads) return;
  const int row = static_cast<int>(unit / heads);
  const int head = static_cast<int>(unit % heads);
  const int d = a.head_dim, half = a.rotary_dim / 2;
  const float* cos_row = a.cosines + static_cast<long long>(row) * half;
  const float* sin_row = a.sines + static_cast<long long>(row) * half;
  if (head < a.query_heads) {
    const HeadInput x{a.qg, (static_cast<long long>(row) * a.query_heads + head) * 2 * d,
                      PLUTO_HIP_BF16};
    const long long out = (static_cast<long long>(row) * a.query_heads + head) * d;
    normalize_rotate(x, a.q_norm, d, a.rotary_dim, a.epsilon, a.round, cos_row, sin_row,
                     [&](int c, float v) { store_element(a.q_out, out + c, a.q_out_dtype, v); });
  } else {
    const int kv = head - a.query_heads;
    const long long in = (static_cast<long long>(row) * a.key_value_heads + kv) * d;
    const HeadInput x{a.k, in, PLUTO_HIP_BF16};
    const long long out = static_cast<long long>(a.start_position + row) * a.cache.token_stride +
                          kv * a.cache.head_stride;
    normalize_rotate(x, a.k_norm, d, a.rotary_dim, a.epsilon, a.round, cos_row, sin_row,
                     [&](int c, float v) { store_element(a.cache.keys, out + c, a.cache.dtype, v); });
    for (int c = lane; c < d; c += 64) {
      const float v = load_element(a.v, in + c, PLUTO_HIP_BF16);
      store_element(a.cache.values, out + c, a.cache.dtype, maybe_round(v, a.round));
    }
  }
}

// Decode: one wave per (sequence, head); the angle is evaluated in place.
__global__ void __launch_bounds__(256)
decode_prepare_kernel(DecodePrepareArgs a, DecodeBatch batch) {
  __shared__ float cos_s[4][128];
  __shared__ float sin_s[4][128];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int heads = a.query_heads + a.key_value_heads;
  const long long unit = static_cast<long long>(blockIdx.x) * 4 + wave;
  if (unit >= static_cast<long long>(batch.count) * heads) return;
  const int b = static_cast<int>(unit / heads);
  const int head = static_cast<int>(unit % heads);
  const int d = a.head_dim, half = a.rotary_dim / 2;
  const int position = batch.positions[b];
  for (int f = lane; f < half; f += 64) {
    const double angle = static_cast<double>(position) *
                         pow(static_cast<double>(a.theta), -2.0 * f / a.rotary_dim);
    cos_s[wave][f] = maybe_round(static_cast<float>(cos(angle)), a.round);
    sin_s[wave][f] = maybe_round(static_cast<float>(sin(angle)), a.round);
  }
  // Only this wave reads what it wrote; a wave executes in lock step.
  __builtin_amdgcn_wave_barrier();
  const int seq = batch.first + b;
  if (head < a.query_heads) {
    const HeadInput x{a.q_gate, (static_cast<long long>(seq) * a.query_heads + head) * 2 * d,
                      a.io_dtype};
    const long long out = (static_cast<long long>(seq) * a.query_heads + head) * d;
    normalize_rotate(x, a.q_norm, d, a.rotary_dim, a.epsilon, a.round, cos_s[wave],
                     sin_s[wave],
                     [&](int c, float v) { store_element(a.q_out, out + c, a.q_out_dtype, v); });
  } else {
    const int kv = head - a.query_heads;
    const long long in = (static_cast<long long>(seq) * a.key_value_heads + kv) * d;
    const HeadInput x{a.k, in, a.io_dtype};
    const long long out =
        static_cast<long long>(position) * a.token_stride + kv * a.head_stride;
    void* keys = batch.keys[b];
    void* values = batch.values[b];
    normalize_rotate(x, a.k_norm, d, a.rotary_dim, a.epsilon, a.round, cos_s[wave],
                     sin_s[wave],
                     [&](int c, float v) { store_element(keys, out + c, a.cache_dtype, v); });
    for (int c = lane; c < d; c += 64) {
      const float v = load_element(a.v, in + c, a.io_dtype);
      store_element(values, out + c, a.cache_dtype, maybe_round(v, a.round));
    }
  }
}

}  // namespace

int launch_rope_table(hipStream_t stream, int start_position, int length,
                      int rotary_dim, float theta, bool round, float* cosines,
                      float* sines) {
  const long long count = static_cast<long long>(length) * (rotary_dim / 2);
  rope_table_kernel<<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(
      start_position, length, rotary_dim, theta, round, cosines, sines);
  return launch_status();
}

int launch_prefill_prepare(hipStream_t stream, const PrefillPrepareArgs& a) {
  const long long units =
      static_cast<long long>(a.length) * (a.query_heads + a.key_value_heads);
  prefill_prepare_kernel<<<static_cast<unsigned>((units + 3) / 4), 256, 0, stream>>>(a);
  return launch_status();
}

int launch_decode_prepare(hipStream_t stream, const DecodePrepareArgs& a,
                          const DecodeBatch& batch) {
  const long long units =
      static_cast<long long>(batch.count) * (a.query_heads + a.key_value_heads);
  decode_prepare_kernel<<<static_cast<unsigned>((units + 3) / 4), 256, 0, stream>>>(a, batch);
  return launch_status();
}

}  // namespace pluto_hip
