// Per-head RMSNorm with (1 + w) and split-half partial RoPE for one wave per
// head vector, shared by the preparation kernels and the fused decode kernel.
// Semantics and rounding points: PrepareAttentionKernel
// (src/llm/layers/util/cached_attention_ops.cc:30-79) as spelled out by the
// reference's scalar specification (cached_attention_ops_test.cc:56-78).
#pragma once

#include "common.h"

namespace pluto_hip {

__device__ inline float maybe_round(float x, bool round) {
  return round ? round_to_bf16(x) : x;
}

// Two already bf16-representable floats as packed bf16 bits.
__device__ inline uint32_t pack_bf16_bits(float lo, float hi) {
  return (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
}

__device__ inline double wave_sum_f64(double v) {
  for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, 64);
  return v;
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

}  // namespace pluto_hip
