// Backward of the gated delta-net layer over a sequence
// (SequenceDeltaNetLayer::bwd_impl, src/llm/layers/sequence_delta_net.cc:
// 482-561) in FP32, token by token as the reference does it: the forward pass
// is repeated with every state S_t kept, then the recurrence is differentiated
// in reverse.  Kernels and the reference kernels they follow:
//   conv_train_kernel            ConvForward            (:31-51), keeps `pre`
//   recurrence_states_kernel     RecurrenceForward      (:55-102)
//   output_backward_kernel       OutputBackward         (:125-155)
//   recurrence_backward_kernel   RecurrenceBackward     (:171-253)
//   gather_qk_kernel             GatherQkGradient       (:255-276)
//   gather_scalar_kernel         GatherScalarGradient   (:278-305)
//   conv_silu_backward_kernel    ConvSiluBackward       (:307-318)
//   conv_input_backward_kernel   ConvInputBackward      (:320-336)
//   conv_weight_*_kernel         ConvWeightBackward     (:338-355), two levels
//   sum_rows_*_kernel            SumNormGradient        (:157-166), two levels
//
// The two recurrence kernels share one layout: a workgroup owns the
// [key_dim, 32] slice of one head's state (as the reference's programs do),
// thread (kg, c) = (tid / 32, tid % 32) holds rows 16 kg .. 16 kg + 15 of
// column c in registers.  Sums over rows go through LDS (8 partials a column),
// sums over columns through LDS as well (one padded row of products per state
// row, added up by one thread per row).  What a token reads from global memory
// is requested one token ahead.
#include "gdn.h"

namespace pluto_hip {
namespace {

constexpr int kRows = 16;        // state rows per thread
constexpr int kGroups = 8;       // row groups per workgroup
constexpr int kColumns = 32;     // state columns per workgroup
constexpr int kMaxKey = kRows * kGroups;  // 128
constexpr int kConvSlices = 64;  // token slices of the convolution weight gradient

__device__ inline float round_if(float x, bool round) { return round ? round_to_bf16(x) : x; }

// VEC consecutive elements of a row as one access (VEC is 1 or 4).
template <int VEC>
struct Pack {
  float e[VEC];
};
template <int VEC>
__device__ inline Pack<VEC> load_floats(const float* p) {
  Pack<VEC> r;
  if constexpr (VEC == 4) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    r.e[0] = v.x; r.e[1] = v.y; r.e[2] = v.z; r.e[3] = v.w;
  } else {
    r.e[0] = p[0];
  }
  return r;
}
template <int VEC>
__device__ inline void store_floats(float* p, const Pack<VEC>& v) {
  if constexpr (VEC == 4)
    *reinterpret_cast<float4*>(p) = make_float4(v.e[0], v.e[1], v.e[2], v.e[3]);
  else
    p[0] = v.e[0];
}
template <int VEC>
__device__ inline Pack<VEC> load_bf16s(const uint16_t* p) {
  Pack<VEC> r;
  if constexpr (VEC == 4) {
    const uint2 bits = *reinterpret_cast<const uint2*>(p);
    r.e[0] = __uint_as_float(bits.x << 16);
    r.e[1] = __uint_as_float(bits.x & 0xffff0000u);
    r.e[2] = __uint_as_float(bits.y << 16);
    r.e[3] = __uint_as_float(bits.y & 0xffff0000u);
  } else {
    r.e[0] = bf16_bits_to_float(p[0]);
  }
  return r;
}

// One thread per VEC channels of a token (channels % VEC == 0).
template <int VEC>
__global__ void __launch_bounds__(256)
conv_train_kernel(const uint16_t* input, const float* __restrict__ weight, int length,
                  int channels, int kernel, bool round, float* pre, float* post) {
  const int groups = channels / VEC;
  const long long i = blockIdx.x * 256LL + threadIdx.x;
  if (i >= 1LL * length * groups) return;
  const int c = static_cast<int>(i % groups) * VEC, t = static_cast<int>(i / groups);
  Pack<VEC> sum;
#pragma unroll
  for (int e = 0; e < VEC; ++e) sum.e[e] = 0.0f;
  for (int tap = 0; tap < kernel; ++tap) {
    const int source = t + tap - kernel + 1;
    if (source < 0) continue;
    const Pack<VEC> x = load_bf16s<VEC>(input + 1LL * source * channels + c);
#pragma unroll
    for (int e = 0; e < VEC; ++e) sum.e[e] += x.e[e] * weight[1LL * (c + e) * kernel + tap];
  }
  Pack<VEC> activated;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    sum.e[e] = round_if(sum.e[e], round);
    activated.e[e] = round_if(sum.e[e] / (1.0f + expf(-sum.e[e])), round);
  }
  store_floats<VEC>(pre + 1LL * t * channels + c, sum);
  store_floats<VEC>(post + 1LL * t * channels + c, activated);
}

struct RecurrenceArgs {
  const float* post = nullptr;     // [T, channels]
  const uint16_t* a = nullptr;     // bf16 [T, vh]
  const uint16_t* b = nullptr;
  const float* a_log = nullptr;
  const float* dt_bias = nullptr;
  float* states = nullptr;         // [(T + 1), vh, kd, vd]
  float* core = nullptr;           // [T, vh, vd]
  const float* dcore = nullptr;    // [T, vh, vd]
  float* qk_partials = nullptr;    // [T, vh, tiles, 2, kd]
  float* scalar_partials = nullptr;  // [T, vh, tiles, 3]
  float* dpost = nullptr;          // [T, channels]; the value part is written here
  int length = 0, kh = 0, vh = 0, kd = 0, vd = 0;
  bool round = true;
};

struct TokenScalars {
  float alpha, softplus, rate, decay, sigmoid, beta;
};

// What a thread reads from global memory for one token.  It is requested one
// token ahead, so that the sequential chain never waits for these loads.
struct TokenInputs {
  float q[2], k[2];   // wave 0: raw q and k channels lane and lane + 64
  float a, b;         // the head's gate logits
  float v, dy;        // this thread's value column and (backward) its gradient
};

__device__ inline TokenInputs fetch_token(const RecurrenceArgs& a, int t, int head, int key_head,
                                          int column, bool column_ok, bool with_gradient) {
  TokenInputs in;
  const int channels = 2 * a.kh * a.kd + a.vh * a.vd;
  const int tid = threadIdx.x;
  in.q[0] = in.q[1] = in.k[0] = in.k[1] = 0.0f;
  if (tid < 64) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int d = tid + 64 * j;
      if (d < a.kd) {
        in.q[j] = a.post[1LL * t * channels + key_head * a.kd + d];
        in.k[j] = a.post[1LL * t * channels + (a.kh + key_head) * a.kd + d];
      }
    }
  }
  in.a = bf16_bits_to_float(a.a[1LL * t * a.vh + head]);
  in.b = bf16_bits_to_float(a.b[1LL * t * a.vh + head]);
  in.v = column_ok ? a.post[1LL * t * channels + 2 * a.kh * a.kd + head * a.vd + column] : 0.0f;
  in.dy = (with_gradient && column_ok) ? a.dcore[(1LL * t * a.vh + head) * a.vd + column] : 0.0f;
  return in;
}

__device__ inline TokenScalars token_scalars(const RecurrenceArgs& a, const TokenInputs& in,
                                             int head) {
  TokenScalars s;
  s.alpha = in.a + a.dt_bias[head];
  s.softplus = fmaxf(s.alpha, 0.0f) + logf(1.0f + expf(-fabsf(s.alpha)));
  s.rate = expf(a.a_log[head]);
  s.decay = expf(-s.rate * s.softplus);
  s.sigmoid = 1.0f / (1.0f + expf(-in.b));
  s.beta = round_if(s.sigmoid, a.round);
  return s;
}

// Raw q and k of the token into LDS together with 1/|q|, 1/|k| (1e-6 added to
// the sums of squares, sequence_delta_net.cc:84-85).
__device__ inline void publish_token_qk(const TokenInputs& in, float* raw_q, float* raw_k,
                                        float* inverses) {
  const int tid = threadIdx.x;
  if (tid < 64) {
    float qq = 0.0f, kk = 0.0f;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      raw_q[tid + 64 * j] = in.q[j];
      raw_k[tid + 64 * j] = in.k[j];
      qq += in.q[j] * in.q[j];
      kk += in.k[j] * in.k[j];
    }
    qq = wave_sum(qq);
    kk = wave_sum(kk);
    if (tid == 0) {
      inverses[0] = rsqrtf(qq + 1e-6f);
      inverses[1] = rsqrtf(kk + 1e-6f);
    }
  }
}

// Sum over the kGroups row groups of a per-column partial.
__device__ inline float column_total(float partial, float (*scratch)[kColumns], int kg, int c) {
  scratch[kg][c] = partial;
  __syncthreads();
  float total = 0.0f;
#pragma unroll
  for (int g = 0; g < kGroups; ++g) total += scratch[g][c];
  __syncthreads();
  return total;
}

__global__ void __launch_bounds__(256)
recurrence_states_kernel(RecurrenceArgs a) {
  __shared__ float raw_q[kMaxKey], raw_k[kMaxKey], inverses[2];
  __shared__ float scratch[kGroups][kColumns];
  const int tiles = (a.vd + kColumns - 1) / kColumns;
  const int head = blockIdx.x / tiles, tile = blockIdx.x % tiles;
  const int key_head = head / (a.vh / a.kh);
  const int kg = threadIdx.x / kColumns, c = threadIdx.x % kColumns;
  const int column = tile * kColumns + c;
  const bool column_ok = column < a.vd;
  const int channels = 2 * a.kh * a.kd + a.vh * a.vd;
  const size_t stride = static_cast<size_t>(a.vh) * a.kd * a.vd;
  const float norm_scale = sqrtf(static_cast<float>(a.kd));
  float m[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    m[r] = 0.0f;
    const int row = kg * kRows + r;
    if (row < a.kd && column_ok) a.states[(static_cast<size_t>(head) * a.kd + row) * a.vd + column] = 0.0f;
  }
  TokenInputs next = fetch_token(a, 0, head, key_head, column, column_ok, false);
  for (int t = 0; t < a.length; ++t) {
    const TokenInputs in = next;
    if (t + 1 < a.length) next = fetch_token(a, t + 1, head, key_head, column, column_ok, false);
    publish_token_qk(in, raw_q, raw_k, inverses);
    __syncthreads();
    const TokenScalars s = token_scalars(a, in, head);
    const float iq = inverses[0], ik = inverses[1];
    float prediction = 0.0f;
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      m[r] *= s.decay;
      prediction += m[r] * (raw_k[kg * kRows + r] * ik);
    }
    prediction = column_total(prediction, scratch, kg, c);
    const float delta = (in.v - prediction) * s.beta;
    float out = 0.0f;
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int row = kg * kRows + r;
      m[r] += (raw_k[row] * ik) * delta;
      out += m[r] * (raw_q[row] * iq / norm_scale);
      if (row < a.kd && column_ok)
        a.states[(t + 1) * stride + (static_cast<size_t>(head) * a.kd + row) * a.vd + column] = m[r];
    }
    out = column_total(out, scratch, kg, c);
    if (kg == 0 && column_ok) a.core[(1LL * t * a.vh + head) * a.vd + column] = round_if(out, a.round);
  }
}

__global__ void __launch_bounds__(256)
recurrence_backward_kernel(RecurrenceArgs a) {
  __shared__ float raw_q[kMaxKey], raw_k[kMaxKey], inverses[2];
  __shared__ float scratch[kGroups][kColumns];
  __shared__ float dq_rows[kMaxKey], dk_rows[kMaxKey];
  __shared__ float block_sums[4][3];
  // per-element products whose sums over the 32 columns give dq and dk: one
  // padded row per state row, summed by one thread per row (a lane shuffle
  // tree per row costs a multiple of this)
  __shared__ float q_products[kMaxKey][kColumns + 1], k_products[kMaxKey][kColumns + 1];
  const int tiles = (a.vd + kColumns - 1) / kColumns;
  const int head = blockIdx.x / tiles, tile = blockIdx.x % tiles;
  const int key_head = head / (a.vh / a.kh);
  const int tid = threadIdx.x, wave = tid / 64;
  const int kg = tid / kColumns, c = tid % kColumns;
  const int column = tile * kColumns + c;
  const bool column_ok = column < a.vd;
  const int channels = 2 * a.kh * a.kd + a.vh * a.vd;
  const size_t stride = static_cast<size_t>(a.vh) * a.kd * a.vd;
  const float norm_scale = sqrtf(static_cast<float>(a.kd));
  float dm[kRows];
  // S_{t+1} of a token is S_t of the token processed just before it, and S_t is
  // requested one token ahead: no load of a state is waited for inside a token.
  float after[kRows], before[kRows];
#pragma unroll
  for (int r = 0; r < kRows; ++r) {
    dm[r] = 0.0f;
    const int row = kg * kRows + r;
    const bool ok = row < a.kd && column_ok;
    const size_t at = (static_cast<size_t>(head) * a.kd + row) * a.vd + column;
    after[r] = ok ? a.states[a.length * stride + at] : 0.0f;
    before[r] = ok ? a.states[(a.length - 1) * stride + at] : 0.0f;
  }
  TokenInputs next = fetch_token(a, a.length - 1, head, key_head, column, column_ok, true);
  for (int t = a.length - 1; t >= 0; --t) {
    const TokenInputs in = next;
    if (t > 0) next = fetch_token(a, t - 1, head, key_head, column, column_ok, true);
    publish_token_qk(in, raw_q, raw_k, inverses);
    float ahead[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int row = kg * kRows + r;
      const bool ok = row < a.kd && column_ok && t > 0;
      ahead[r] = ok ? a.states[(t - 1) * stride + (static_cast<size_t>(head) * a.kd + row) * a.vd + column]
                    : 0.0f;
    }
    __syncthreads();
    const TokenScalars s = token_scalars(a, in, head);
    const float iq = inverses[0], ik = inverses[1];
    float previous[kRows], decayed[kRows], q[kRows], k[kRows];
    float prediction = 0.0f;
    const float dy = in.dy;
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int row = kg * kRows + r;
      previous[r] = before[r];
      const float matrix = after[r];
      q[r] = raw_q[row] * iq / norm_scale;
      k[r] = raw_k[row] * ik;
      decayed[r] = previous[r] * s.decay;
      prediction += decayed[r] * k[r];
      // dq[row] = sum over columns of S_{t+1}[row, column] dy[column]
      q_products[row][c] = matrix * dy;
      dm[r] += q[r] * dy;
    }
    prediction = column_total(prediction, scratch, kg, c);
    if (tid < kMaxKey) {
      float sum = 0.0f;
#pragma unroll
      for (int j = 0; j < kColumns; ++j) sum += q_products[tid][j];
      dq_rows[tid] = sum;
    }
    const float difference = in.v - prediction;
    const float delta = difference * s.beta;
    float ddelta = 0.0f;
#pragma unroll
    for (int r = 0; r < kRows; ++r) ddelta += dm[r] * k[r];
    ddelta = column_total(ddelta, scratch, kg, c);
    const float dv = ddelta * s.beta;
    if (kg == 0 && column_ok)
      a.dpost[1LL * t * channels + 2 * a.kh * a.kd + head * a.vd + column] = dv;
    float dg = 0.0f;
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
      const int row = kg * kRows + r;
      k_products[row][c] = dm[r] * delta - decayed[r] * dv;
      const float ddecayed = dm[r] - k[r] * dv;
      dg += ddecayed * previous[r];
      dm[r] = ddecayed * s.decay;
      after[r] = before[r];
      before[r] = ahead[r];
    }
    // workgroup sums: dg over every element, d beta over the columns
    float db_partial = kg == 0 ? ddelta * difference : 0.0f;
    dg = wave_sum(dg);
    db_partial = wave_sum(db_partial);
    if (tid % 64 == 0) {
      block_sums[wave][0] = dg;
      block_sums[wave][1] = db_partial;
    }
    __syncthreads();
    if (tid < kMaxKey) {
      float sum = 0.0f;
#pragma unroll
      for (int j = 0; j < kColumns; ++j) sum += k_products[tid][j];
      dk_rows[tid] = sum;
    }
    __syncthreads();
    const long long partial = (1LL * t * a.vh + head) * tiles + tile;
    if (tid < 64) {
      // the two row-space gradients back through the L2 normalisation
      float q_dot = 0.0f, k_dot = 0.0f;
      for (int d = tid; d < kMaxKey; d += 64) {
        q_dot += dq_rows[d] * raw_q[d];
        k_dot += dk_rows[d] * raw_k[d];
      }
      q_dot = wave_sum(q_dot);
      k_dot = wave_sum(k_dot);
      for (int d = tid; d < a.kd; d += 64) {
        a.qk_partials[partial * 2 * a.kd + d] =
            (dq_rows[d] * iq - raw_q[d] * iq * iq * iq * q_dot) / norm_scale;
        a.qk_partials[partial * 2 * a.kd + a.kd + d] =
            dk_rows[d] * ik - raw_k[d] * ik * ik * ik * k_dot;
      }
      if (tid == 0) {
        const float dg_total = (block_sums[0][0] + block_sums[1][0]) + (block_sums[2][0] + block_sums[3][0]);
        const float db_total = (block_sums[0][1] + block_sums[1][1]) + (block_sums[2][1] + block_sums[3][1]);
        a.scalar_partials[partial * 3 + 0] = -dg_total * s.decay * s.rate / (1.0f + expf(-s.alpha));
        a.scalar_partials[partial * 3 + 1] = db_total * s.sigmoid * (1.0f - s.sigmoid);
        a.scalar_partials[partial * 3 + 2] = -dg_total * s.decay * s.rate * s.softplus;
      }
    }
    __syncthreads();
  }
}

// One wave per (token, head) row of value_dim <= 256 channels.
__global__ void __launch_bounds__(64)
output_backward_kernel(const float* core, const uint16_t* z, const float* __restrict__ norm,
                       const float* dy, int vd, float epsilon, bool round, float* dcore,
                       float* dz, float* norm_partials) {
  const long long row = blockIdx.x;
  const int lane = threadIdx.x;
  float x[4], dn[4], gate[4], sigmoid[4], grad[4];
  float squares = 0.0f, dot = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = lane + 64 * j;
    x[j] = dn[j] = gate[j] = sigmoid[j] = grad[j] = 0.0f;
    if (c < vd) {
      x[j] = core[row * vd + c];
      gate[j] = bf16_bits_to_float(z[row * vd + c]);
      sigmoid[j] = 1.0f / (1.0f + expf(-gate[j]));
      grad[j] = dy[row * vd + c];
      dn[j] = grad[j] * gate[j] * sigmoid[j] * norm[c];
    }
    squares += x[j] * x[j];
    dot += dn[j] * x[j];
  }
  squares = wave_sum(squares);
  dot = wave_sum(dot);
  const float inverse = rsqrtf(squares / static_cast<float>(vd) + epsilon);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = lane + 64 * j;
    if (c >= vd) continue;
    const float normalized = round_if(x[j] * inverse, round);
    const float affine = round_if(normalized * norm[c], round);
    dcore[row * vd + c] = inverse * dn[j] - x[j] * inverse * inverse * inverse / static_cast<float>(vd) * dot;
    dz[row * vd + c] = grad[j] * affine * sigmoid[j] * (1.0f + gate[j] * (1.0f - sigmoid[j]));
    if (norm_partials) norm_partials[row * vd + c] = grad[j] * gate[j] * sigmoid[j] * normalized;
  }
}

// Heads of a key head and their column tiles add up, in ascending order.
__global__ void __launch_bounds__(128)
gather_qk_kernel(const float* partials, int kh, int vh, int kd, int tiles, int channels,
                 float* dpost) {
  const int key_head = blockIdx.x, t = blockIdx.y, d = threadIdx.x;
  if (d >= kd) return;
  const int group = vh / kh;
  float dq = 0.0f, dk = 0.0f;
  for (int h = key_head * group; h < (key_head + 1) * group; ++h)
    for (int tile = 0; tile < tiles; ++tile) {
      const long long at = ((1LL * t * vh + h) * tiles + tile) * 2 * kd;
      dq += partials[at + d];
      dk += partials[at + kd + d];
    }
  dpost[1LL * t * channels + key_head * kd + d] = dq;
  dpost[1LL * t * channels + (kh + key_head) * kd + d] = dk;
}

// da, db per token; the two per-head parameter gradients summed over the
// sequence by one workgroup per head in a fixed order.
__global__ void __launch_bounds__(256)
gather_scalar_kernel(const float* partials, int length, int vh, int tiles, float* da, float* db,
                     float* da_log, float* ddt_bias) {
  __shared__ float sums[256][2];
  const int head = blockIdx.x, tid = threadIdx.x;
  float log_sum = 0.0f, bias_sum = 0.0f;
  for (int t = tid; t < length; t += 256) {
    float ga = 0.0f, gb = 0.0f, glog = 0.0f;
    for (int tile = 0; tile < tiles; ++tile) {
      const long long at = ((1LL * t * vh + head) * tiles + tile) * 3;
      ga += partials[at];
      gb += partials[at + 1];
      glog += partials[at + 2];
    }
    da[1LL * t * vh + head] = ga;
    db[1LL * t * vh + head] = gb;
    log_sum += glog;
    bias_sum += ga;
  }
  sums[tid][0] = log_sum;
  sums[tid][1] = bias_sum;
  __syncthreads();
  for (int width = 128; width > 0; width >>= 1) {
    if (tid < width) {
      sums[tid][0] += sums[tid + width][0];
      sums[tid][1] += sums[tid + width][1];
    }
    __syncthreads();
  }
  if (tid == 0) {
    if (da_log) da_log[head] += sums[0][0];
    if (ddt_bias) ddt_bias[head] += sums[0][1];
  }
}

template <int VEC>
__global__ void __launch_bounds__(256)
conv_silu_backward_kernel(const float* pre, const float* dpost, long long elements, float* dpre) {
  const long long i = (blockIdx.x * 256LL + threadIdx.x) * VEC;
  if (i >= elements) return;
  const Pack<VEC> x = load_floats<VEC>(pre + i), g = load_floats<VEC>(dpost + i);
  Pack<VEC> r;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    const float sigmoid = 1.0f / (1.0f + expf(-x.e[e]));
    r.e[e] = g.e[e] * sigmoid * (1.0f + x.e[e] * (1.0f - sigmoid));
  }
  store_floats<VEC>(dpre + i, r);
}

template <int VEC>
__global__ void __launch_bounds__(256)
conv_input_backward_kernel(const float* dpre, const float* __restrict__ weight, int length,
                           int channels, int kernel, float* dx) {
  const int groups = channels / VEC;
  const long long i = blockIdx.x * 256LL + threadIdx.x;
  if (i >= 1LL * length * groups) return;
  const int c = static_cast<int>(i % groups) * VEC, t = static_cast<int>(i / groups);
  Pack<VEC> sum;
#pragma unroll
  for (int e = 0; e < VEC; ++e) sum.e[e] = 0.0f;
  for (int tap = 0; tap < kernel; ++tap) {
    const int future = t + kernel - 1 - tap;
    if (future >= length) continue;
    const Pack<VEC> g = load_floats<VEC>(dpre + 1LL * future * channels + c);
#pragma unroll
    for (int e = 0; e < VEC; ++e) sum.e[e] += g.e[e] * weight[1LL * (c + e) * kernel + tap];
  }
  store_floats<VEC>(dx + 1LL * t * channels + c, sum);
}

// dw[c, tap] += sum over t of dpre[t, c] x[t + tap - kernel + 1, c], in two
// levels with a fixed order: blockIdx.z sums one slice of the tokens.
__global__ void __launch_bounds__(256)
conv_weight_partial_kernel(const uint16_t* input, const float* dpre, int length, int channels,
                           int kernel, int slices, float* partial) {
  const int c = blockIdx.x * 256 + threadIdx.x, tap = blockIdx.y, slice = blockIdx.z;
  if (c >= channels) return;
  const int per = (length + slices - 1) / slices;
  const int first = max(slice * per, kernel - 1 - tap), last = min((slice + 1) * per, length);
  float sum = 0.0f;
  for (int t = first; t < last; ++t)
    sum += dpre[1LL * t * channels + c] *
           bf16_bits_to_float(input[1LL * (t + tap - kernel + 1) * channels + c]);
  partial[(1LL * slice * channels + c) * kernel + tap] = sum;
}

__global__ void __launch_bounds__(256)
conv_weight_final_kernel(const float* partial, long long elements, int slices, float* dw) {
  const long long i = blockIdx.x * 256LL + threadIdx.x;
  if (i >= elements) return;
  float sum = 0.0f;
  for (int slice = 0; slice < slices; ++slice) sum += partial[slice * elements + i];
  dw[i] += sum;
}

// gradient[c] += sum over rows of partials[row, c], two levels, fixed order.
// Sum of rows first..last-1 of a [rows, width] matrix (width <= 256), per
// column.  The 256 threads form up to 8 groups of `width`; group g takes rows
// first + g, first + g + groups, ...; the groups' sums are added in ascending
// order.  Returns the column's total in the threads of group 0.
__device__ inline float sum_block_rows(const float* parts, long long first, long long last,
                                       int width) {
  __shared__ float scratch[8][256];
  const int fit = 256 / width, groups = fit < 8 ? fit : 8;
  const int c = threadIdx.x % width, g = threadIdx.x / width;
  if (g < groups) {
    float sum = 0.0f;
#pragma unroll 8
    for (long long row = first + g; row < last; row += groups) sum += parts[row * width + c];
    scratch[g][c] = sum;
  }
  __syncthreads();
  float total = 0.0f;
  if (g == 0)
    for (int j = 0; j < groups; ++j) total += scratch[j][c];
  return total;
}

__global__ void __launch_bounds__(256)
sum_rows_partial_kernel(const float* parts, long long rows, int width, int chunks, float* partial) {
  const long long per = (rows + chunks - 1) / chunks;
  const long long first = blockIdx.x * per;
  const long long last = first + per < rows ? first + per : rows;
  const float total = sum_block_rows(parts, first, last, width);
  if (threadIdx.x < width) partial[1LL * blockIdx.x * width + threadIdx.x] = total;
}

__global__ void __launch_bounds__(256)
sum_rows_final_kernel(const float* partial, int chunks, int width, float* gradient) {
  const float total = sum_block_rows(partial, 0, chunks, width);
  if (threadIdx.x < width) gradient[threadIdx.x] += total;
}

unsigned blocks_for(long long elements) { return static_cast<unsigned>((elements + 255) / 256); }

}  // namespace

bool force_generic();  // mha_capi.hip

namespace {
bool use_chunks(const pluto_hip_delta_params* p) {
  return !force_generic() && gdn_backward_chunked_supported(p);
}
}  // namespace

size_t gdn_backward_workspace_bytes(const pluto_hip_delta_params* p, int length, bool norm_grad) {
  const size_t T = static_cast<size_t>(length);
  const size_t kh = p->key_heads, vh = p->value_heads, kd = p->key_head_dim, vd = p->value_head_dim;
  const size_t channels = 2 * kh * kd + vh * vd;
  const bool chunked = use_chunks(p);
  const size_t tiles = chunked ? 1 : (vd + kColumns - 1) / kColumns;
  size_t bytes = 0;
  bytes += 4 * align_up(T * channels * 4, 256);          // pre, post, dpost, dpre
  bytes += 2 * align_up(T * vh * vd * 4, 256);           // core, dcore
  bytes += chunked ? gdn_backward_chunked_bytes(p, length)
                   : align_up((T + 1) * vh * kd * vd * 4, 256);  // states
  bytes += align_up(T * vh * tiles * 2 * kd * 4, 256);   // q/k partials
  bytes += align_up(T * vh * tiles * 3 * 4, 256);        // scalar partials
  if (norm_grad) bytes += align_up(T * vh * vd * 4, 256) + align_up(kGdnSumChunks * vd * 4, 256);
  bytes += align_up(kConvSlices * channels * p->conv_kernel_dim * 4, 256);  // conv weight partials
  return bytes;
}

int launch_gdn_backward(hipStream_t stream, const pluto_hip_delta_params* p, int length,
                        const void* qkv, const void* z, const void* a, const void* b,
                        const float* conv_weight, const float* a_log, const float* dt_bias,
                        const float* norm, const float* dy, float* dqkv, float* dz, float* da,
                        float* db, float* d_conv_weight, float* d_a_log, float* d_dt_bias,
                        float* d_norm, void* workspace) {
  note_path(use_chunks(p) ? PLUTO_HIP_PATH_CHUNKED : PLUTO_HIP_PATH_RECURRENCE);
  const size_t T = static_cast<size_t>(length);
  const int kh = p->key_heads, vh = p->value_heads, kd = p->key_head_dim, vd = p->value_head_dim;
  const int channels = 2 * kh * kd + vh * vd, kernel = p->conv_kernel_dim;
  const bool chunked = use_chunks(p);
  const int tiles = chunked ? 1 : (vd + kColumns - 1) / kColumns;
  const bool round = p->round_to_bfloat16 != 0;
  char* at = static_cast<char*>(workspace);
  auto take = [&](size_t bytes) {
    char* result = at;
    at += align_up(bytes, 256);
    return reinterpret_cast<float*>(result);
  };
  float* pre = take(T * channels * 4);
  float* post = take(T * channels * 4);
  float* dpost = take(T * channels * 4);
  float* dpre = take(T * channels * 4);
  float* core = take(T * vh * vd * 4);
  float* dcore = take(T * vh * vd * 4);
  float* states = take(chunked ? gdn_backward_chunked_bytes(p, length) : (T + 1) * vh * kd * vd * 4);
  float* qk_partials = take(T * vh * tiles * 2 * kd * 4);
  float* scalar_partials = take(T * vh * tiles * 3 * 4);
  float* norm_partials = d_norm ? take(T * vh * vd * 4) : nullptr;
  float* norm_chunks = d_norm ? take(static_cast<size_t>(kGdnSumChunks) * vd * 4) : nullptr;
  float* conv_partials = take(static_cast<size_t>(kConvSlices) * channels * kernel * 4);

  const long long elements = 1LL * length * channels;
  // one channel a thread: four a thread (one wide access instead of four) was
  // measured slower for the two kernels that also read the weights
  conv_train_kernel<1><<<blocks_for(elements), 256, 0, stream>>>(
      static_cast<const uint16_t*>(qkv), conv_weight, length, channels, kernel, round, pre, post);
  int status = launch_status();
  if (status != 0) return status;
  RecurrenceArgs r;
  r.post = post;
  r.a = static_cast<const uint16_t*>(a);
  r.b = static_cast<const uint16_t*>(b);
  r.a_log = a_log;
  r.dt_bias = dt_bias;
  r.states = states;
  r.core = core;
  r.dcore = dcore;
  r.qk_partials = qk_partials;
  r.scalar_partials = scalar_partials;
  r.dpost = dpost;
  r.length = length;
  r.kh = kh;
  r.vh = vh;
  r.kd = kd;
  r.vd = vd;
  r.round = round;
  GdnChunkedBackward c;
  c.post = post;
  c.a = r.a;
  c.b = r.b;
  c.a_log = a_log;
  c.dt_bias = dt_bias;
  c.dcore = dcore;
  c.core = core;
  c.dpost = dpost;
  c.qk_partials = qk_partials;
  c.scalar_partials = scalar_partials;
  c.records = states;
  c.length = length;
  c.key_heads = kh;
  c.value_heads = vh;
  c.round = round;
  if (chunked) {
    status = launch_gdn_backward_chunked_forward(stream, c);
  } else {
    recurrence_states_kernel<<<vh * tiles, 256, 0, stream>>>(r);
    status = launch_status();
  }
  if (status != 0) return status;
  output_backward_kernel<<<static_cast<unsigned>(length) * vh, 64, 0, stream>>>(
      core, static_cast<const uint16_t*>(z), norm, dy, vd, p->rms_norm_epsilon, round, dcore, dz,
      norm_partials);
  status = launch_status();
  if (status != 0) return status;
  if (d_norm) {
    sum_rows_partial_kernel<<<kGdnSumChunks, 256, 0, stream>>>(norm_partials, 1LL * length * vh, vd,
                                                               kGdnSumChunks, norm_chunks);
    sum_rows_final_kernel<<<1, 256, 0, stream>>>(norm_chunks, kGdnSumChunks, vd, d_norm);
    status = launch_status();
    if (status != 0) return status;
  }
  if (chunked) {
    status = launch_gdn_backward_chunked_reverse(stream, c);
  } else {
    recurrence_backward_kernel<<<vh * tiles, 256, 0, stream>>>(r);
    status = launch_status();
  }
  if (status != 0) return status;
  gather_qk_kernel<<<dim3(kh, length), 128, 0, stream>>>(qk_partials, kh, vh, kd, tiles, channels,
                                                         dpost);
  gather_scalar_kernel<<<vh, 256, 0, stream>>>(scalar_partials, length, vh, tiles, da, db, d_a_log,
                                               d_dt_bias);
  if (elements % 4 == 0)
    conv_silu_backward_kernel<4><<<blocks_for(elements / 4), 256, 0, stream>>>(pre, dpost, elements,
                                                                               dpre);
  else
    conv_silu_backward_kernel<1><<<blocks_for(elements), 256, 0, stream>>>(pre, dpost, elements,
                                                                           dpre);
  conv_input_backward_kernel<1><<<blocks_for(elements), 256, 0, stream>>>(
      dpre, conv_weight, length, channels, kernel, dqkv);
  if (d_conv_weight) {
    conv_weight_partial_kernel<<<dim3((channels + 255) / 256, kernel, kConvSlices), 256, 0, stream>>>(
        static_cast<const uint16_t*>(qkv), dpre, length, channels, kernel, kConvSlices,
        conv_partials);
    const long long weights = 1LL * channels * kernel;
    conv_weight_final_kernel<<<blocks_for(weights), 256, 0, stream>>>(conv_partials, weights,
                                                                      kConvSlices, d_conv_weight);
  }
  return launch_status();
}

}  // namespace pluto_hip
