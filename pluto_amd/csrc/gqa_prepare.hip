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
#include "gqa_rotate.h"
#include "mfma_tile.h"

namespace pluto_hip {
namespace {

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

// Vectorised form of the same preparation for bf16 inputs, a bf16 query buffer
// and a bf16 cache with rounding on: a thread owns 8 consecutive channels (one
// 16-byte load and store), the D/8 threads of a (row, head) are neighbouring
// lanes.  Requires rotary_dim/2 to be a multiple of 8 so that a thread's RoPE
// partners all sit in one other thread.  Arithmetic and rounding points are
// those of normalize_rotate above.
template <int D>
__global__ void __launch_bounds__(256)
prefill_prepare_bf16_kernel(PrefillPrepareArgs a) {
  constexpr int LANES = D / 8;
  const int heads = a.query_heads + a.key_value_heads;
  const long long thread = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  const long long unit = thread / LANES;
  if (unit >= static_cast<long long>(a.length) * heads) return;  // whole groups drop out
  const int chunk = static_cast<int>(thread % LANES);
  const int row = static_cast<int>(unit / heads);
  const int head = static_cast<int>(unit % heads);
  const int half = a.rotary_dim / 2;
  const bool is_query = head < a.query_heads;
  const int kv = head - a.query_heads;
  const uint16_t* in;
  uint16_t* out;
  const float* weight;
  if (is_query) {
    in = static_cast<const uint16_t*>(a.qg) +
         (static_cast<long long>(row) * a.query_heads + head) * 2 * D;
    out = static_cast<uint16_t*>(a.q_out) + (static_cast<long long>(row) * a.query_heads + head) * D;
    weight = a.q_norm;
  } else {
    in = static_cast<const uint16_t*>(a.k) +
         (static_cast<long long>(row) * a.key_value_heads + kv) * D;
    out = static_cast<uint16_t*>(a.cache.keys) +
          static_cast<long long>(a.start_position + row) * a.cache.token_stride +
          kv * a.cache.head_stride;
    weight = a.k_norm;
  }
  const uint4 bits = *reinterpret_cast<const uint4*>(in + 8 * chunk);
  const uint32_t words[4] = {bits.x, bits.y, bits.z, bits.w};
  float x[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x[2 * i] = __uint_as_float(words[i] << 16);
    x[2 * i + 1] = __uint_as_float(words[i] & 0xffff0000u);
  }
  double square = 0.0;
#pragma unroll
  for (int e = 0; e < 8; ++e) square += static_cast<double>(x[e] * x[e]);
#pragma unroll
  for (int offset = 1; offset < LANES; offset <<= 1) square += __shfl_xor(square, offset, 64);
  const double inverse = 1.0 / sqrt(square / D + static_cast<double>(a.epsilon));
  const float4 w0 = *reinterpret_cast<const float4*>(weight + 8 * chunk);
  const float4 w1 = *reinterpret_cast<const float4*>(weight + 8 * chunk + 4);
  const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
  // Rounding to bf16 is the hardware's conversion (round to nearest even, two
  // values an instruction); a rounded pair stays packed until its values are
  // needed again as floats.
  uint32_t normalized[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    normalized[i] = pack_bf16(
        static_cast<float>(x[2 * i] * inverse * (1.0 + static_cast<double>(w[2 * i]))),
        static_cast<float>(x[2 * i + 1] * inverse * (1.0 + static_cast<double>(w[2 * i + 1]))));
  // RoPE partner channels c +- half live `half / 8` lanes away: four packed
  // words travel instead of eight floats.
  const int first = 8 * chunk;
  const bool rotated = first < a.rotary_dim;
  const bool lower = first < half;
  const int lane = threadIdx.x % 64;
  const int partner_lane = rotated ? (lower ? lane + half / 8 : lane - half / 8) : lane;
  uint32_t partner[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) partner[i] = __shfl(normalized[i], partner_lane, 64);
  uint32_t result[4] = {normalized[0], normalized[1], normalized[2], normalized[3]};
  if (rotated) {
    const long long table = static_cast<long long>(row) * half + (lower ? first : first - half);
    const float4 c0 = *reinterpret_cast<const float4*>(a.cosines + table);
    const float4 c1 = *reinterpret_cast<const float4*>(a.cosines + table + 4);
    const float4 s0 = *reinterpret_cast<const float4*>(a.sines + table);
    const float4 s1 = *reinterpret_cast<const float4*>(a.sines + table + 4);
    const float cosine[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    const float sine[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float n0 = __uint_as_float(normalized[i] << 16);
      const float n1 = __uint_as_float(normalized[i] & 0xffff0000u);
      const float p0 = __uint_as_float(partner[i] << 16);
      const float p1 = __uint_as_float(partner[i] & 0xffff0000u);
      const uint32_t own = pack_bf16(n0 * cosine[2 * i], n1 * cosine[2 * i + 1]);
      const uint32_t other = pack_bf16(p0 * sine[2 * i], p1 * sine[2 * i + 1]);
      const float a0 = __uint_as_float(own << 16), a1 = __uint_as_float(own & 0xffff0000u);
      const float b0 = __uint_as_float(other << 16), b1 = __uint_as_float(other & 0xffff0000u);
      result[i] = lower ? pack_bf16(a0 - b0, a1 - b1) : pack_bf16(a0 + b0, a1 + b1);
    }
  }
  *reinterpret_cast<uint4*>(out + 8 * chunk) = make_uint4(result[0], result[1], result[2], result[3]);
  if (!is_query) {
    const uint16_t* v_in = static_cast<const uint16_t*>(a.v) +
                           (static_cast<long long>(row) * a.key_value_heads + kv) * D;
    uint16_t* v_out = static_cast<uint16_t*>(a.cache.values) +
                      static_cast<long long>(a.start_position + row) * a.cache.token_stride +
                      kv * a.cache.head_stride;
    *reinterpret_cast<uint4*>(v_out + 8 * chunk) = *reinterpret_cast<const uint4*>(v_in + 8 * chunk);
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
  const int seq = batch.sequence[b];
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
  if (!kernel_enabled(kAuxiliaryKernel)) return 0;
  rope_table_kernel<<<static_cast<unsigned>((count + 255) / 256), 256, 0, stream>>>(
      start_position, length, rotary_dim, theta, round, cosines, sines);
  return launch_status();
}

int launch_prefill_prepare(hipStream_t stream, const PrefillPrepareArgs& a) {
  const long long units =
      static_cast<long long>(a.length) * (a.query_heads + a.key_value_heads);
  const int d = a.head_dim;
  if (!kernel_enabled(kAuxiliaryKernel)) return 0;
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  const bool vectorised =
      a.round && a.q_out_dtype == PLUTO_HIP_BF16 && a.cache.dtype == PLUTO_HIP_BF16 &&
      (d == 64 || d == 128 || d == 256) && (a.rotary_dim / 2) % 8 == 0 &&
      a.cache.token_stride % 8 == 0 && a.cache.head_stride % 8 == 0 && aligned(a.qg) &&
      aligned(a.k) && aligned(a.v) && aligned(a.q_out) && aligned(a.cache.keys) &&
      aligned(a.cache.values) && aligned(a.q_norm) && aligned(a.k_norm) && aligned(a.cosines) &&
      aligned(a.sines);
  if (vectorised) {
    const long long threads = units * (d / 8);
    const unsigned blocks = static_cast<unsigned>((threads + 255) / 256);
    if (d == 64)
      prefill_prepare_bf16_kernel<64><<<blocks, 256, 0, stream>>>(a);
    else if (d == 128)
      prefill_prepare_bf16_kernel<128><<<blocks, 256, 0, stream>>>(a);
    else
      prefill_prepare_bf16_kernel<256><<<blocks, 256, 0, stream>>>(a);
    return launch_status();
  }
  prefill_prepare_kernel<<<static_cast<unsigned>((units + 3) / 4), 256, 0, stream>>>(a);
  return launch_status();
}

int launch_decode_prepare(hipStream_t stream, const DecodePrepareArgs& a,
                          const DecodeBatch& batch) {
  const long long units =
      static_cast<long long>(batch.count) * (a.query_heads + a.key_value_heads);
  if (!kernel_enabled(kAuxiliaryKernel)) return 0;
  decode_prepare_kernel<<<static_cast<unsigned>((units + 3) / 4), 256, 0, stream>>>(a, batch);
  return launch_status();
}

}  // namespace pluto_hip
