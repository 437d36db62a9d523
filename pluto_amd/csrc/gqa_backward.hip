// Backward of the whole-sequence Qwen GQA layer
// (QwenAttentionLayer::SequenceBackward, src/llm/layers/qwen_attention.cc:
// 450-499 and its kernels :124-239), without the reference's two quadratic
// buffers (saved probabilities and score gradients).
//
// The attention core of the backward is the multi-head kernel pair of this
// library run on a packed [T, 3 * qh * d] view in which every query head
// carries a copy of its kv head's K and V rows; the dK and dV of the copies
// are then summed per kv head in ascending head order.  Around it:
//   gate_backward_kernel        GateBackwardKernel        (:124-141)
//   pack_heads_kernel           layout only
//   norm_rope_backward_kernel   NormBackwardKernel        (:201-228), fused with
//                               the per-kv-head sums
//   reduce_norm_*_kernel        ReduceNormKernel          (:230-239), two
//                               levels, fixed order
#include "gqa.h"

namespace pluto_hip {
namespace {

// [T, qh, d] prepared queries, [T, kh, d] prepared keys and values ->
// packed [T, 3E] (E = qh * d): Q | K of the head's kv head | V of it.  Moved in
// pieces of PIECE elements (16 bytes when the head width allows).
template <typename Element, int PIECE>
__global__ void __launch_bounds__(256)
pack_heads_kernel(const Element* q, const Element* k, const Element* v, int length, int qh,
                  int kh, int d, Element* packed) {
  struct alignas(sizeof(Element) * PIECE) Piece {
    Element e[PIECE];
  };
  const int pieces_per_head = d / PIECE;
  const long long pieces_per_part = 1LL * qh * pieces_per_head;
  const long long total = 3LL * length * pieces_per_part;
  const int group = qh / kh;
  for (long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += 256LL * gridDim.x) {
    const long long t = i / (3 * pieces_per_part);
    const long long within = i % (3 * pieces_per_part);
    const int part = static_cast<int>(within / pieces_per_part);
    const int h = static_cast<int>((within % pieces_per_part) / pieces_per_head);
    const int c = static_cast<int>(within % pieces_per_head) * PIECE;
    const Element* source = part == 0 ? q + (t * qh + h) * d + c
                                      : (part == 1 ? k : v) + (t * kh + h / group) * d + c;
    *reinterpret_cast<Piece*>(packed + i * PIECE) = *reinterpret_cast<const Piece*>(source);
  }
}

// dC = dy * Round(sigmoid(gate)); d gate = dy * Round(core) * s (1 - s).
__global__ void __launch_bounds__(256)
gate_backward_kernel(const uint16_t* qg, const void* core, int core_dtype, const float* dy,
                     long long elements, int d, bool round, float* dc, float* dqg) {
  for (long long i = blockIdx.x * 256LL + threadIdx.x; i < elements; i += 256LL * gridDim.x) {
    const long long unit = i / d;  // (row, head)
    const int c = static_cast<int>(i % d);
    const float gate = bf16_bits_to_float(qg[(unit * 2 + 1) * d + c]);
    const float sigmoid = 1.0f / (1.0f + expf(-gate));
    const float grad = dy[i];
    float value = load_element(core, i, core_dtype);
    if (round) value = round_to_bf16(value);
    dc[i] = grad * (round ? round_to_bf16(sigmoid) : sigmoid);
    dqg[(unit * 2 + 1) * d + c] = grad * value * sigmoid * (1.0f - sigmoid);
  }
}

struct NormBackwardArgs {
  const uint16_t* input = nullptr;  // raw bf16 rows, `input_stride` apart
  const float* weight = nullptr;    // zero-centred norm weight [d]
  const float* packed_grad = nullptr;  // fp32 [T, 3E]
  const float* cosines = nullptr;      // [T, rotary/2]
  const float* sines = nullptr;
  float* dx = nullptr;        // rows `input_stride` apart
  float* dv = nullptr;        // key mode: [T, kh, d]
  float* parts = nullptr;     // optional [T * heads, d]
  int length = 0, heads = 0, d = 0, rotary = 0, input_stride = 0;
  int query_heads = 0, group = 0;
  bool key_mode = false;
  float epsilon = 1e-6f;
};

// One wave per (row, head).  Query mode: the gradient of head h is its slice
// of the packed dQ.  Key mode: the gradients of the kv head's `group` copies
// are summed in ascending head order, for dK (which continues through RoPE and
// the norm) and for dV (which is final).
__global__ void __launch_bounds__(64)
norm_rope_backward_kernel(NormBackwardArgs a) {
  __shared__ float grads[256];
  const int lane = threadIdx.x;
  const int unit = blockIdx.x, row = unit / a.heads, head = unit % a.heads;
  const int d = a.d;
  const long long E = 1LL * a.query_heads * d;
  const float* packed_row = a.packed_grad + 3 * E * row;
  float x[4], g[4];
  float sum_squares = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = lane + 64 * j;
    x[j] = 0.0f;
    g[j] = 0.0f;
    if (c < d) {
      x[j] = bf16_bits_to_float(a.input[1LL * unit * a.input_stride + c]);
      if (!a.key_mode) {
        g[j] = packed_row[head * d + c];
      } else {
        float key_sum = 0.0f, value_sum = 0.0f;
        for (int copy = 0; copy < a.group; ++copy) {
          const int h = head * a.group + copy;
          key_sum += packed_row[E + h * d + c];
          value_sum += packed_row[2 * E + h * d + c];
        }
        g[j] = key_sum;
        a.dv[1LL * unit * d + c] = value_sum;
      }
      grads[c] = g[j];
    }
    sum_squares += x[j] * x[j];
  }
  __syncthreads();
  sum_squares = wave_sum(sum_squares);
  const float inv = rsqrtf(sum_squares / static_cast<float>(d) + a.epsilon);
  const int half = a.rotary / 2;
  float normalized[4], weighted[4];
  float dot = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = lane + 64 * j;
    normalized[j] = 0.0f;
    weighted[j] = 0.0f;
    if (c < d) {
      float ng = g[j];
      if (c < a.rotary) {
        const int frequency = c < half ? c : c - half;
        const float co = a.cosines[1LL * row * half + frequency];
        const float si = a.sines[1LL * row * half + frequency];
        const float partner = grads[c < half ? c + half : c - half];
        ng = g[j] * co + (c < half ? partner * si : -partner * si);
      }
      normalized[j] = ng;
      weighted[j] = ng * (1.0f + a.weight[c]);
      dot += weighted[j] * x[j];
    }
  }
  dot = wave_sum(dot);
  const float cubic = inv * inv * inv / static_cast<float>(d);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = lane + 64 * j;
    if (c < d) {
      a.dx[1LL * unit * a.input_stride + c] = inv * weighted[j] - x[j] * cubic * dot;
      if (a.parts) a.parts[1LL * unit * d + c] = normalized[j] * x[j] * inv;
    }
  }
}

// dw[c] += sum over rows of parts[row, c], in two levels with a fixed order.
__global__ void __launch_bounds__(256)
reduce_norm_partial_kernel(const float* parts, long long rows, int d, int chunks, float* partial) {
  const int c = threadIdx.x;
  if (c >= d) return;
  const long long per = (rows + chunks - 1) / chunks;
  const long long first = blockIdx.x * per;
  const long long last = first + per < rows ? first + per : rows;
  float sum = 0.0f;
  for (long long row = first; row < last; ++row) sum += parts[row * d + c];
  partial[1LL * blockIdx.x * d + c] = sum;
}

__global__ void __launch_bounds__(256)
reduce_norm_final_kernel(const float* partial, int chunks, int d, float* dw) {
  const int c = threadIdx.x;
  if (c >= d) return;
  float sum = 0.0f;
  for (int chunk = 0; chunk < chunks; ++chunk) sum += partial[1LL * chunk * d + c];
  dw[c] += sum;
}

int grid_for(long long elements) {
  const long long blocks = (elements + 255) / 256;
  return static_cast<int>(blocks < 65536 ? blocks : 65536);
}

}  // namespace

int launch_pack_heads(hipStream_t stream, const void* q, const void* k, const void* v, int dtype,
                      int length, int qh, int kh, int d, void* packed) {
  const long long elements = 3LL * length * qh * d;
  if (dtype == PLUTO_HIP_BF16) {
    auto* qs = static_cast<const uint16_t*>(q);
    auto* ks = static_cast<const uint16_t*>(k);
    auto* vs = static_cast<const uint16_t*>(v);
    auto* out = static_cast<uint16_t*>(packed);
    if (d % 8 == 0)
      pack_heads_kernel<uint16_t, 8><<<grid_for(elements / 8), 256, 0, stream>>>(qs, ks, vs, length,
                                                                                 qh, kh, d, out);
    else
      pack_heads_kernel<uint16_t, 1><<<grid_for(elements), 256, 0, stream>>>(qs, ks, vs, length, qh,
                                                                             kh, d, out);
  } else {
    auto* qs = static_cast<const float*>(q);
    auto* ks = static_cast<const float*>(k);
    auto* vs = static_cast<const float*>(v);
    auto* out = static_cast<float*>(packed);
    if (d % 4 == 0)
      pack_heads_kernel<float, 4><<<grid_for(elements / 4), 256, 0, stream>>>(qs, ks, vs, length, qh,
                                                                              kh, d, out);
    else
      pack_heads_kernel<float, 1><<<grid_for(elements), 256, 0, stream>>>(qs, ks, vs, length, qh, kh,
                                                                          d, out);
  }
  return launch_status();
}

int launch_gate_backward(hipStream_t stream, const void* qg, const void* core, int core_dtype,
                         const float* dy, int length, int qh, int d, bool round, float* dc,
                         float* dqg) {
  const long long elements = 1LL * length * qh * d;
  gate_backward_kernel<<<grid_for(elements), 256, 0, stream>>>(
      static_cast<const uint16_t*>(qg), core, core_dtype, dy, elements, d, round, dc, dqg);
  return launch_status();
}

int launch_norm_rope_backward(hipStream_t stream, const void* input, const float* weight,
                              const float* packed_grad, const float* cosines, const float* sines,
                              int length, int heads, int query_heads, int d, int rotary,
                              int input_stride, float epsilon, bool key_mode, float* dx,
                              float* dv, float* parts) {
  NormBackwardArgs a;
  a.input = static_cast<const uint16_t*>(input);
  a.weight = weight;
  a.packed_grad = packed_grad;
  a.cosines = cosines;
  a.sines = sines;
  a.dx = dx;
  a.dv = dv;
  a.parts = parts;
  a.length = length;
  a.heads = heads;
  a.d = d;
  a.rotary = rotary;
  a.input_stride = input_stride;
  a.query_heads = query_heads;
  a.group = query_heads / (key_mode ? heads : query_heads);
  a.key_mode = key_mode;
  a.epsilon = epsilon;
  norm_rope_backward_kernel<<<static_cast<unsigned>(length) * heads, 64, 0, stream>>>(a);
  return launch_status();
}

int launch_reduce_norm(hipStream_t stream, const float* parts, long long rows, int d,
                       float* partial, int chunks, float* dw) {
  reduce_norm_partial_kernel<<<chunks, 256, 0, stream>>>(parts, rows, d, chunks, partial);
  int status = launch_status();
  if (status != 0) return status;
  reduce_norm_final_kernel<<<1, 256, 0, stream>>>(partial, chunks, d, dw);
  return launch_status();
}

}  // namespace pluto_hip
