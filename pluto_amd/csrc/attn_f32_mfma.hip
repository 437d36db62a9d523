// Causal attention forward with FP32 storage and FP32 matrix-core arithmetic
// (v_mfma_f32_32x32x2_f32): the reference's FP32 mode of
// FlashAttentionForwardKernel (src/llm/layers/attention.cc:98-170), where
// products and sums stay in FP32.
//
// A workgroup of four waves owns 32 query rows of one (sequence, head); wave w
// walks the visible key tiles (32 keys each) w, w + 4, ... with its own running
// maximum, sum and output, and wave 0 merges the four partial results through
// LDS in wave order.  The FP32 matrix instruction is slow (64 cycles for
// 32x32x2), a row block near the end of a sequence has many tiles and there
// are few row blocks, so splitting the keys is what fills the machine.  As in
// the bf16 kernels the products are transposed,
// S^T = K Q^T and O^T = V^T P^T, so that a lane owns one query column: its row
// maximum and sum are lane-local up to one exchange between the two lane
// halves, and P^T leaves the accumulator in B-operand order.  The contraction
// order of a matrix instruction is free as long as both operands agree:
//   S^T  step j contracts channels (j, j + D/2): lane half h reads the
//        contiguous half row [h D/2, (h+1) D/2) of its key and of its query;
//   O^T  step i contracts keys (8(i/4) + i%4, that + 4): exactly the keys
//        accumulator register i holds in the two lane halves.
#include "attn_generic.h"
#include "mfma_tile.h"

namespace pluto_hip {
namespace {

constexpr int kKeySplit = 4;  // waves per workgroup, each taking every fourth key tile

template <int D>
__global__ void __launch_bounds__(64 * kKeySplit)
f32_forward_kernel(GenericForwardArgs a) {
  constexpr int HALF = D / 2, DB = D / 32;
  __shared__ float part_o[kKeySplit - 1][DB * 16][64];
  __shared__ float part_max[kKeySplit - 1][64], part_sum[kKeySplit - 1][64];
  const int lane = threadIdx.x % 64, h = lane / 32, n = lane % 32;
  const int wave = threadIdx.x / 64;
  const int q0 = blockIdx.x * 32, head = blockIdx.y, seq = blockIdx.z;
  const int kv_head = head / a.group;
  const float* q_base = static_cast<const float*>(a.q.base) + seq * a.q.seq_stride +
                        head * a.q.head_stride;
  const float* k_base = static_cast<const float*>(a.k.base) + seq * a.k.seq_stride +
                        kv_head * a.k.head_stride;
  const float* v_base = static_cast<const float*>(a.v.base) + seq * a.v.seq_stride +
                        kv_head * a.v.head_stride;
  const int query = q0 + n;
  const int query_load = min(query, a.q_rows - 1);
  const float scale2 = a.scale * kLog2e;

  float qf[HALF];
  {
    const float4* row = reinterpret_cast<const float4*>(q_base + query_load * a.q.row_stride + h * HALF);
#pragma unroll
    for (int j = 0; j < HALF / 4; ++j) {
      const float4 piece = row[j];
      qf[4 * j] = piece.x; qf[4 * j + 1] = piece.y; qf[4 * j + 2] = piece.z; qf[4 * j + 3] = piece.w;
    }
  }
  floatx16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.0f;
  float running_max = kMasked, running_sum = 0.0f;  // base-2 scaled scores

  const int last_query = min(q0 + 32, a.q_rows) - 1;
  const int visible_keys = min(a.kv_rows, a.start_position + last_query + 1);
  const int key_tiles = (visible_keys + 31) / 32;
  const int my_last_key = a.start_position + query;  // keys beyond it are masked
  // The key rows of a tile are requested one tile ahead and its value rows
  // before its softmax: a wave runs alone on its SIMD, so nothing else hides
  // the latency of these loads.
  float4 k_next[HALF / 4];
  {
    const float4* row = reinterpret_cast<const float4*>(
        k_base + min(wave * 32 + n, a.kv_rows - 1) * a.k.row_stride + h * HALF);
#pragma unroll
    for (int j = 0; j < HALF / 4; ++j) k_next[j] = row[j];
  }
  for (int kt = wave; kt < key_tiles; kt += kKeySplit) {
    float kf[HALF];
#pragma unroll
    for (int j = 0; j < HALF / 4; ++j) {
      kf[4 * j] = k_next[j].x; kf[4 * j + 1] = k_next[j].y;
      kf[4 * j + 2] = k_next[j].z; kf[4 * j + 3] = k_next[j].w;
    }
    if (kt + kKeySplit < key_tiles) {
      const float4* row = reinterpret_cast<const float4*>(
          k_base + min((kt + kKeySplit) * 32 + n, a.kv_rows - 1) * a.k.row_stride + h * HALF);
#pragma unroll
      for (int j = 0; j < HALF / 4; ++j) k_next[j] = row[j];
    }
    float values[DB][16];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = min(kt * 32 + 8 * (i / 4) + 4 * h + (i % 4), a.kv_rows - 1);
        values[db][i] = v_base[key * a.v.row_stride + 32 * db + n];
      }
    floatx16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.0f;
#pragma unroll
    for (int j = 0; j < HALF; ++j)
      s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[j], qf[j], s, 0, 0, 0);
    // register i = (key kt*32 + 8(i/4) + 4h + i%4, query n)
    float tile_max = kMasked;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = kt * 32 + 8 * (i / 4) + 4 * h + (i % 4);
      const bool visible = key <= my_last_key && key < a.kv_rows;
      s[i] = visible ? s[i] * scale2 : kMasked;
      tile_max = fmaxf(tile_max, s[i]);
    }
    tile_max = half_swap_max(tile_max);
    const float new_max = fmaxf(running_max, tile_max);
    const float correction = __builtin_amdgcn_exp2f(running_max - new_max);
    running_max = new_max;
    float tile_sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float p = s[i] == kMasked ? 0.0f : __builtin_amdgcn_exp2f(s[i] - new_max);
      s[i] = p;
      tile_sum += p;
    }
    running_sum = running_sum * correction + half_swap_sum(tile_sum);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] *= correction;
#pragma unroll
      for (int i = 0; i < 16; ++i)
        o[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(values[db][i], s[i], o[db], 0, 0, 0);
    }
  }
  // ---- merge: every wave's result is relative to its own maximum ------------
  if (wave > 0) {
    part_max[wave - 1][lane] = running_max;
    part_sum[wave - 1][lane] = running_sum;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) part_o[wave - 1][db * 16 + i][lane] = o[db][i];
  }
  __syncthreads();
  if (wave > 0) return;
  {
    float maximum = running_max;
#pragma unroll
    for (int w = 0; w < kKeySplit - 1; ++w) maximum = fmaxf(maximum, part_max[w][lane]);
    // a wave without tiles contributes weight 2^(kMasked - maximum) = 0
    const float own = __builtin_amdgcn_exp2f(running_max - maximum);
    running_sum *= own;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] *= own;
#pragma unroll
    for (int w = 0; w < kKeySplit - 1; ++w) {
      const float weight = __builtin_amdgcn_exp2f(part_max[w][lane] - maximum);
      running_sum += part_sum[w][lane] * weight;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] += part_o[w][db * 16 + i][lane] * weight;
    }
    running_max = maximum;
  }
  if (query >= a.q_rows) return;
  const float normalizer = running_sum > 0.0f ? running_sum : 1.0f;
  const float inverse = 1.0f / normalizer;
  float* out = static_cast<float*>(a.out) + seq * a.o_seq_stride + query * a.o_row_stride +
               head * a.o_head_stride;
  // O^T register i of block db = (channel 32 db + 8(i/4) + 4h + i%4, query n)
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float4 piece;
      piece.x = o[db][4 * j] * inverse;
      piece.y = o[db][4 * j + 1] * inverse;
      piece.z = o[db][4 * j + 2] * inverse;
      piece.w = o[db][4 * j + 3] * inverse;
      *reinterpret_cast<float4*>(out + 32 * db + 8 * j + 4 * h) = piece;
    }
  if (h == 0) {
    const float maximum = running_max * (1.0f / kLog2e);
    const long long stat = (static_cast<long long>(seq) * a.query_heads + head) * a.q_rows + query;
    if (a.maxima) a.maxima[stat] = maximum;
    if (a.normalizers) a.normalizers[stat] = normalizer;
    if (a.lse)
      a.lse[(static_cast<long long>(seq) * a.q_rows + query) * a.query_heads + head] =
          maximum + logf(normalizer);
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

bool f32_forward_supported(const GenericForwardArgs& a) {
  if (a.head_dim != 32 && a.head_dim != 64 && a.head_dim != 128) return false;
  if (a.q.dtype != PLUTO_HIP_F32 || a.k.dtype != PLUTO_HIP_F32 || a.v.dtype != PLUTO_HIP_F32 ||
      a.o_dtype != PLUTO_HIP_F32 || a.gate.base != nullptr)
    return false;
  if (a.q_rows <= 0 || a.kv_rows <= 0) return false;
  auto mult4 = [](long long s) { return (s % 4) == 0; };
  return aligned16(a.q.base) && aligned16(a.k.base) && aligned16(a.v.base) && aligned16(a.out) &&
         mult4(a.q.seq_stride) && mult4(a.q.row_stride) && mult4(a.q.head_stride) &&
         mult4(a.k.seq_stride) && mult4(a.k.row_stride) && mult4(a.k.head_stride) &&
         mult4(a.v.seq_stride) && mult4(a.v.row_stride) && mult4(a.v.head_stride) &&
         mult4(a.o_seq_stride) && mult4(a.o_row_stride) && mult4(a.o_head_stride);
}

int launch_f32_forward(hipStream_t stream, const GenericForwardArgs& a, int sequences) {
  const dim3 grid((a.q_rows + 31) / 32, a.query_heads, sequences);
  if (grid.y > 65535u || grid.z > 65535u) return PLUTO_HIP_EUNSUPPORTED;
  if (!kernel_enabled(kMainKernel)) return 0;
  switch (a.head_dim) {
    case 32: f32_forward_kernel<32><<<grid, 64 * kKeySplit, 0, stream>>>(a); break;
    case 64: f32_forward_kernel<64><<<grid, 64 * kKeySplit, 0, stream>>>(a); break;
    case 128: f32_forward_kernel<128><<<grid, 64 * kKeySplit, 0, stream>>>(a); break;
    default: return PLUTO_HIP_EUNSUPPORTED;
  }
  return launch_status();
}

}  // namespace pluto_hip
