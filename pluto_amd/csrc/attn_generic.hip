// Any-shape causal attention kernels in plain FP32 arithmetic.
//
// These serve every configuration the MFMA kernels do not specialise: FP32
// storage (the reference's DataType::FP16 policy), head widths that are not 64
// or 128, caches kept in FP32, and unrounded Qwen activations.  They follow
// the reference kernels' structure (src/llm/layers/attention.cc:98-396): 32x32
// score tiles, online softmax with a finite sentinel, query-owned dQ and
// key-owned dK/dV tiles with fixed reduction order and no atomics.
#include "attn_generic.h"

namespace pluto_hip {
namespace {

constexpr int kTile = 32;      // query rows / keys per tile
constexpr int kChunk = 64;     // head channels staged through LDS at a time
constexpr int kThreads = 128;  // (ty 0..3) x (tx 0..31); thread owns 8 rows
constexpr int kRowsPerThread = 8;
constexpr int kMaxColumnGroups = 8;  // head_dim <= 256 = 8 * 32

__device__ inline long long view_offset(const StridedView& v, int seq, int row,
                                        int head) {
  return seq * v.seq_stride + row * v.row_stride + head * v.head_stride;
}

// Stage rows [row0, row0+32) x channels [c0, c0+64) of one head into LDS,
// zero filled outside [0, rows) x [0, dim).
__device__ inline void stage_tile(float (*dst)[kChunk + 1],
                                  const StridedView& view, int seq, int head,
                                  int row0, int rows, int c0, int dim) {
  for (int i = threadIdx.x; i < kTile * kChunk; i += kThreads) {
    const int r = i / kChunk, c = i % kChunk;
    const int row = row0 + r, channel = c0 + c;
    float value = 0.0f;
    if (row < rows && channel < dim)
      value = load_element(view.base, view_offset(view, seq, row, head) + channel,
                           view.dtype);
    dst[r][c] = value;
  }
}

__global__ void __launch_bounds__(kThreads)
generic_forward_kernel(GenericForwardArgs a) {
  __shared__ float Qs[kTile][kChunk + 1];
  __shared__ float Ks[kTile][kChunk + 1];
  __shared__ float Ps[kTile][kTile + 1];
  const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
  const int q0 = blockIdx.x * kTile;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int kv_head = head / a.group;
  const int chunks = (a.head_dim + kChunk - 1) / kChunk;

  float m[kRowsPerThread], l[kRowsPerThread];
  float acc[kRowsPerThread][kMaxColumnGroups];
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) {
    m[r] = kMasked;
    l[r] = 0.0f;
#pragma unroll
    for (int j = 0; j < kMaxColumnGroups; ++j) acc[r][j] = 0.0f;
  }
  // Keys visible to the last query row of this tile.
  const int last_row = min(q0 + kTile, a.q_rows) - 1;
  const int visible_keys = min(a.kv_rows, a.start_position + last_row + 1);
  const int key_tiles = (visible_keys + kTile - 1) / kTile;
  if (chunks == 1) {
    stage_tile(Qs, a.q, seq, head, q0, a.q_rows, 0, a.head_dim);
  }
  for (int kt = 0; kt < key_tiles; ++kt) {
    float s[kRowsPerThread];
#pragma unroll
    for (int r = 0; r < kRowsPerThread; ++r) s[r] = 0.0f;
    for (int dc = 0; dc < chunks; ++dc) {
      __syncthreads();
      if (chunks > 1)
        stage_tile(Qs, a.q, seq, head, q0, a.q_rows, dc * kChunk, a.head_dim);
      stage_tile(Ks, a.k, seq, kv_head, kt * kTile, a.kv_rows, dc * kChunk,
                 a.head_dim);
      __syncthreads();
      const int width = min(kChunk, a.head_dim - dc * kChunk);
      for (int c = 0; c < width; ++c) {
        const float key = Ks[tx][c];
#pragma unroll
        for (int r = 0; r < kRowsPerThread; ++r)
          s[r] += Qs[ty * kRowsPerThread + r][c] * key;
      }
    }
    const int key = kt * kTile + tx;
#pragma unroll
    for (int r = 0; r < kRowsPerThread; ++r) {
      const int row = q0 + ty * kRowsPerThread + r;
      const bool visible = row < a.q_rows && key < a.kv_rows &&
                           key <= a.start_position + row;
      const float score = visible ? s[r] * a.scale : kMasked;
      const float new_max = fmaxf(m[r], wave_half_max(score));
      const float correction = expf(m[r] - new_max);
      const float p = visible ? expf(score - new_max) : 0.0f;
      l[r] = l[r] * correction + wave_half_sum(p);
      m[r] = new_max;
#pragma unroll
      for (int j = 0; j < kMaxColumnGroups; ++j) acc[r][j] *= correction;
      Ps[ty * kRowsPerThread + r][tx] = p;
    }
    // V reuses the K staging area, one channel chunk at a time.
    for (int dc = 0; dc < chunks; ++dc) {
      __syncthreads();
      stage_tile(Ks, a.v, seq, kv_head, kt * kTile, a.kv_rows, dc * kChunk,
                 a.head_dim);
      __syncthreads();
      for (int j = 0; j < kTile; ++j) {
        const float v0 = Ks[j][tx], v1 = Ks[j][tx + 32];
#pragma unroll
        for (int r = 0; r < kRowsPerThread; ++r) {
          const float p = Ps[ty * kRowsPerThread + r][j];
#pragma unroll
          for (int g = 0; g < kMaxColumnGroups / 2; ++g) {
            if (g == dc) {
              acc[r][2 * g] += p * v0;
              acc[r][2 * g + 1] += p * v1;
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) {
    const int row = q0 + ty * kRowsPerThread + r;
    if (row >= a.q_rows) continue;
    const float normalizer = l[r] > 0.0f ? l[r] : 1.0f;
    const long long o_base = seq * a.o_seq_stride + row * a.o_row_stride +
                             head * a.o_head_stride;
#pragma unroll
    for (int j = 0; j < kMaxColumnGroups; ++j) {
      const int channel = tx + 32 * j;
      if (channel >= a.head_dim) continue;
      float value = acc[r][j] / normalizer;
      if (a.gate.base != nullptr) {
        const float logit = load_element(
            a.gate.base, view_offset(a.gate, seq, row, head) + channel,
            a.gate.dtype);
        float sigmoid = gate_sigmoid(logit);
        if (a.round_to_bf16) {
          value = round_to_bf16(round_to_bf16(value) * round_to_bf16(sigmoid));
        } else {
          value = value * sigmoid;
        }
      }
      store_element(a.out, o_base + channel, a.o_dtype, value);
    }
    if (tx == 0) {
      const long long stat =
          (static_cast<long long>(seq) * a.query_heads + head) * a.q_rows + row;
      if (a.maxima) a.maxima[stat] = m[r];
      if (a.normalizers) a.normalizers[stat] = normalizer;
      if (a.lse)
        a.lse[(static_cast<long long>(seq) * a.q_rows + row) * a.query_heads +
              head] = m[r] + logf(normalizer);
    }
  }
}

// Probabilities rebuilt from saved statistics: attention.cc:176-230.
__global__ void __launch_bounds__(kThreads)
generic_probabilities_kernel(GenericForwardArgs a, float* probabilities) {
  __shared__ float Qs[kTile][kChunk + 1];
  __shared__ float Ks[kTile][kChunk + 1];
  const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
  const int tiles = (a.q_rows + kTile - 1) / kTile;
  const int kt = blockIdx.x % tiles, qt = blockIdx.x / tiles;
  const int head = blockIdx.y, seq = blockIdx.z;
  const int chunks = (a.head_dim + kChunk - 1) / kChunk;
  float s[kRowsPerThread];
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) s[r] = 0.0f;
  if (kt <= qt) {
    for (int dc = 0; dc < chunks; ++dc) {
      __syncthreads();
      stage_tile(Qs, a.q, seq, head, qt * kTile, a.q_rows, dc * kChunk,
                 a.head_dim);
      stage_tile(Ks, a.k, seq, head / a.group, kt * kTile, a.kv_rows,
                 dc * kChunk, a.head_dim);
      __syncthreads();
      const int width = min(kChunk, a.head_dim - dc * kChunk);
      for (int c = 0; c < width; ++c) {
        const float key = Ks[tx][c];
#pragma unroll
        for (int r = 0; r < kRowsPerThread; ++r)
          s[r] += Qs[ty * kRowsPerThread + r][c] * key;
      }
    }
  }
  const int key = kt * kTile + tx;
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) {
    const int row = qt * kTile + ty * kRowsPerThread + r;
    if (row >= a.q_rows || key >= a.q_rows) continue;
    const long long stat =
        (static_cast<long long>(seq) * a.query_heads + head) * a.q_rows + row;
    float p = 0.0f;
    if (key <= row) {
      const float normalizer = a.normalizers[stat] > 0.0f ? a.normalizers[stat] : 1.0f;
      p = expf(s[r] * a.scale - a.maxima[stat]) / normalizer;
    }
    probabilities[stat * a.q_rows + key] = p;
  }
}

// delta = sum(dO * O) per (row, head): attention.cc:283-291.  One wave per
// (row, head).
__global__ void __launch_bounds__(256)
generic_delta_kernel(GenericBackwardArgs a) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const long long unit = static_cast<long long>(blockIdx.x) * 4 + wave;
  const long long units = static_cast<long long>(a.rows) * a.num_heads;
  if (unit >= units) return;
  const int row = static_cast<int>(unit / a.num_heads);
  const int head = static_cast<int>(unit % a.num_heads);
  const int dim = a.embedding_dim / a.num_heads;
  const long long base = static_cast<long long>(row) * a.embedding_dim + head * dim;
  float sum = 0.0f;
  for (int c = lane; c < dim; c += 64)
    sum += a.d_out[base + c] * load_element(a.out, base + c, a.dtype);
  sum = wave_sum(sum);
  if (lane == 0) {
    const int seq = row / a.context_length, pos = row % a.context_length;
    a.deltas[(static_cast<long long>(seq) * a.num_heads + head) * a.context_length +
             pos] = sum;
  }
}

__device__ inline void stage_packed(float (*dst)[kChunk + 1], const void* base,
                                    int dtype, long long row_stride,
                                    long long column0, int row0, int row_limit,
                                    long long sequence_row0, int c0, int dim) {
  for (int i = threadIdx.x; i < kTile * kChunk; i += kThreads) {
    const int r = i / kChunk, c = i % kChunk;
    const int row = row0 + r, channel = c0 + c;
    float value = 0.0f;
    if (row < row_limit && channel < dim)
      value = load_element(base, (sequence_row0 + row) * row_stride + column0 + channel,
                           dtype);
    dst[r][c] = value;
  }
}

// Scores and dP for one [32 queries x 32 keys] tile; thread (ty, tx) ends with
// rows ty*8.. of key column tx.  Stages Q, K, dO, V by channel chunk.
__device__ inline void score_and_dp_tile(
    const GenericBackwardArgs& a, float (*Qs)[kChunk + 1],
    float (*Ks)[kChunk + 1], float (*Gs)[kChunk + 1], float (*Vs)[kChunk + 1],
    long long sequence_row0, int head, int q0, int k0, float* s, float* dp) {
  const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
  const int E = a.embedding_dim, dim = E / a.num_heads;
  const int chunks = (dim + kChunk - 1) / kChunk;
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) {
    s[r] = 0.0f;
    dp[r] = 0.0f;
  }
  for (int dc = 0; dc < chunks; ++dc) {
    __syncthreads();
    stage_packed(Qs, a.qkv, a.dtype, 3LL * E, head * dim, q0, a.context_length,
                 sequence_row0, dc * kChunk, dim);
    stage_packed(Ks, a.qkv, a.dtype, 3LL * E, E + head * dim, k0,
                 a.context_length, sequence_row0, dc * kChunk, dim);
    stage_packed(Vs, a.qkv, a.dtype, 3LL * E, 2LL * E + head * dim, k0,
                 a.context_length, sequence_row0, dc * kChunk, dim);
    stage_packed(Gs, a.d_out, PLUTO_HIP_F32, E, head * dim, q0,
                 a.context_length, sequence_row0, dc * kChunk, dim);
    __syncthreads();
    const int width = min(kChunk, dim - dc * kChunk);
    for (int c = 0; c < width; ++c) {
      const float key = Ks[tx][c], value = Vs[tx][c];
#pragma unroll
      for (int r = 0; r < kRowsPerThread; ++r) {
        s[r] += Qs[ty * kRowsPerThread + r][c] * key;
        dp[r] += Gs[ty * kRowsPerThread + r][c] * value;
      }
    }
  }
}

// P and dS of the tile from scores, dP and the saved row statistics:
// attention.cc:304-308.
__device__ inline void probability_and_ds(const GenericBackwardArgs& a,
                                          long long stats_base, int q0, int k0,
                                          const float* s, const float* dp,
                                          float (*Ps)[kTile + 1],
                                          float (*Ds)[kTile + 1]) {
  const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
  const int key = k0 + tx;
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) {
    const int row = q0 + ty * kRowsPerThread + r;
    float p = 0.0f, ds = 0.0f;
    if (row < a.context_length && key <= row) {
      const float normalizer = a.normalizers[stats_base + row];
      p = expf(s[r] * a.scale - a.maxima[stats_base + row]) /
          (normalizer > 0.0f ? normalizer : 1.0f);
      ds = p * (dp[r] - a.deltas[stats_base + row]) * a.scale;
    }
    Ps[ty * kRowsPerThread + r][tx] = p;
    Ds[ty * kRowsPerThread + r][tx] = ds;
  }
}

// Query-owned dQ tiles: attention.cc:235-314.
__global__ void __launch_bounds__(kThreads)
generic_dq_kernel(GenericBackwardArgs a) {
  __shared__ float Qs[kTile][kChunk + 1];
  __shared__ float Ks[kTile][kChunk + 1];
  __shared__ float Gs[kTile][kChunk + 1];
  __shared__ float Vs[kTile][kChunk + 1];
  __shared__ float Ps[kTile][kTile + 1];
  __shared__ float Ds[kTile][kTile + 1];
  const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
  const int q0 = blockIdx.x * kTile, head = blockIdx.y, seq = blockIdx.z;
  const int E = a.embedding_dim, dim = E / a.num_heads;
  const int chunks = (dim + kChunk - 1) / kChunk;
  const long long sequence_row0 = static_cast<long long>(seq) * a.context_length;
  const long long stats_base =
      (static_cast<long long>(seq) * a.num_heads + head) * a.context_length;
  float acc[kRowsPerThread][kMaxColumnGroups];
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r)
#pragma unroll
    for (int j = 0; j < kMaxColumnGroups; ++j) acc[r][j] = 0.0f;
  const int last_row = min(q0 + kTile, a.context_length) - 1;
  const int key_tiles = last_row / kTile + 1;
  for (int kt = 0; kt < key_tiles; ++kt) {
    float s[kRowsPerThread], dp[kRowsPerThread];
    score_and_dp_tile(a, Qs, Ks, Gs, Vs, sequence_row0, head, q0, kt * kTile, s, dp);
    probability_and_ds(a, stats_base, q0, kt * kTile, s, dp, Ps, Ds);
    for (int dc = 0; dc < chunks; ++dc) {
      __syncthreads();
      if (chunks > 1)
        stage_packed(Ks, a.qkv, a.dtype, 3LL * E, E + head * dim, kt * kTile,
                     a.context_length, sequence_row0, dc * kChunk, dim);
      __syncthreads();
      for (int j = 0; j < kTile; ++j) {
        const float k0v = Ks[j][tx], k1v = Ks[j][tx + 32];
#pragma unroll
        for (int r = 0; r < kRowsPerThread; ++r) {
          const float ds = Ds[ty * kRowsPerThread + r][j];
#pragma unroll
          for (int g = 0; g < kMaxColumnGroups / 2; ++g) {
            if (g == dc) {
              acc[r][2 * g] += ds * k0v;
              acc[r][2 * g + 1] += ds * k1v;
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) {
    const int row = q0 + ty * kRowsPerThread + r;
    if (row >= a.context_length) continue;
#pragma unroll
    for (int j = 0; j < kMaxColumnGroups; ++j) {
      const int channel = tx + 32 * j;
      if (channel < dim)
        a.d_qkv[(sequence_row0 + row) * 3LL * E + head * dim + channel] = acc[r][j];
    }
  }
}

// Key-owned dK and dV tiles, query tiles visited in ascending order:
// attention.cc:319-396.
__global__ void __launch_bounds__(kThreads)
generic_dkv_kernel(GenericBackwardArgs a) {
  __shared__ float Qs[kTile][kChunk + 1];
  __shared__ float Ks[kTile][kChunk + 1];
  __shared__ float Gs[kTile][kChunk + 1];
  __shared__ float Vs[kTile][kChunk + 1];
  __shared__ float Ps[kTile][kTile + 1];
  __shared__ float Ds[kTile][kTile + 1];
  const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
  const int k0 = blockIdx.x * kTile, head = blockIdx.y, seq = blockIdx.z;
  const int E = a.embedding_dim, dim = E / a.num_heads;
  const int chunks = (dim + kChunk - 1) / kChunk;
  const long long sequence_row0 = static_cast<long long>(seq) * a.context_length;
  const long long stats_base =
      (static_cast<long long>(seq) * a.num_heads + head) * a.context_length;
  float dk[kRowsPerThread][kMaxColumnGroups], dv[kRowsPerThread][kMaxColumnGroups];
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r)
#pragma unroll
    for (int j = 0; j < kMaxColumnGroups; ++j) {
      dk[r][j] = 0.0f;
      dv[r][j] = 0.0f;
    }
  const int row_tiles = (a.context_length + kTile - 1) / kTile;
  for (int qt = blockIdx.x; qt < row_tiles; ++qt) {
    float s[kRowsPerThread], dp[kRowsPerThread];
    score_and_dp_tile(a, Qs, Ks, Gs, Vs, sequence_row0, head, qt * kTile, k0, s, dp);
    probability_and_ds(a, stats_base, qt * kTile, k0, s, dp, Ps, Ds);
    for (int dc = 0; dc < chunks; ++dc) {
      __syncthreads();
      if (chunks > 1) {
        stage_packed(Qs, a.qkv, a.dtype, 3LL * E, head * dim, qt * kTile,
                     a.context_length, sequence_row0, dc * kChunk, dim);
        stage_packed(Gs, a.d_out, PLUTO_HIP_F32, E, head * dim, qt * kTile,
                     a.context_length, sequence_row0, dc * kChunk, dim);
      }
      __syncthreads();
      // Thread (ty, tx) owns keys ty*8.. and channels tx, tx+32 of the chunk.
      for (int j = 0; j < kTile; ++j) {
        const float q0v = Qs[j][tx], q1v = Qs[j][tx + 32];
        const float g0v = Gs[j][tx], g1v = Gs[j][tx + 32];
#pragma unroll
        for (int r = 0; r < kRowsPerThread; ++r) {
          const float ds = Ds[j][ty * kRowsPerThread + r];
          const float p = Ps[j][ty * kRowsPerThread + r];
#pragma unroll
          for (int g = 0; g < kMaxColumnGroups / 2; ++g) {
            if (g == dc) {
              dk[r][2 * g] += ds * q0v;
              dk[r][2 * g + 1] += ds * q1v;
              dv[r][2 * g] += p * g0v;
              dv[r][2 * g + 1] += p * g1v;
            }
          }
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < kRowsPerThread; ++r) {
    const int key = k0 + ty * kRowsPerThread + r;
    if (key >= a.context_length) continue;
#pragma unroll
    for (int j = 0; j < kMaxColumnGroups; ++j) {
      const int channel = tx + 32 * j;
      if (channel >= dim) continue;
      const long long base = (sequence_row0 + key) * 3LL * E + head * dim + channel;
      a.d_qkv[base + E] = dk[r][j];
      a.d_qkv[base + 2LL * E] = dv[r][j];
    }
  }
}

}  // namespace

int launch_generic_forward(hipStream_t stream, const GenericForwardArgs& a,
                           int sequences) {
  if (a.head_dim > 32 * kMaxColumnGroups) return PLUTO_HIP_EUNSUPPORTED;
  dim3 grid((a.q_rows + kTile - 1) / kTile, a.query_heads, sequences);
  generic_forward_kernel<<<grid, kThreads, 0, stream>>>(a);
  return launch_status();
}

int launch_generic_probabilities(hipStream_t stream,
                                 const GenericForwardArgs& a, int sequences,
                                 float* probabilities) {
  if (a.head_dim > 32 * kMaxColumnGroups) return PLUTO_HIP_EUNSUPPORTED;
  const int tiles = (a.q_rows + kTile - 1) / kTile;
  dim3 grid(tiles * tiles, a.query_heads, sequences);
  generic_probabilities_kernel<<<grid, kThreads, 0, stream>>>(a, probabilities);
  return launch_status();
}

int launch_generic_delta(hipStream_t stream, const GenericBackwardArgs& a) {
  const long long units = static_cast<long long>(a.rows) * a.num_heads;
  generic_delta_kernel<<<static_cast<int>((units + 3) / 4), 256, 0, stream>>>(a);
  return launch_status();
}

int launch_generic_backward(hipStream_t stream, const GenericBackwardArgs& a) {
  const int dim = a.embedding_dim / a.num_heads;
  if (dim > 32 * kMaxColumnGroups) return PLUTO_HIP_EUNSUPPORTED;
  int status = launch_generic_delta(stream, a);
  if (status != 0) return status;
  dim3 grid((a.context_length + kTile - 1) / kTile, a.num_heads,
            a.rows / a.context_length);
  generic_dq_kernel<<<grid, kThreads, 0, stream>>>(a);
  status = launch_status();
  if (status != 0) return status;
  generic_dkv_kernel<<<grid, kThreads, 0, stream>>>(a);
  return launch_status();
}

}  // namespace pluto_hip
