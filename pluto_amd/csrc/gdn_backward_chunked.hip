// Chunked backward of the gated delta rule for 128 x 128 heads: the same
// gradients as the token-by-token kernels of gdn_backward.hip
// (RecurrenceForward / RecurrenceBackward, src/llm/layers/
// sequence_delta_net.cc:55-102 and :171-253), computed 64 tokens at a time on
// the FP32 matrix cores, and with one saved state per chunk instead of one per
// token.
//
// For a chunk entered with state S (rows: key channels, columns: value
// channels), tokens i = 0..63, G_i the running sum of the log decays inside
// the chunk, E_i = exp(G_i), D_ij = exp(G_i - G_j) (i >= j), L_j = exp(G_63 -
// G_j), q^ and k^ the normalised (and, for q, scaled) rows:
//   A   = strict_lower(beta_i (k^_i . k^_j) D_ij)        T = (I + A)^-1
//   W   = T diag(beta E) K^                               U = T diag(beta) V
//   Dl  = U - W S                 (the 64 delta rows of the chunk)
//   P   = lower((q^_i . k^_j) D_ij)
//   O   = diag(E) Q^ S + P Dl
//   S'  = E_63 S + (diag(L) K^)^T Dl
// which is the recurrence S <- decay S; delta = beta (v - S^T k^); S += k^ x
// delta; o = S^T q^ unrolled over the chunk.  Eliminating Dl, the state obeys
// an affine recurrence whose matrices depend on one chunk only,
//   S' = M S + B,     M = E_63 I - (diag(L) K^)^T W,    B = (diag(L) K^)^T U,
// and so does its gradient:
//   dS = M^T dS' + C,  C = Y^T dO,   Y = diag(E) Q^ - P W.
// The kernels, in launch order:
//   chunk_prepare_kernel           T, W, U, P of every chunk          (parallel)
//   chunk_transfer_kernel          M, M^T, B, Y                       (parallel)
//   chunk_states_forward_kernel    S entering every chunk             (sequential)
//   chunk_outputs_kernel           Dl and O from S                    (parallel)
//     -- the caller turns O into dO here --
//   chunk_local_kernel             C                                  (parallel)
//   chunk_states_backward_kernel   dS' leaving every chunk            (sequential)
//   chunk_gradients_kernel         dDl, then dq, dk, dv, d beta and
//                                  d log-decay of the chunk           (parallel)
// The sequential kernels run one workgroup per (head, 32 value columns) and
// do one 128 x 128 x 32 product a chunk, with the next chunk's matrix already
// in registers.  Matrix products run on v_mfma_f32_32x32x2_f32; operands are
// read straight from global memory or from LDS.
#include "gdn.h"

namespace pluto_hip {
namespace {

constexpr int kC = 64;       // tokens per chunk
constexpr int kD = 128;      // key and value channels per head
constexpr int kSlice = 32;   // value columns per workgroup of the sequential kernels
constexpr int kWide = kC * kD;     // elements of a [64, 128] record
constexpr int kSquare = kC * kC;   // elements of a [64, 64] record
constexpr int kState = kD * kD;    // elements of a state

// Per (head, chunk) records in the workspace, in floats.
struct Records {
  float *qn, *kn;             // q^, k^                                  [64][128]
  float *w, *u, *y, *dl;      // W, U, Y, Dl                             [64][128]
  float *p, *tm, *kkd;        // P, T, strict_lower((k^_i . k^_j) D_ij)  [64][64]
  float *gates;               // [6][64]: G, beta, 1/|q|, 1/|k|, E, L
  float *m, *mt, *bc, *cc;    // M, M^T, B, C                            [128][128]
  float *s0, *ds1;            // state entering the chunk, gradient of the state leaving it
};

constexpr int kGateRows = 6;
constexpr size_t kRecordFloats = 6 * static_cast<size_t>(kWide) + 3 * kSquare + kGateRows * kC +
                                 6 * static_cast<size_t>(kState);

struct ChunkedArgs {
  const float* post = nullptr;     // [T, channels]
  const uint16_t* a = nullptr;     // bf16 [T, vh]
  const uint16_t* b = nullptr;
  const float* a_log = nullptr;
  const float* dt_bias = nullptr;
  const float* dcore = nullptr;    // [T, vh, 128]
  float* core = nullptr;           // [T, vh, 128]
  float* dpost = nullptr;          // [T, channels]: the value part is written
  float* qk_partials = nullptr;    // [T, vh, 2, 128]
  float* scalar_partials = nullptr;  // [T, vh, 3]
  Records r;
  int length = 0, chunks = 0, kh = 0, vh = 0;
  bool round = true;
};

__device__ inline float round_if(float x, bool round) { return round ? round_to_bf16(x) : x; }

__device__ inline floatx16 zero_tile() {
  floatx16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.0f;
  return z;
}

// Row of accumulator register i of a 32 x 32 tile in a lane of half h; the
// column is lane % 32.
__device__ inline int tile_row(int i, int h) { return 8 * (i / 4) + 4 * h + i % 4; }

// acc[m][n] += sum over k < K of A[m][k] B[k][n] for the lane's operand row m
// and column n: a(k) returns A[m][k], b(k) returns B[k][n].
template <int K, class AF, class BF>
__device__ inline floatx16 product(floatx16 acc, AF a, BF b) {
  const int h = (threadIdx.x % 64) / 32;
#pragma unroll 8
  for (int k = 0; k < K; k += 2)
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a(k + h), b(k + h), acc, 0, 0, 0);
  return acc;
}

// The same sum for operands that are contiguous along k: a4(k) returns
// A[m][k..k+3], b4(k) returns B[k..k+3][n], k a multiple of 4.  The two lane
// halves take alternate groups of four (the order of a contraction is free).
template <int K, class AF, class BF>
__device__ inline floatx16 product4(floatx16 acc, AF a4, BF b4) {
  const int h = (threadIdx.x % 64) / 32;
#pragma unroll 4
  for (int k = 0; k < K; k += 8) {
    const float4 x = a4(k + 4 * h), y = b4(k + 4 * h);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.x, y.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.y, y.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.z, y.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.w, y.w, acc, 0, 0, 0);
  }
  return acc;
}

__device__ inline float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }

__device__ inline float4 scaled(float4 v, float s) {
  return make_float4(v.x * s, v.y * s, v.z * s, v.w * s);
}

__device__ inline float4 gather4(const float* p, int stride) {
  return make_float4(p[0], p[stride], p[2 * stride], p[3 * stride]);
}

// Barrier for data exchanged through LDS only: pending global loads and
// stores stay in flight across it.
__device__ inline void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---------------------------------------------------------------------------
// T, W, U, P and the gates of one chunk.
__global__ void __launch_bounds__(256)
chunk_prepare_kernel(ChunkedArgs a) {
  __shared__ float qs[kC][kD + 1], ks[kC][kD + 1];
  __shared__ float am[kC][kC + 4];                  // A, rows 16-byte aligned
  __shared__ float tk[kC][kC + 1], tv[kC][kC + 1];  // T diag(beta E), T diag(beta)
  __shared__ float log_decay[kC], g_cum[kC], beta_s[kC];
  const int chunk = blockIdx.x, head = blockIdx.y;
  const int key_head = head / (a.vh / a.kh);
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int channels = 2 * a.kh * kD + a.vh * kD;
  const size_t rec = static_cast<size_t>(head) * a.chunks + chunk;
  const int t0 = chunk * kC;
  const float norm_scale = sqrtf(static_cast<float>(kD));
  float* gates = a.r.gates + rec * kGateRows * kC;

  // normalised rows (1e-6 added to the sums of squares, sequence_delta_net.cc:84-85)
  for (int r = 0; r < kC / 4; ++r) {
    const int i = wave * (kC / 4) + r, t = t0 + i;
    const bool ok = t < a.length;
    const float* row = a.post + static_cast<size_t>(ok ? t : 0) * channels;
    float q[2], k[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      q[j] = ok ? row[key_head * kD + lane + 64 * j] : 0.0f;
      k[j] = ok ? row[(a.kh + key_head) * kD + lane + 64 * j] : 0.0f;
    }
    const float iq = rsqrtf(wave_sum(q[0] * q[0] + q[1] * q[1]) + 1e-6f);
    const float ik = rsqrtf(wave_sum(k[0] * k[0] + k[1] * k[1]) + 1e-6f);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const float qv = q[j] * iq / norm_scale, kv = k[j] * ik;
      qs[i][lane + 64 * j] = qv;
      ks[i][lane + 64 * j] = kv;
      a.r.qn[rec * kWide + i * kD + lane + 64 * j] = qv;
      a.r.kn[rec * kWide + i * kD + lane + 64 * j] = kv;
    }
    if (lane == 0) {
      gates[2 * kC + i] = iq;
      gates[3 * kC + i] = ik;
    }
  }
  // gates (sequence_delta_net.cc:88-96); tokens beyond the sequence neither
  // decay nor write
  if (tid < kC) {
    const int t = t0 + tid;
    const bool ok = t < a.length;
    float g = 0.0f, beta = 0.0f;
    if (ok) {
      const float alpha = bf16_bits_to_float(a.a[static_cast<size_t>(t) * a.vh + head]) + a.dt_bias[head];
      const float softplus = fmaxf(alpha, 0.0f) + logf(1.0f + expf(-fabsf(alpha)));
      g = -expf(a.a_log[head]) * softplus;
      const float bv = bf16_bits_to_float(a.b[static_cast<size_t>(t) * a.vh + head]);
      beta = round_if(1.0f / (1.0f + expf(-bv)), a.round);
    }
    log_decay[tid] = g;
    beta_s[tid] = beta;
    gates[kC + tid] = beta;
  }
  __syncthreads();
  if (tid == 0) {
    float c = 0.0f;
    for (int i = 0; i < kC; ++i) {
      c += log_decay[i];
      g_cum[i] = c;
    }
  }
  __syncthreads();
  if (tid < kC) {
    gates[tid] = g_cum[tid];
    gates[4 * kC + tid] = expf(g_cum[tid]);
    gates[5 * kC + tid] = expf(g_cum[kC - 1] - g_cum[tid]);
  }

  // k^ k^T and q^ k^T, one 32 x 32 tile a wave (tile (0, 1) is above the diagonal)
  {
    const int ti = wave / 2, tj = wave % 2;
    floatx16 kk = zero_tile(), qk = zero_tile();
    if (ti >= tj) {
      kk = product<kD>(kk, [&](int k) { return ks[32 * ti + n][k]; },
                       [&](int k) { return ks[32 * tj + n][k]; });
      qk = product<kD>(qk, [&](int k) { return qs[32 * ti + n][k]; },
                       [&](int k) { return ks[32 * tj + n][k]; });
    }
    const int col = 32 * tj + n;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      const float d = row >= col ? expf(g_cum[row] - g_cum[col]) : 0.0f;
      const float kv = row > col ? kk[i] * d : 0.0f;
      a.r.p[rec * kSquare + row * kC + col] = row >= col ? qk[i] * d : 0.0f;
      a.r.kkd[rec * kSquare + row * kC + col] = kv;
      am[row][col] = beta_s[row] * kv;
    }
  }
  __syncthreads();
  // T = (I + A)^-1 by forward substitution, one column a lane
  if (wave == 0) {
    float x[kC];
#pragma unroll
    for (int i = 0; i < kC; ++i) {
      float s = i == lane ? 1.0f : 0.0f;
#pragma unroll
      for (int j = 0; j < i; ++j) s -= am[i][j] * x[j];
      x[i] = s;
    }
    const float fv = beta_s[lane], fk = fv * expf(g_cum[lane]);
#pragma unroll
    for (int i = 0; i < kC; ++i) {
      tk[i][lane] = x[i] * fk;
      tv[i][lane] = x[i] * fv;
      a.r.tm[rec * kSquare + i * kC + lane] = x[i];
    }
  }
  __syncthreads();
  // W = T diag(beta E) K^, U = T diag(beta) V: the wave owns 32 columns
  {
    const int col = 32 * wave + n;
    const size_t value_offset = 2 * static_cast<size_t>(a.kh) * kD + static_cast<size_t>(head) * kD;
#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
      const floatx16 wacc = product<kC>(zero_tile(), [&](int k) { return tk[32 * ti + n][k]; },
                                        [&](int k) { return ks[k][col]; });
      const floatx16 uacc = product<kC>(
          zero_tile(), [&](int k) { return tv[32 * ti + n][k]; },
          [&](int k) {
            const int t = t0 + k;
            return t < a.length ? a.post[static_cast<size_t>(t) * channels + value_offset + col] : 0.0f;
          });
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = 32 * ti + tile_row(i, h);
        a.r.w[rec * kWide + row * kD + col] = wacc[i];
        a.r.u[rec * kWide + row * kD + col] = uacc[i];
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The matrices of the two affine recurrences that depend on the chunk alone:
// M, M^T, B and Y.  Wave w owns columns 32w..32w+31 of each.
__global__ void __launch_bounds__(256)
chunk_transfer_kernel(ChunkedArgs a) {
  __shared__ float e_s[kC], l_s[kC];
  const int chunk = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const size_t rec = static_cast<size_t>(head) * a.chunks + chunk;
  const float* gates = a.r.gates + rec * kGateRows * kC;
  const float* Q = a.r.qn + rec * kWide;
  const float* K = a.r.kn + rec * kWide;
  const float* W = a.r.w + rec * kWide;
  const float* U = a.r.u + rec * kWide;
  const float* P = a.r.p + rec * kSquare;
  if (tid < kC) {
    e_s[tid] = gates[4 * kC + tid];
    l_s[tid] = gates[5 * kC + tid];
  }
  __syncthreads();
  const int col = 32 * wave + n;
  // Y = diag(E) Q^ - P W
#pragma unroll
  for (int ti = 0; ti < 2; ++ti) {
    floatx16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      acc[i] = e_s[row] * Q[row * kD + col];
    }
    const int m = 32 * ti + n;
    acc = product4<kC>(acc, [&](int k) { return scaled(load4(P + m * kC + k), -1.0f); },
                       [&](int k) { return gather4(W + k * kD + col, kD); });
#pragma unroll
    for (int i = 0; i < 16; ++i) a.r.y[rec * kWide + (32 * ti + tile_row(i, h)) * kD + col] = acc[i];
  }
  // M = E_63 I - (diag(L) K^)^T W and B = (diag(L) K^)^T U
  const float e_last = e_s[kC - 1];
#pragma unroll
  for (int td = 0; td < 4; ++td) {
    const int m = 32 * td + n;
    floatx16 macc;
#pragma unroll
    for (int i = 0; i < 16; ++i) macc[i] = 32 * td + tile_row(i, h) == col ? e_last : 0.0f;
    macc = product<kC>(macc, [&](int k) { return -l_s[k] * K[k * kD + m]; },
                       [&](int k) { return W[k * kD + col]; });
    const floatx16 bacc = product<kC>(zero_tile(), [&](int k) { return l_s[k] * K[k * kD + m]; },
                                      [&](int k) { return U[k * kD + col]; });
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int row = 32 * td + tile_row(4 * i4, h);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        a.r.m[rec * kState + (row + e) * kD + col] = macc[4 * i4 + e];
        a.r.bc[rec * kState + (row + e) * kD + col] = bacc[4 * i4 + e];
      }
      *reinterpret_cast<float4*>(a.r.mt + rec * kState + col * kD + row) =
          make_float4(macc[4 * i4], macc[4 * i4 + 1], macc[4 * i4 + 2], macc[4 * i4 + 3]);
    }
  }
}

// ---------------------------------------------------------------------------
// next = matrix . state + offset over the chunks of one (head, 32 value
// columns): forward (REVERSE false) it stores the state entering every chunk,
// with matrix M (read through its transpose) and offset B; in reverse it
// stores the state gradient leaving every chunk, with matrix M^T (read through
// M) and offset C.  Wave w keeps rows 32w..32w+31 of the slice; the matrix
// column and the offset tile of the next chunk are requested while the
// current product runs.
template <bool REVERSE>
__global__ void __launch_bounds__(256)
chunk_states_kernel(ChunkedArgs a) {
  __shared__ float state[2][kD][kSlice];
  const int head = blockIdx.x / (kD / kSlice), col0 = (blockIdx.x % (kD / kSlice)) * kSlice;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const float* matrices = REVERSE ? a.r.m : a.r.mt;
  const float* offsets = REVERSE ? a.r.cc : a.r.bc;
  float* saved = REVERSE ? a.r.ds1 : a.r.s0;
  auto record = [&](int step) {
    return static_cast<size_t>(head) * a.chunks + (REVERSE ? a.chunks - 1 - step : step);
  };
  float matrix[kD / 2], next_matrix[kD / 2];
  floatx16 offset, next_offset;
  auto request = [&](int step, float* mat, floatx16& off) {
    const size_t rec = record(step);
    const float* source = matrices + rec * kState + 32 * wave + n;
#pragma unroll
    for (int s = 0; s < kD / 2; ++s) mat[s] = source[(2 * s + h) * kD];
#pragma unroll
    for (int i = 0; i < 16; ++i)
      off[i] = offsets[rec * kState + (32 * wave + tile_row(i, h)) * kD + col0 + n];
  };
  request(0, matrix, offset);
  floatx16 acc = zero_tile();
  for (int step = 0; step < a.chunks; ++step) {
    const size_t rec = record(step);
    float (*current)[kSlice] = state[step & 1];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * wave + tile_row(i, h);
      current[row][n] = acc[i];
      saved[rec * kState + row * kD + col0 + n] = acc[i];
    }
    lds_barrier();
    if (step + 1 < a.chunks) request(step + 1, next_matrix, next_offset);
    acc = offset;
#pragma unroll
    for (int s = 0; s < kD / 2; ++s)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(matrix[s], current[2 * s + h][n], acc, 0, 0, 0);
#pragma unroll
    for (int s = 0; s < kD / 2; ++s) matrix[s] = next_matrix[s];
    offset = next_offset;
  }
}

// ---------------------------------------------------------------------------
// Dl = U - W S and O = diag(E) Q^ S + P Dl of one chunk.  Wave w owns value
// columns 32w..32w+31.
__global__ void __launch_bounds__(256)
chunk_outputs_kernel(ChunkedArgs a) {
  __shared__ float delta[kC][kD];
  __shared__ float e_s[kC];
  const int chunk = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const size_t rec = static_cast<size_t>(head) * a.chunks + chunk;
  const float* gates = a.r.gates + rec * kGateRows * kC;
  const float* S0 = a.r.s0 + rec * kState;
  const float* Q = a.r.qn + rec * kWide;
  const float* W = a.r.w + rec * kWide;
  const float* U = a.r.u + rec * kWide;
  const float* P = a.r.p + rec * kSquare;
  if (tid < kC) e_s[tid] = gates[4 * kC + tid];
  const int col = 32 * wave + n;
  floatx16 out[2];
#pragma unroll
  for (int ti = 0; ti < 2; ++ti) {
    const int m = 32 * ti + n;
    floatx16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = U[(32 * ti + tile_row(i, h)) * kD + col];
    acc = product4<kD>(acc, [&](int k) { return scaled(load4(W + m * kD + k), -1.0f); },
                       [&](int k) { return gather4(S0 + k * kD + col, kD); });
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      delta[row][col] = acc[i];
      a.r.dl[rec * kWide + row * kD + col] = acc[i];
    }
    out[ti] = product4<kD>(zero_tile(), [&](int k) { return load4(Q + m * kD + k); },
                           [&](int k) { return gather4(S0 + k * kD + col, kD); });
  }
  __syncthreads();
#pragma unroll
  for (int ti = 0; ti < 2; ++ti) {
    const int m = 32 * ti + n;
#pragma unroll
    for (int i = 0; i < 16; ++i) out[ti][i] *= e_s[32 * ti + tile_row(i, h)];
    // only columns j <= i of P are set: the second row tile needs all 64
    out[ti] = product4<kC>(out[ti], [&](int k) { return load4(P + m * kC + k); },
                           [&](int k) {
                             return make_float4(delta[k][col], delta[k + 1][col], delta[k + 2][col],
                                                delta[k + 3][col]);
                           });
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int t = chunk * kC + 32 * ti + tile_row(i, h);
      if (t < a.length)
        a.core[(static_cast<size_t>(t) * a.vh + head) * kD + col] = round_if(out[ti][i], a.round);
    }
  }
}

// ---------------------------------------------------------------------------
// C = Y^T dO of one chunk.
__global__ void __launch_bounds__(256)
chunk_local_kernel(ChunkedArgs a) {
  const int chunk = blockIdx.x, head = blockIdx.y;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const size_t rec = static_cast<size_t>(head) * a.chunks + chunk;
  const float* Y = a.r.y + rec * kWide;
  const int col = 32 * wave + n, t0 = chunk * kC;
#pragma unroll
  for (int td = 0; td < 4; ++td) {
    const int m = 32 * td + n;
    const floatx16 acc = product<kC>(
        zero_tile(), [&](int k) { return Y[k * kD + m]; },
        [&](int k) {
          const int t = t0 + k;
          return t < a.length ? a.dcore[(static_cast<size_t>(t) * a.vh + head) * kD + col] : 0.0f;
        });
#pragma unroll
    for (int i = 0; i < 16; ++i)
      a.r.cc[rec * kState + (32 * td + tile_row(i, h)) * kD + col] = acc[i];
  }
}

// ---------------------------------------------------------------------------
// Sum over the 32 lanes of a half wave, into lane n == 0 of the half (and
// every other lane of it).
__device__ inline float half_sum(float v) { return wave_half_sum(v); }

// Gradients of one chunk: dDl = P^T dO + diag(L) K^ dS', then everything
// the chunk's formulas feed.  Wave w owns columns 32w..32w+31 of the [64, 128]
// matrices (two 32-row tiles each) and one 32 x 32 tile of every [64, 64]
// intermediate.
__global__ void __launch_bounds__(256)
chunk_gradients_kernel(ChunkedArgs a) {
  __shared__ float dw[kC][kD + 1];
  __shared__ __attribute__((aligned(16))) float ddl[kC][kD + 4];
  __shared__ float mx[kC][kC + 1], my[kC][kC + 1], mz[kC][kC + 1], mu[kC][kC + 1];
  __shared__ float g_s[kC], e_s[kC], l_s[kC], beta_s[kC], dg_s[kC];
  __shared__ float row_parts[6][kC][4];
  __shared__ float row_sums[4][kC];
  __shared__ float reduce[256];
  const int chunk = blockIdx.x, head = blockIdx.y;
  const int key_head = head / (a.vh / a.kh);
  (void)key_head;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int channels = 2 * a.kh * kD + a.vh * kD;
  const size_t value_offset = 2 * static_cast<size_t>(a.kh) * kD + static_cast<size_t>(head) * kD;
  const size_t rec = static_cast<size_t>(head) * a.chunks + chunk;
  const int t0 = chunk * kC;
  const float* gates = a.r.gates + rec * kGateRows * kC;
  const float* S0 = a.r.s0 + rec * kState;
  const float* dS1 = a.r.ds1 + rec * kState;
  const float* Dl = a.r.dl + rec * kWide;
  const float* Q = a.r.qn + rec * kWide;
  const float* K = a.r.kn + rec * kWide;
  const float* Tm = a.r.tm + rec * kSquare;
  const float* P = a.r.p + rec * kSquare;
  const float* KKD = a.r.kkd + rec * kSquare;
  // rows of dO and V of tokens beyond the sequence are zero
  auto dO4 = [&](int i, int c) {
    const int t = t0 + i;
    return t < a.length ? load4(a.dcore + (static_cast<size_t>(t) * a.vh + head) * kD + c)
                        : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  };
  auto dO1 = [&](int i, int c) {
    const int t = t0 + i;
    return t < a.length ? a.dcore[(static_cast<size_t>(t) * a.vh + head) * kD + c] : 0.0f;
  };
  auto V4 = [&](int j, int c) {
    const int t = t0 + j;
    return t < a.length ? load4(a.post + static_cast<size_t>(t) * channels + value_offset + c)
                        : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  };
  auto V1 = [&](int j, int c) {
    const int t = t0 + j;
    return t < a.length ? a.post[static_cast<size_t>(t) * channels + value_offset + c] : 0.0f;
  };
  if (tid < kC) {
    const float g = gates[tid];
    g_s[tid] = g;
    e_s[tid] = gates[4 * kC + tid];
    l_s[tid] = gates[5 * kC + tid];
    beta_s[tid] = gates[kC + tid];
  }
  __syncthreads();
  const int dcol = 32 * wave + n;

  // ---- dDl = P^T dO + diag(L) K^ dS' ----------------------------------------
#pragma unroll
  for (int ti = 0; ti < 2; ++ti) {
    const int m = 32 * ti + n;
    floatx16 acc = product<kC>(zero_tile(), [&](int k) { return P[k * kC + m]; },
                               [&](int k) { return dO1(k, dcol); });
    const float l = l_s[m];
    acc = product4<kD>(acc, [&](int k) { return scaled(load4(K + m * kD + k), l); },
                       [&](int k) { return gather4(dS1 + k * kD + dcol, kD); });
#pragma unroll
    for (int i = 0; i < 16; ++i) ddl[32 * ti + tile_row(i, h)][dcol] = acc[i];
  }
  __syncthreads();

  // ---- products against the two states ------------------------------------
  floatx16 dq[2], dk[2];
#pragma unroll
  for (int ti = 0; ti < 2; ++ti) {
    const int m = 32 * ti + n;
    // dW = -dDl S^T
    const floatx16 dwt = product4<kD>(
        zero_tile(), [&](int k) { return scaled(load4(&ddl[m][k]), -1.0f); },
        [&](int k) { return load4(S0 + dcol * kD + k); });
#pragma unroll
    for (int i = 0; i < 16; ++i) dw[32 * ti + tile_row(i, h)][dcol] = dwt[i];
    // d(diag(E) Q^) = dO S^T, times E
    const float e = e_s[m];
    dq[ti] = product4<kD>(zero_tile(), [&](int k) { return scaled(dO4(m, k), e); },
                          [&](int k) { return load4(S0 + dcol * kD + k); });
    // d(diag(L) K^) = Dl dS'^T, times L
    const float l = l_s[m];
    dk[ti] = product4<kD>(zero_tile(), [&](int k) { return scaled(load4(Dl + m * kD + k), l); },
                          [&](int k) { return load4(dS1 + dcol * kD + k); });
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      const float gq = half_sum(dq[ti][i] * Q[row * kD + dcol]);
      const float g1 = half_sum(dk[ti][i] * K[row * kD + dcol]);
      if (n == 0) {
        row_parts[0][row][wave] = gq;
        row_parts[1][row][wave] = g1;
      }
    }
  }
  // dP = lower(dO Dl^T): Pd = dP D and dP P
  const int ti = wave / 2, tj = wave % 2;
  {
    floatx16 dp = zero_tile();
    if (ti >= tj)
      dp = product4<kD>(dp, [&](int k) { return dO4(32 * ti + n, k); },
                        [&](int k) { return load4(Dl + (32 * tj + n) * kD + k); });
    const int col = 32 * tj + n;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      const bool keep = row >= col;
      const float value = keep ? dp[i] : 0.0f;
      my[row][col] = keep ? value * expf(g_s[row] - g_s[col]) : 0.0f;
      mu[row][col] = value * P[row * kC + col];
    }
  }
  // <dS', S>
  {
    float dot = 0.0f;
    for (int idx = tid; idx < kState; idx += 256) dot += S0[idx] * dS1[idx];
    reduce[tid] = dot;
  }
  __syncthreads();

  // ---- dT = dW (diag(beta E) K^)^T + dDl (diag(beta) V)^T ------------------
  {
    const int j = 32 * tj + n;
    const float fv = beta_s[j], fk = fv * e_s[j];
    floatx16 acc = product<kD>(zero_tile(), [&](int k) { return dw[32 * ti + n][k]; },
                               [&](int k) { return K[j * kD + k] * fk; });
    acc = product4<kD>(acc, [&](int k) { return load4(&ddl[32 * ti + n][k]); },
                       [&](int k) { return scaled(V4(j, k), fv); });
#pragma unroll
    for (int i = 0; i < 16; ++i) mx[32 * ti + tile_row(i, h)][j] = acc[i];
  }
  __syncthreads();
  // ---- X = T^T dT ----------------------------------------------------------
  {
    const floatx16 acc = product<kC>(zero_tile(), [&](int k) { return Tm[k * kC + 32 * ti + n]; },
                                     [&](int k) { return mx[k][32 * tj + n]; });
#pragma unroll
    for (int i = 0; i < 16; ++i) mz[32 * ti + tile_row(i, h)][32 * tj + n] = acc[i];
  }
  __syncthreads();
  // ---- dA = -strict_lower(X T^T) ------------------------------------------
  {
    floatx16 acc = zero_tile();
    if (ti >= tj)
      acc = product<kC>(acc, [&](int k) { return -mz[32 * ti + n][k]; },
                        [&](int k) { return Tm[(32 * tj + n) * kC + k]; });
    __syncthreads();  // X has been read by every wave
    const int col = 32 * tj + n;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      const bool keep = row > col;
      const float da = keep ? acc[i] : 0.0f;
      mz[row][col] = da * KKD[row * kC + col];                                         // N
      mx[row][col] = keep ? da * beta_s[row] * expf(g_s[row] - g_s[col]) : 0.0f;     // R
    }
  }
  __syncthreads();
  if (tid < kC) {
    // row sums of N and of dP P; column sums of diag(beta) N and of dP P
    float row_n = 0.0f, col_m = 0.0f, row_p = 0.0f, col_p = 0.0f;
    for (int j = 0; j < kC; ++j) {
      row_n += mz[tid][j];
      col_m += beta_s[j] * mz[j][tid];
      row_p += mu[tid][j];
      col_p += mu[j][tid];
    }
    row_sums[0][tid] = row_n;
    row_sums[1][tid] = col_m;
    row_sums[2][tid] = row_p;
    row_sums[3][tid] = col_p;
  }

  // ---- the three outputs ----------------------------------------------------
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2) {
    const int m = 32 * t2 + n;
    // dq^ += Pd K^
    dq[t2] = product<kC>(dq[t2], [&](int k) { return my[m][k]; },
                         [&](int k) { return K[k * kD + dcol]; });
    // T^T dW: d(diag(beta E) K^)
    const floatx16 tw = product<kC>(zero_tile(), [&](int k) { return Tm[k * kC + m]; },
                                    [&](int k) { return dw[k][dcol]; });
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * t2 + tile_row(i, h);
      const float r = half_sum(tw[i] * K[row * kD + dcol]) * e_s[row];
      if (n == 0) row_parts[2][row][wave] = r;
      dk[t2][i] += beta_s[row] * e_s[row] * tw[i];
    }
    // dk^ += (R + R^T) K^ + Pd^T Q^
    dk[t2] = product<kC>(dk[t2], [&](int k) { return mx[m][k] + mx[k][m]; },
                         [&](int k) { return K[k * kD + dcol]; });
    dk[t2] = product<kC>(dk[t2], [&](int k) { return my[k][m]; },
                         [&](int k) { return Q[k * kD + dcol]; });
    // dv = diag(beta) T^T dDl
    const floatx16 tu = product<kC>(zero_tile(), [&](int k) { return Tm[k * kC + m]; },
                                    [&](int k) { return ddl[k][dcol]; });
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * t2 + tile_row(i, h), t = t0 + row;
      const float rv = half_sum(tu[i] * V1(row, dcol));
      const float q_dot = half_sum(dq[t2][i] * Q[row * kD + dcol]);
      const float k_dot = half_sum(dk[t2][i] * K[row * kD + dcol]);
      if (n == 0) {
        row_parts[3][row][wave] = rv;
        row_parts[4][row][wave] = q_dot;
        row_parts[5][row][wave] = k_dot;
      }
      if (t < a.length) a.dpost[static_cast<size_t>(t) * channels + value_offset + dcol] = beta_s[row] * tu[i];
    }
  }
  __syncthreads();
  auto parts = [&](int which, int row) {
    return (row_parts[which][row][0] + row_parts[which][row][1]) +
           (row_parts[which][row][2] + row_parts[which][row][3]);
  };
  // back through the L2 normalisations (and the 1/sqrt(d) of q)
  const float norm_scale = sqrtf(static_cast<float>(kD));
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * t2 + tile_row(i, h), t = t0 + row;
      if (t >= a.length) continue;
      const float iq = gates[2 * kC + row], ik = gates[3 * kC + row];
      const float qv = Q[row * kD + dcol], kv = K[row * kD + dcol];
      float* out = a.qk_partials + (static_cast<size_t>(t) * a.vh + head) * 2 * kD;
      out[dcol] = iq / norm_scale * (dq[t2][i] - static_cast<float>(kD) * qv * parts(4, row));
      out[kD + dcol] = ik * (dk[t2][i] - kv * parts(5, row));
    }
  // d log-decay and d beta
  if (tid < kC) {
    const float beta = beta_s[tid];
    const float g1 = parts(1, tid), r = parts(2, tid);
    float dG = parts(0, tid) + beta * r + (beta * row_sums[0][tid] - row_sums[1][tid]) +
               (row_sums[2][tid] - row_sums[3][tid]) - g1;
    if (tid == kC - 1) {
      float total = 0.0f;
      for (int j = 0; j < kC; ++j) total += parts(1, j);
      float dot = 0.0f;
      for (int j = 0; j < 256; ++j) dot += reduce[j];
      dG += total + dot * e_s[kC - 1];
    }
    dg_s[tid] = dG;
  }
  __syncthreads();
  if (tid < kC) {
    const int t = t0 + tid;
    if (t < a.length) {
      float dg = 0.0f;
      for (int i = kC - 1; i >= tid; --i) dg += dg_s[i];
      const float dbeta = row_sums[0][tid] + parts(2, tid) + parts(3, tid);
      const float alpha = bf16_bits_to_float(a.a[static_cast<size_t>(t) * a.vh + head]) + a.dt_bias[head];
      const float softplus = fmaxf(alpha, 0.0f) + logf(1.0f + expf(-fabsf(alpha)));
      const float rate = expf(a.a_log[head]);
      const float bv = bf16_bits_to_float(a.b[static_cast<size_t>(t) * a.vh + head]);
      const float sigmoid = 1.0f / (1.0f + expf(-bv));
      float* out = a.scalar_partials + (static_cast<size_t>(t) * a.vh + head) * 3;
      out[0] = -dg * rate / (1.0f + expf(-alpha));
      out[1] = dbeta * sigmoid * (1.0f - sigmoid);
      out[2] = -dg * rate * softplus;
    }
  }
}

ChunkedArgs make_args(const GdnChunkedBackward& c) {
  ChunkedArgs a;
  a.post = c.post;
  a.a = c.a;
  a.b = c.b;
  a.a_log = c.a_log;
  a.dt_bias = c.dt_bias;
  a.dcore = c.dcore;
  a.core = c.core;
  a.dpost = c.dpost;
  a.qk_partials = c.qk_partials;
  a.scalar_partials = c.scalar_partials;
  a.length = c.length;
  a.chunks = (c.length + kC - 1) / kC;
  a.kh = c.key_heads;
  a.vh = c.value_heads;
  a.round = c.round;
  const size_t n = static_cast<size_t>(a.chunks) * a.vh;
  float* at = c.records;
  auto take = [&](size_t floats) {
    float* result = at;
    at += n * floats;
    return result;
  };
  a.r.qn = take(kWide);
  a.r.kn = take(kWide);
  a.r.w = take(kWide);
  a.r.u = take(kWide);
  a.r.y = take(kWide);
  a.r.dl = take(kWide);
  a.r.p = take(kSquare);
  a.r.tm = take(kSquare);
  a.r.kkd = take(kSquare);
  a.r.gates = take(kGateRows * kC);
  a.r.m = take(kState);
  a.r.mt = take(kState);
  a.r.bc = take(kState);
  a.r.cc = take(kState);
  a.r.s0 = take(kState);
  a.r.ds1 = take(kState);
  return a;
}

}  // namespace

bool gdn_backward_chunked_supported(const pluto_hip_delta_params* p) {
  return p->key_head_dim == kD && p->value_head_dim == kD && p->key_heads > 0 &&
         p->value_heads % p->key_heads == 0;
}

size_t gdn_backward_chunked_bytes(const pluto_hip_delta_params* p, int length) {
  const size_t chunks = (static_cast<size_t>(length) + kC - 1) / kC;
  return align_up(chunks * p->value_heads * kRecordFloats * sizeof(float), 256);
}

int launch_gdn_backward_chunked_forward(hipStream_t stream, const GdnChunkedBackward& c) {
  const ChunkedArgs a = make_args(c);
  const dim3 per_chunk(a.chunks, a.vh);
  chunk_prepare_kernel<<<per_chunk, 256, 0, stream>>>(a);
  int status = launch_status();
  if (status != 0) return status;
  chunk_transfer_kernel<<<per_chunk, 256, 0, stream>>>(a);
  status = launch_status();
  if (status != 0) return status;
  chunk_states_kernel<false><<<a.vh * (kD / kSlice), 256, 0, stream>>>(a);
  status = launch_status();
  if (status != 0) return status;
  chunk_outputs_kernel<<<per_chunk, 256, 0, stream>>>(a);
  return launch_status();
}

int launch_gdn_backward_chunked_reverse(hipStream_t stream, const GdnChunkedBackward& c) {
  const ChunkedArgs a = make_args(c);
  const dim3 per_chunk(a.chunks, a.vh);
  chunk_local_kernel<<<per_chunk, 256, 0, stream>>>(a);
  int status = launch_status();
  if (status != 0) return status;
  chunk_states_kernel<true><<<a.vh * (kD / kSlice), 256, 0, stream>>>(a);
  status = launch_status();
  if (status != 0) return status;
  chunk_gradients_kernel<<<per_chunk, 256, 0, stream>>>(a);
  return launch_status();
}

}  // namespace pluto_hip
