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
//   chunk_delta_gradient_kernel    dDl from dO and dS'                (parallel)
//   chunk_state_products_kernel    dW and the state terms of dq^, dk^ (parallel)
//   chunk_triangle_kernel          dP, dT, dA: the [64, 64] matrices  (parallel)
//   chunk_finish_kernel            dq, dk, dv                         (parallel)
//   chunk_gates_kernel             d beta, d log-decay -> da, db      (parallel)
// The sequential kernels run one workgroup per (head, 16 value columns) and
// do one 128 x 128 x 16 product a chunk, with the next chunk's matrix already
// in registers.  Matrix products run on v_mfma_f32_32x32x2_f32; operands are
// read straight from global memory or from LDS.
#include "gdn.h"

namespace pluto_hip {
namespace {

constexpr int kC = 64;       // tokens per chunk
constexpr int kD = 128;      // key and value channels per head
constexpr int kSlice = 16;   // value columns per workgroup of the sequential kernels
constexpr int kWide = kC * kD;     // elements of a [64, 128] record
constexpr int kSquare = kC * kC;   // elements of a [64, 64] record
constexpr int kState = kD * kD;    // elements of a state

// Per (head, chunk) records in the workspace, in floats.
struct Records {
  float *qn, *kn;             // q^, k^                                  [64][128]
  float *w, *u, *y, *dl;      // W, U, Y, Dl                             [64][128]
  float *ddl, *dwm;           // dDl, dW                                 [64][128]
  float *dqp, *dkp;           // the parts of dq^ and dk^ that come from the states
  float *p, *tm, *kkd;        // P, T, strict_lower((k^_i . k^_j) D_ij)  [64][64]
  float *pd, *rr;             // dP D, diag(beta) dA D                   [64][64]
  float *gates;               // [6][64]: G, beta, 1/|q|, 1/|k|, E, L
  float *sums;                // [9][64]: row and column sums for d beta and d log-decay
  float *m, *mt, *bc, *cc;    // M, M^T, B, C                            [128][128]
  float *s0, *ds1;            // state entering the chunk, gradient of the state leaving it
};

constexpr int kGateRows = 6, kSumRows = 9;
constexpr size_t kRecordFloats = 10 * static_cast<size_t>(kWide) + 5 * kSquare +
                                 (kGateRows + kSumRows) * kC + 6 * static_cast<size_t>(kState);

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
// and column n: a(k) returns A[m][k], b(k) returns B[k][n].  Every operand of
// the product is requested before the first multiplication (one memory
// latency a product instead of one every few steps) unless STREAM is set:
// kernels whose registers allow many resident waves do better with the loads
// spread between the multiplications.
template <int K, bool STREAM = false, class AF, class BF>
__device__ inline floatx16 product(floatx16 acc, AF a, BF b) {
  const int h = (threadIdx.x % 64) / 32;
  if constexpr (STREAM) {
#pragma unroll 8
    for (int k = 0; k < K; k += 2)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a(k + h), b(k + h), acc, 0, 0, 0);
    return acc;
  }
  float av[K / 2], bv[K / 2];
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < K / 2; ++s) {
    av[s] = a(2 * s + h);
    bv[s] = b(2 * s + h);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < K / 2; ++s)
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s], bv[s], acc, 0, 0, 0);
  __builtin_amdgcn_sched_barrier(0);
  return acc;
}

// The same sum for operands that are contiguous along k: a4(k) returns
// A[m][k..k+3], b4(k) returns B[k..k+3][n], k a multiple of 4.  The two lane
// halves take alternate groups of four (the order of a contraction is free).
template <int K, bool STREAM = false, class AF, class BF>
__device__ inline floatx16 product4(floatx16 acc, AF a4, BF b4) {
  const int h = (threadIdx.x % 64) / 32;
  if constexpr (STREAM) {
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
  float4 av[K / 8], bv[K / 8];
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < K / 8; ++s) {
    av[s] = a4(8 * s + 4 * h);
    bv[s] = b4(8 * s + 4 * h);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int s = 0; s < K / 8; ++s) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s].x, bv[s].x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s].y, bv[s].y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s].z, bv[s].z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s].w, bv[s].w, acc, 0, 0, 0);
  }
  __builtin_amdgcn_sched_barrier(0);
  return acc;
}

__device__ inline float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }

__device__ inline float4 scaled(float4 v, float s) {
  return make_float4(v.x * s, v.y * s, v.z * s, v.w * s);
}

// Rows of tokens beyond the sequence read as zero: the load itself is always
// made (from the last row), so that it needs no branch.
__device__ inline float keep(bool ok, float v) { return ok ? v : 0.0f; }
__device__ inline float4 keep(bool ok, float4 v) {
  return make_float4(ok ? v.x : 0.0f, ok ? v.y : 0.0f, ok ? v.z : 0.0f, ok ? v.w : 0.0f);
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
            const int t = t0 + k, row = min(t, a.length - 1);
            return keep(t < a.length, a.post[static_cast<size_t>(row) * channels + value_offset + col]);
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
// next = matrix . state + offset over the chunks of one (head, 16 value
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
  // The eight column slices of a head read the same matrices: they are given
  // block numbers with the same remainder mod 8, which the hardware places on
  // one XCD, so that seven of the eight reads are served by that XCD's L2.
  constexpr int kSlices = kD / kSlice;
  static_assert(kSlices == 8, "one slice of a head per block of an XCD's share");
  int head = blockIdx.x / kSlices, slice = blockIdx.x % kSlices;
  if (a.vh % 8 == 0) {
    head = (blockIdx.x % 8) * (a.vh / 8) + blockIdx.x / 64;
    slice = (blockIdx.x / 8) % kSlices;
  }
  const int col0 = slice * kSlice;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int quarter = lane / 16, n = lane % 16;
  const float* matrices = REVERSE ? a.r.m : a.r.mt;
  const float* offsets = REVERSE ? a.r.cc : a.r.bc;
  float* saved = REVERSE ? a.r.ds1 : a.r.s0;
  auto record = [&](int step) {
    return static_cast<size_t>(head) * a.chunks + (REVERSE ? a.chunks - 1 - step : step);
  };
  // v_mfma_f32_16x16x4_f32: lane (quarter, n) supplies A[n][quarter] and
  // B[quarter][n] and receives C[4 quarter + e][n], e = 0..3.  The wave's 32
  // rows are two such tiles, interleaved (tile t holds rows 2i + t) so that a
  // lane's two matrix elements of a step are neighbours in memory.
  constexpr int kSteps = kD / 4;
  struct Operands {
    float2 matrix[kSteps];
    floatx4 offset[2];
  };
  auto row_of = [&](int tile, int e) { return 32 * wave + 8 * quarter + 2 * e + tile; };
  auto matrix_of = [&](int step) {
    return matrices + record(min(step, a.chunks - 1)) * kState + 32 * wave + 2 * n + quarter * kD;
  };
  auto request_matrix = [&](const float* source, Operands& o, int s) {
    o.matrix[s] = *reinterpret_cast<const float2*>(source + 4 * s * kD);
  };
  auto request_offset = [&](int step, Operands& o) {
    const size_t rec = record(min(step, a.chunks - 1));
#pragma unroll
    for (int tile = 0; tile < 2; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        o.offset[tile][e] = offsets[rec * kState + row_of(tile, e) * kD + col0 + n];
  };
  auto request = [&](int step, Operands& o) {
    const float* source = matrix_of(step);
#pragma unroll
    for (int s = 0; s < kSteps; ++s) request_matrix(source, o, s);
    request_offset(step, o);
  };
  floatx4 acc[2];
#pragma unroll
  for (int tile = 0; tile < 2; ++tile)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[tile][e] = 0.0f;
  // One chunk: publish the state, multiply with the operands requested two
  // chunks ago, request those of the chunk after next.  Three register sets
  // take turns.  The requests are spread between the multiplications (their
  // address arithmetic runs while the matrix pipe is busy) and come after the
  // first of them in program order: the wait for this chunk's operands then
  // has fewer than 64 younger memory operations behind it, which is as far as
  // the counter reaches.  Requests are unconditional (past the end they repeat
  // the last chunk's) so that the number in flight is the same on every path.
  auto advance = [&](int step, const Operands& now, Operands& later) {
    float (*current)[kSlice] = state[step & 1];
#pragma unroll
    for (int tile = 0; tile < 2; ++tile)
#pragma unroll
      for (int e = 0; e < 4; ++e) current[row_of(tile, e)][n] = acc[tile][e];
    if (step < a.chunks) {
      const size_t rec = record(step);
#pragma unroll
      for (int tile = 0; tile < 2; ++tile)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          saved[rec * kState + row_of(tile, e) * kD + col0 + n] = acc[tile][e];
    }
    lds_barrier();
    acc[0] = now.offset[0];
    acc[1] = now.offset[1];
    const float* source = matrix_of(step + 2);
    float b[kSteps];
#pragma unroll
    for (int s = 0; s < kSteps; ++s) b[s] = current[4 * s + quarter][n];
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(now.matrix[s].x, b[s], acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(now.matrix[s].y, b[s], acc[1], 0, 0, 0);
      request_matrix(source, later, s);
      __builtin_amdgcn_sched_barrier(0);
    }
    request_offset(step + 2, later);
  };
  Operands set0, set1, set2;
  request(0, set0);
  request(1, set1);
  for (int step = 0; step < a.chunks; step += 3) {
    advance(step, set0, set2);
    advance(step + 1, set1, set0);
    advance(step + 2, set2, set1);
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
    acc = product4<kD, true>(acc, [&](int k) { return scaled(load4(W + m * kD + k), -1.0f); },
                       [&](int k) { return gather4(S0 + k * kD + col, kD); });
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      delta[row][col] = acc[i];
      a.r.dl[rec * kWide + row * kD + col] = acc[i];
    }
    out[ti] = product4<kD, true>(zero_tile(), [&](int k) { return load4(Q + m * kD + k); },
                           [&](int k) { return gather4(S0 + k * kD + col, kD); });
  }
  __syncthreads();
#pragma unroll
  for (int ti = 0; ti < 2; ++ti) {
    const int m = 32 * ti + n;
#pragma unroll
    for (int i = 0; i < 16; ++i) out[ti][i] *= e_s[32 * ti + tile_row(i, h)];
    // only columns j <= i of P are set: the second row tile needs all 64
    out[ti] = product4<kC, true>(out[ti], [&](int k) { return load4(P + m * kC + k); },
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
          const int t = t0 + k, row = min(t, a.length - 1);
          return keep(t < a.length, a.dcore[(static_cast<size_t>(row) * a.vh + head) * kD + col]);
        });
#pragma unroll
    for (int i = 0; i < 16; ++i)
      a.r.cc[rec * kState + (32 * td + tile_row(i, h)) * kD + col] = acc[i];
  }
}

// ---------------------------------------------------------------------------
// The gradients of one chunk, in four kernels that exchange [64, 128] and
// [64, 64] matrices through the records.  In each, wave w owns columns
// 32w..32w+31 of the [64, 128] matrices (two 32-row tiles) or one 32 x 32 tile
// of a [64, 64] matrix.

// Sums over the 32 lanes of a half wave of sixteen values at once: the five
// exchange stages are the outer loop, so that the sixteen exchanges of a stage
// are in flight together (one value at a time, each stage waits for the one
// before and the sums cost ten times as much).
__device__ inline void half_sums(float (&v)[16]) {
#pragma unroll
  for (int offset = 16; offset > 0; offset >>= 1) {
    float other[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) other[i] = __shfl_xor(v[i], offset, 64);
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] += other[i];
  }
}

// Sums over the four waves of per-row partial sums left in parts[row][wave].
__device__ inline float across_waves(const float (*parts)[4], int row) {
  return (parts[row][0] + parts[row][1]) + (parts[row][2] + parts[row][3]);
}

struct ChunkView {
  size_t rec;
  int t0, head, channels;
  size_t value_offset;
  const float *gates, *S0, *dS1, *Dl, *Q, *K, *Tm, *P, *KKD;
};

__device__ inline ChunkView chunk_view(const ChunkedArgs& a, int chunk, int head) {
  ChunkView v;
  v.rec = static_cast<size_t>(head) * a.chunks + chunk;
  v.t0 = chunk * kC;
  v.head = head;
  v.channels = 2 * a.kh * kD + a.vh * kD;
  v.value_offset = 2 * static_cast<size_t>(a.kh) * kD + static_cast<size_t>(head) * kD;
  v.gates = a.r.gates + v.rec * kGateRows * kC;
  v.S0 = a.r.s0 + v.rec * kState;
  v.dS1 = a.r.ds1 + v.rec * kState;
  v.Dl = a.r.dl + v.rec * kWide;
  v.Q = a.r.qn + v.rec * kWide;
  v.K = a.r.kn + v.rec * kWide;
  v.Tm = a.r.tm + v.rec * kSquare;
  v.P = a.r.p + v.rec * kSquare;
  v.KKD = a.r.kkd + v.rec * kSquare;
  return v;
}

// A 1-D grid of `parts` workgroups per (head, chunk) unit that read the same
// records: the parts of a unit get block numbers with the same remainder mod 8
// (one XCD, hence one L2) and next to each other in launch order.
struct UnitPart {
  int chunk, head, part;
};
__device__ inline UnitPart unit_part(const ChunkedArgs& a, int parts) {
  const int units = a.chunks * a.vh, b = blockIdx.x;
  int unit = b / parts, part = b % parts;
  if (units % 8 == 0) {
    part = (b / 8) % parts;
    unit = (b / (8 * parts)) * 8 + b % 8;
  }
  return {unit % a.chunks, unit / a.chunks, part};
}

// Rows of dO and V; tokens beyond the sequence read as zero.
__device__ inline float4 d_out4(const ChunkedArgs& a, const ChunkView& v, int i, int c) {
  const int t = v.t0 + i, row = min(t, a.length - 1);
  return keep(t < a.length, load4(a.dcore + (static_cast<size_t>(row) * a.vh + v.head) * kD + c));
}
__device__ inline float d_out1(const ChunkedArgs& a, const ChunkView& v, int i, int c) {
  const int t = v.t0 + i, row = min(t, a.length - 1);
  return keep(t < a.length, a.dcore[(static_cast<size_t>(row) * a.vh + v.head) * kD + c]);
}
__device__ inline float4 value4(const ChunkedArgs& a, const ChunkView& v, int j, int c) {
  const int t = v.t0 + j, row = min(t, a.length - 1);
  return keep(t < a.length, load4(a.post + static_cast<size_t>(row) * v.channels + v.value_offset + c));
}
__device__ inline float value1(const ChunkedArgs& a, const ChunkView& v, int j, int c) {
  const int t = v.t0 + j, row = min(t, a.length - 1);
  return keep(t < a.length, a.post[static_cast<size_t>(row) * v.channels + v.value_offset + c]);
}

// dDl = P^T dO + diag(L) K^ dS'
__global__ void __launch_bounds__(256)
chunk_delta_gradient_kernel(ChunkedArgs a) {
  const ChunkView v = chunk_view(a, blockIdx.x, blockIdx.y);
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int h = lane / 32, n = lane % 32, col = 32 * wave + n;
#pragma unroll
  for (int ti = 0; ti < 2; ++ti) {
    const int m = 32 * ti + n;
    floatx16 acc = product<kC, true>(zero_tile(), [&](int k) { return v.P[k * kC + m]; },
                               [&](int k) { return d_out1(a, v, k, col); });
    const float l = v.gates[5 * kC + m];
    acc = product4<kD, true>(acc, [&](int k) { return scaled(load4(v.K + m * kD + k), l); },
                       [&](int k) { return gather4(v.dS1 + k * kD + col, kD); });
#pragma unroll
    for (int i = 0; i < 16; ++i) a.r.ddl[v.rec * kWide + (32 * ti + tile_row(i, h)) * kD + col] = acc[i];
  }
}

// Products against the two states, one per part of a unit:
//   0: dW = -dDl S^T
//   1: diag(E) dO S^T (the first part of dq^) and its row sums against q^
//   2: diag(L) Dl dS'^T (the first part of dk^), its row sums against k^, <dS', S>
// Both operands are contiguous along the contraction and are read in 16-byte
// pieces, one row a lane.  (Staging them in LDS with coalesced loads first
// measured the same 88 us: the kernel moves 270 MB.)
__global__ void __launch_bounds__(256)
chunk_state_products_kernel(ChunkedArgs a) {
  __shared__ float parts[kC][4];
  __shared__ float reduce[256];
  const UnitPart u = unit_part(a, 3);
  const ChunkView v = chunk_view(a, u.chunk, u.head);
  const int which = u.part;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int h = lane / 32, n = lane % 32, col = 32 * wave + n;
  const float* dDl = a.r.ddl + v.rec * kWide;
  float* sums = a.r.sums + v.rec * kSumRows * kC;
  const float* state = which == 2 ? v.dS1 : v.S0;
  float* target = (which == 0 ? a.r.dwm : which == 1 ? a.r.dqp : a.r.dkp) + v.rec * kWide;
  const float* against = which == 1 ? v.Q : v.K;
  float dot = 0.0f;
  if (which == 2) {
    const int c4 = 4 * (tid % 32);
#pragma unroll
    for (int j = 0; j < kD / 8; ++j) {
      const int row = tid / 32 + 8 * j;
      const float4 x = load4(v.S0 + row * kD + c4), y = load4(v.dS1 + row * kD + c4);
      dot += (x.x * y.x + x.y * y.y) + (x.z * y.z + x.w * y.w);
    }
  }
  reduce[tid] = dot;
#pragma unroll
  for (int ti = 0; ti < 2; ++ti) {
    const int m = 32 * ti + n;
    const float factor = which == 0 ? -1.0f : v.gates[(which == 1 ? 4 : 5) * kC + m];
    const floatx16 acc = product4<kD, true>(
        zero_tile(),
        [&](int k) {
          const float4 row = which == 0   ? load4(dDl + m * kD + k)
                             : which == 1 ? d_out4(a, v, m, k)
                                          : load4(v.Dl + m * kD + k);
          return scaled(row, factor);
        },
        [&](int k) { return load4(state + col * kD + k); });
    float weighted[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      target[row * kD + col] = acc[i];
      weighted[i] = which != 0 ? acc[i] * against[row * kD + col] : 0.0f;
    }
    if (which != 0) {
      half_sums(weighted);
      if (n == 0) {
#pragma unroll
        for (int i = 0; i < 16; ++i) parts[32 * ti + tile_row(i, h)][wave] = weighted[i];
      }
    }
  }
  if (which == 0) return;
  __syncthreads();
  if (tid < kC) sums[(which - 1) * kC + tid] = across_waves(parts, tid);
  if (which == 2 && tid == 0) {
    float total = 0.0f;
    for (int j = 0; j < 256; ++j) total += reduce[j];
    sums[6 * kC] = total;
  }
}

// The [64, 64] part: dP = lower(dO Dl^T), dT = dW (diag(beta E) K^)^T +
// dDl (diag(beta) V)^T, dA = -strict_lower(T^T dT T^T); leaves Pd = dP D and
// R = diag(beta) dA D in the records, and the row and column sums that feed
// d beta and d log-decay.
__global__ void __launch_bounds__(256)
chunk_triangle_kernel(ChunkedArgs a) {
  __shared__ float mx[kC][kC + 1], mz[kC][kC + 1], mu[kC][kC + 1];
  __shared__ float g_s[kC], beta_s[kC];
  const ChunkView v = chunk_view(a, blockIdx.x, blockIdx.y);
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int h = lane / 32, n = lane % 32;
  const int ti = wave / 2, tj = wave % 2;
  const float* dDl = a.r.ddl + v.rec * kWide;
  const float* dW = a.r.dwm + v.rec * kWide;
  float* sums = a.r.sums + v.rec * kSumRows * kC;
  if (tid < kC) {
    g_s[tid] = v.gates[tid];
    beta_s[tid] = v.gates[kC + tid];
  }
  __syncthreads();
  const int col = 32 * tj + n;
  {
    floatx16 dp = zero_tile();
    if (ti >= tj)
      dp = product4<kD>(dp, [&](int k) { return d_out4(a, v, 32 * ti + n, k); },
                        [&](int k) { return load4(v.Dl + col * kD + k); });
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      const bool lower = row >= col;
      const float value = lower ? dp[i] : 0.0f;
      a.r.pd[v.rec * kSquare + row * kC + col] = lower ? value * expf(g_s[row] - g_s[col]) : 0.0f;
      mu[row][col] = value * v.P[row * kC + col];
    }
  }
  {
    const float fv = beta_s[col], fk = fv * v.gates[4 * kC + col];
    floatx16 acc = product4<kD>(zero_tile(), [&](int k) { return load4(dW + (32 * ti + n) * kD + k); },
                                [&](int k) { return scaled(load4(v.K + col * kD + k), fk); });
    acc = product4<kD>(acc, [&](int k) { return load4(dDl + (32 * ti + n) * kD + k); },
                       [&](int k) { return scaled(value4(a, v, col, k), fv); });
#pragma unroll
    for (int i = 0; i < 16; ++i) mx[32 * ti + tile_row(i, h)][col] = acc[i];
  }
  __syncthreads();
  {
    const floatx16 acc = product<kC>(zero_tile(), [&](int k) { return v.Tm[k * kC + 32 * ti + n]; },
                                     [&](int k) { return mx[k][col]; });
#pragma unroll
    for (int i = 0; i < 16; ++i) mz[32 * ti + tile_row(i, h)][col] = acc[i];
  }
  __syncthreads();
  {
    floatx16 acc = zero_tile();
    if (ti >= tj)
      acc = product<kC>(acc, [&](int k) { return -mz[32 * ti + n][k]; },
                        [&](int k) { return v.Tm[col * kC + k]; });
    __syncthreads();  // X has been read by every wave
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      const bool lower = row > col;
      const float da = lower ? acc[i] : 0.0f;
      mz[row][col] = da * v.KKD[row * kC + col];  // N
      a.r.rr[v.rec * kSquare + row * kC + col] =
          lower ? da * beta_s[row] * expf(g_s[row] - g_s[col]) : 0.0f;
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
    sums[2 * kC + tid] = row_n;
    sums[3 * kC + tid] = col_m;
    sums[4 * kC + tid] = row_p;
    sums[5 * kC + tid] = col_p;
  }
}

// dq and dk (back through the normalisations) and dv of 32 rows of a chunk
// (the unit's part picks the row tile), and the row sums of those rows that the
// gate gradients need.
__global__ void __launch_bounds__(256)
chunk_finish_kernel(ChunkedArgs a) {
  __shared__ float parts[4][kC / 2][4];
  __shared__ float e_s[kC], beta_s[kC];
  const UnitPart u = unit_part(a, 2);
  const ChunkView v = chunk_view(a, u.chunk, u.head);
  const int ti = u.part;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int h = lane / 32, n = lane % 32, col = 32 * wave + n;
  const float* dDl = a.r.ddl + v.rec * kWide;
  const float* dW = a.r.dwm + v.rec * kWide;
  const float* Pd = a.r.pd + v.rec * kSquare;
  const float* R = a.r.rr + v.rec * kSquare;
  float* sums = a.r.sums + v.rec * kSumRows * kC;
  if (tid < kC) {
    e_s[tid] = v.gates[4 * kC + tid];
    beta_s[tid] = v.gates[kC + tid];
  }
  __syncthreads();
  const int m = 32 * ti + n;
  floatx16 dq, dk;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int row = 32 * ti + tile_row(i, h);
    dq[i] = a.r.dqp[v.rec * kWide + row * kD + col];
    dk[i] = a.r.dkp[v.rec * kWide + row * kD + col];
  }
  // dq^ += Pd K^
  dq = product4<kC>(dq, [&](int k) { return load4(Pd + m * kC + k); },
                    [&](int k) { return gather4(v.K + k * kD + col, kD); });
  // T^T dW = d(diag(beta E) K^)
  const floatx16 tw = product<kC>(zero_tile(), [&](int k) { return v.Tm[k * kC + m]; },
                                  [&](int k) { return dW[k * kD + col]; });
  {
    float weighted[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h);
      weighted[i] = tw[i] * v.K[row * kD + col] * e_s[row];
      dk[i] += beta_s[row] * e_s[row] * tw[i];
    }
    half_sums(weighted);
    if (n == 0) {
#pragma unroll
      for (int i = 0; i < 16; ++i) parts[0][tile_row(i, h)][wave] = weighted[i];
    }
  }
  // dk^ += (R + R^T) K^ + Pd^T Q^
  dk = product4<kC>(dk, [&](int k) { return load4(R + m * kC + k); },
                    [&](int k) { return gather4(v.K + k * kD + col, kD); });
  dk = product<kC>(dk, [&](int k) { return R[k * kC + m]; },
                   [&](int k) { return v.K[k * kD + col]; });
  dk = product<kC>(dk, [&](int k) { return Pd[k * kC + m]; },
                   [&](int k) { return v.Q[k * kD + col]; });
  // dv = diag(beta) T^T dDl
  const floatx16 tu = product<kC>(zero_tile(), [&](int k) { return v.Tm[k * kC + m]; },
                                  [&](int k) { return dDl[k * kD + col]; });
  {
    float rv[16], q_dot[16], k_dot[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + tile_row(i, h), t = v.t0 + row;
      rv[i] = tu[i] * value1(a, v, row, col);
      q_dot[i] = dq[i] * v.Q[row * kD + col];
      k_dot[i] = dk[i] * v.K[row * kD + col];
      if (t < a.length)
        a.dpost[static_cast<size_t>(t) * v.channels + v.value_offset + col] = beta_s[row] * tu[i];
    }
    half_sums(rv);
    half_sums(q_dot);
    half_sums(k_dot);
    if (n == 0) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int local = tile_row(i, h);
        parts[1][local][wave] = rv[i];
        parts[2][local][wave] = q_dot[i];
        parts[3][local][wave] = k_dot[i];
      }
    }
  }
  __syncthreads();
  // back through the L2 normalisations (and the 1/sqrt(d) of q)
  const float norm_scale = sqrtf(static_cast<float>(kD));
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int local = tile_row(i, h), row = 32 * ti + local, t = v.t0 + row;
    if (t >= a.length) continue;
    const float iq = v.gates[2 * kC + row], ik = v.gates[3 * kC + row];
    const float qv = v.Q[row * kD + col], kv = v.K[row * kD + col];
    float* out = a.qk_partials + (static_cast<size_t>(t) * a.vh + v.head) * 2 * kD;
    out[col] = iq / norm_scale *
               (dq[i] - static_cast<float>(kD) * qv * across_waves(parts[2], local));
    out[kD + col] = ik * (dk[i] - kv * across_waves(parts[3], local));
  }
  if (tid < kC / 2) {
    sums[7 * kC + 32 * ti + tid] = across_waves(parts[0], tid);
    sums[8 * kC + 32 * ti + tid] = across_waves(parts[1], tid);
  }
}

// d log-decay and d beta of the 64 tokens of a chunk from the row and column
// sums the other kernels left, then through the gates to da, db and the
// contribution to d A_log.
__global__ void __launch_bounds__(64)
chunk_gates_kernel(ChunkedArgs a) {
  __shared__ float dg_s[kC];
  const ChunkView v = chunk_view(a, blockIdx.x, blockIdx.y);
  const float* sums = a.r.sums + v.rec * kSumRows * kC;
  const int tid = threadIdx.x;
  const float beta = v.gates[kC + tid];
  const float r = sums[7 * kC + tid];
  float dG = sums[tid] + beta * r + (beta * sums[2 * kC + tid] - sums[3 * kC + tid]) +
             (sums[4 * kC + tid] - sums[5 * kC + tid]) - sums[kC + tid];
  if (tid == kC - 1) {
    float total = 0.0f;
    for (int j = 0; j < kC; ++j) total += sums[kC + j];
    dG += total + sums[6 * kC] * v.gates[4 * kC + kC - 1];
  }
  dg_s[tid] = dG;
  __syncthreads();
  const int t = v.t0 + tid;
  if (t >= a.length) return;
  float dg = 0.0f;
  for (int i = kC - 1; i >= tid; --i) dg += dg_s[i];
  const float dbeta = sums[2 * kC + tid] + r + sums[8 * kC + tid];
  const float alpha = bf16_bits_to_float(a.a[static_cast<size_t>(t) * a.vh + v.head]) + a.dt_bias[v.head];
  const float softplus = fmaxf(alpha, 0.0f) + logf(1.0f + expf(-fabsf(alpha)));
  const float rate = expf(a.a_log[v.head]);
  const float bv = bf16_bits_to_float(a.b[static_cast<size_t>(t) * a.vh + v.head]);
  const float sigmoid = 1.0f / (1.0f + expf(-bv));
  float* out = a.scalar_partials + (static_cast<size_t>(t) * a.vh + v.head) * 3;
  out[0] = -dg * rate / (1.0f + expf(-alpha));
  out[1] = dbeta * sigmoid * (1.0f - sigmoid);
  out[2] = -dg * rate * softplus;
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
  a.r.ddl = take(kWide);
  a.r.dwm = take(kWide);
  a.r.dqp = take(kWide);
  a.r.dkp = take(kWide);
  a.r.p = take(kSquare);
  a.r.tm = take(kSquare);
  a.r.kkd = take(kSquare);
  a.r.pd = take(kSquare);
  a.r.rr = take(kSquare);
  a.r.sums = take(kSumRows * kC);
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
  chunk_delta_gradient_kernel<<<per_chunk, 256, 0, stream>>>(a);
  status = launch_status();
  if (status != 0) return status;
  chunk_state_products_kernel<<<a.chunks * a.vh * 3, 256, 0, stream>>>(a);
  status = launch_status();
  if (status != 0) return status;
  chunk_triangle_kernel<<<per_chunk, 256, 0, stream>>>(a);
  status = launch_status();
  if (status != 0) return status;
  chunk_finish_kernel<<<a.chunks * a.vh * 2, 256, 0, stream>>>(a);
  status = launch_status();
  if (status != 0) return status;
  chunk_gates_kernel<<<per_chunk, kC, 0, stream>>>(a);
  return launch_status();
}

}  // namespace pluto_hip
