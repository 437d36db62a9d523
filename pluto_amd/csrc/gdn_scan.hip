// Gated delta-net: chunked linear-attention scan for gfx950, plus the
// token-by-token recurrence.
//
// Recurrence (RecurrenceForward, src/llm/layers/sequence_delta_net.cc:55-102;
// DeltaRecurrenceKernel, src/llm/layers/util/cached_attention_ops.cc:205-251),
// per head, state S in R^{dk x dv}:
//     S <- a_t S;  d_t = b_t (v_t - S^T k_t);  S <- S + k_t d_t^T;  o_t = S^T q_t
// with a_t = exp(g_t) and b_t = beta_t.
//
// Chunked form used here (C = 64 tokens, c_i = g_1 + .. + g_i inside a chunk,
// S0 = state entering the chunk):
//     A[i,j]  = b_i exp(c_i - c_j) (k_i . k_j)        for j <  i
//     (I + A) U = diag(b) V,      (I + A) W = diag(b exp(c)) K
//     D  = U - W S0                                   (the d_t of the chunk)
//     O  = diag(exp(c)) Q S0 + (M o Q K^T) D,   M[i,j] = exp(c_i - c_j), j <= i
//     S  = exp(c_C) S0 + (diag(exp(c_C - c)) K)^T D
// Only differences c_i - c_j <= 0 are exponentiated, so nothing overflows.
//
// Kernel 1 (gdn_chunk_prepare, one workgroup per chunk, fully parallel): the
// two Gram matrices on the matrix cores from the raw bf16 inputs (normalisation
// and scale factors are applied afterwards in FP32), an FP32 forward
// substitution for [U | W] with one thread per column, and the operands of the
// sequential kernel written out in matrix-core register order.
// Kernel 2 (gdn_chunk_scan, one wave per (sequence, head, 16 state columns)):
// walks the chunks with v_mfma_f32_16x16x32_bf16, state kept in FP32
// accumulator registers; no barriers, no LDS.  State columns are independent,
// which is what gives the sequential part 8 x batch x heads way parallelism.
#include "gdn.h"

namespace pluto_hip {
namespace {

constexpr int C = 64;     // tokens per chunk
constexpr int DK = 128;   // key width of the chunked path
constexpr int DV = 128;   // value width of the chunked path
constexpr int SLICES = DV / 16;

typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;

__device__ inline bf16x8 bits_to_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

// Contraction-slot order of an operand that multiplies two stacked 16x16
// accumulator tiles: slot (hq, e) of 32-block kb is element
// 32*kb + 16*(e/4) + 4*hq + e%4 (see file header of mfma_tile.h for the
// 32x32 analogue).

struct ChunkSmem {
  uint16_t k[C][DK + 8];    // raw K rows (bf16)
  uint16_t q[C][DK + 8];    // raw Q rows
  uint16_t vw[C][DV + 8];   // V rows, later -W rows
  float a[C][C + 4];        // strictly lower triangular A (FP32)
  uint16_t a2[C][C + 8];    // M o (Q K^T) with all factors, bf16
  float cum[C];             // inclusive cumulative log decay
  float beta[C];
  float inv_k[C];           // 1/|k| (or 1)
  float q_factor[C];        // q_scale / |q| (or q_scale)
  float rhs_factor[2][C];   // [0]: beta (U columns), [1]: beta exp(c) / |k| (W columns)
};

__global__ void __launch_bounds__(256)
gdn_chunk_prepare(GdnArgs a) {
  __shared__ __attribute__((aligned(16))) ChunkSmem sm;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int chunks = (a.length + C - 1) / C;
  const int chunk = blockIdx.x % chunks;
  const int bh = blockIdx.x / chunks;            // sequence * value_heads + head
  const int head = bh % a.value_heads, seq = bh / a.value_heads;
  const int key_head = head / (a.value_heads / a.key_heads);
  const int t0 = chunk * C;
  const int valid = min(C, a.length - t0);

  // ---- stage K, Q, V rows (16-byte pieces), zero beyond the sequence -------
  for (int piece = tid; piece < C * (DK / 8); piece += 256) {
    const int row = piece / (DK / 8), c8 = piece % (DK / 8);
    uint4 kb = make_uint4(0, 0, 0, 0), qb = kb, vb = kb;
    if (row < valid) {
      const long long token = static_cast<long long>(seq) * a.length + t0 + row;
      kb = *reinterpret_cast<const uint4*>(a.k + token * a.k_token_stride + key_head * DK + 8 * c8);
      qb = *reinterpret_cast<const uint4*>(a.q + token * a.q_token_stride + key_head * DK + 8 * c8);
      vb = *reinterpret_cast<const uint4*>(a.v + token * a.v_token_stride + head * DV + 8 * c8);
    }
    *reinterpret_cast<uint4*>(&sm.k[row][8 * c8]) = kb;
    *reinterpret_cast<uint4*>(&sm.q[row][8 * c8]) = qb;
    *reinterpret_cast<uint4*>(&sm.vw[row][8 * c8]) = vb;
  }
  if (wave == 0) {
    float g = 0.0f, b = 0.0f;
    if (lane < valid) {
      const long long at = (static_cast<long long>(seq) * a.length + t0 + lane) * a.value_heads + head;
      g = a.log_decay[at];
      b = a.beta[at];
    }
    // inclusive prefix sum over the 64 lanes
    for (int offset = 1; offset < 64; offset <<= 1) {
      const float up = __shfl_up(g, offset, 64);
      if (lane >= offset) g += up;
    }
    sm.cum[lane] = g;
    sm.beta[lane] = b;
  }
  __syncthreads();
  {
    // row norms: 4 threads per row, 32 channels each
    const int row = tid / 4, part = tid % 4;
    float kk = 0.0f, qq = 0.0f;
    for (int c = 32 * part; c < 32 * part + 32; ++c) {
      const float kv = bf16_bits_to_float(sm.k[row][c]);
      const float qv = bf16_bits_to_float(sm.q[row][c]);
      kk += kv * kv;
      qq += qv * qv;
    }
    kk += __shfl_xor(kk, 1, 64);
    kk += __shfl_xor(kk, 2, 64);
    qq += __shfl_xor(qq, 1, 64);
    qq += __shfl_xor(qq, 2, 64);
    if (part == 0) {
      // sequence_delta_net.cc:84-85: x * rsqrt(sum(x^2) + 1e-6)
      const float inv_k = a.normalize_qk ? rsqrtf(kk + 1e-6f) : 1.0f;
      sm.inv_k[row] = inv_k;
      sm.q_factor[row] = a.normalize_qk ? a.q_scale * rsqrtf(qq + 1e-6f) : a.q_scale;
      sm.rhs_factor[0][row] = sm.beta[row];
      sm.rhs_factor[1][row] = sm.beta[row] * __expf(sm.cum[row]) * inv_k;
    }
  }
  __syncthreads();

  // ---- Gram matrices on the matrix cores: wave (ti, tj) owns a 32x32 tile --
  {
    const int ti = wave / 2, tj = wave % 2;
    const int h = lane / 32, n = lane % 32;
    if (tj <= ti) {
      floatx16 gk, gq;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        gk[i] = 0.0f;
        gq[i] = 0.0f;
      }
#pragma unroll
      for (int ks = 0; ks < DK / 16; ++ks) {
        const bf16x8 kr = bits_to_bf16x8(*reinterpret_cast<const uint4*>(&sm.k[32 * ti + n][16 * ks + 8 * h]));
        const bf16x8 qr = bits_to_bf16x8(*reinterpret_cast<const uint4*>(&sm.q[32 * ti + n][16 * ks + 8 * h]));
        const bf16x8 kc = bits_to_bf16x8(*reinterpret_cast<const uint4*>(&sm.k[32 * tj + n][16 * ks + 8 * h]));
        gk = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kr, kc, gk, 0, 0, 0);
        gq = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qr, kc, gq, 0, 0, 0);
      }
      const int col = 32 * tj + n;  // token j
      const float cum_j = sm.cum[col], inv_kj = sm.inv_k[col];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = 32 * ti + 8 * (i / 4) + 4 * h + (i % 4);  // token i
        const float decay = __expf(fminf(sm.cum[row] - cum_j, 0.0f));
        float av = 0.0f, a2v = 0.0f;
        if (col < row) av = sm.beta[row] * decay * sm.inv_k[row] * inv_kj * gk[i];
        if (col <= row) a2v = decay * sm.q_factor[row] * inv_kj * gq[i];
        sm.a[row][col] = av;
        sm.a2[row][col] = float_to_bf16_bits(a2v);
      }
    } else {
      for (int i = lane; i < 32 * 32; i += 64) {
        const int row = 32 * ti + i / 32, col = 32 * tj + i % 32;
        sm.a[row][col] = 0.0f;
        sm.a2[row][col] = 0;
      }
    }
  }
  __syncthreads();

  // ---- forward substitution, one thread per column of [U | W] -------------
  float x[C];
  {
    const bool is_u = tid < DV;
    const int c = is_u ? tid : tid - DV;
    const uint16_t* column = is_u ? &sm.vw[0][c] : &sm.k[0][c];  // same row stride
    const float* factor = sm.rhs_factor[is_u ? 0 : 1];
#pragma unroll
    for (int i = 0; i < C; ++i) {
      const float rhs = factor[i] * bf16_bits_to_float(column[i * (DK + 8)]);
      // four partial sums shorten the dependent chain of a row
      float acc0 = rhs, acc1 = 0.0f, acc2 = 0.0f, acc3 = 0.0f;
#pragma unroll
      for (int j4 = 0; j4 < (i + 3) / 4; ++j4) {
        const float4 row = *reinterpret_cast<const float4*>(&sm.a[i][4 * j4]);
        // entries at or beyond the diagonal are zero
        acc0 -= row.x * x[4 * j4];
        if (4 * j4 + 1 < i) acc1 -= row.y * x[4 * j4 + 1];
        if (4 * j4 + 2 < i) acc2 -= row.z * x[4 * j4 + 2];
        if (4 * j4 + 3 < i) acc3 -= row.w * x[4 * j4 + 3];
      }
      const float acc = (acc0 + acc1) + (acc2 + acc3);
      // keep the scheduler from hoisting later rows' LDS reads over this row:
      // that only lengthens live ranges until registers spill
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      x[i] = acc;
    }
  }
  char* out = a.workspace + (static_cast<size_t>(bh) * chunks + chunk) * kGdnChunkBytes;
  float* u_out = reinterpret_cast<float*>(out + kGdnOffsetU);
  __syncthreads();  // everyone is done reading V before -W overwrites it
  if (tid < DV) {
    // U in accumulator order: [tile i][slice][lane = 16*hq + m][r]
    const int slice = tid / 16, m = tid % 16;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int hq = 0; hq < 4; ++hq) {
        const float4 value = make_float4(x[16 * i + 4 * hq], x[16 * i + 4 * hq + 1],
                                         x[16 * i + 4 * hq + 2], x[16 * i + 4 * hq + 3]);
        *reinterpret_cast<float4*>(u_out + ((i * SLICES + slice) * 64 + 16 * hq + m) * 4) = value;
      }
  } else {
    const int c = tid - DV;
#pragma unroll
    for (int i = 0; i < C; ++i) sm.vw[i][c] = float_to_bf16_bits(-x[i]);
  }
  __syncthreads();

  // ---- operand fragments for the sequential kernel --------------------------
  const float cum_last = sm.cum[C - 1];
  uint4* neg_w = reinterpret_cast<uint4*>(out + kGdnOffsetW);
  uint4* q_out = reinterpret_cast<uint4*>(out + kGdnOffsetQ);
  uint4* a2_out = reinterpret_cast<uint4*>(out + kGdnOffsetA2);
  uint4* kt_out = reinterpret_cast<uint4*>(out + kGdnOffsetKt);
  // -W and exp(c) Q: fragment f = 4*tile + kb, 64 lanes each
  for (int piece = tid; piece < 16 * 64; piece += 256) {
    const int f = piece / 64, l = piece % 64;
    const int tile = f / 4, kb = f % 4, hq = l / 16, m = l % 16;
    const int row = 16 * tile + m, lo = 32 * kb + 4 * hq;
    uint2 w0 = *reinterpret_cast<const uint2*>(&sm.vw[row][lo]);
    uint2 w1 = *reinterpret_cast<const uint2*>(&sm.vw[row][lo + 16]);
    neg_w[piece] = make_uint4(w0.x, w0.y, w1.x, w1.y);
    const float factor = sm.q_factor[row] * __expf(sm.cum[row]);
    uint16_t packed[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int col = lo + 16 * (e / 4) + (e % 4);
      packed[e] = float_to_bf16_bits(factor * bf16_bits_to_float(sm.q[row][col]));
    }
    q_out[piece] = *reinterpret_cast<const uint4*>(packed);
  }
  // M o (Q K^T): fragment f = 2*tile + kb (contraction over tokens j)
  for (int piece = tid; piece < 8 * 64; piece += 256) {
    const int f = piece / 64, l = piece % 64;
    const int tile = f / 2, kb = f % 2, hq = l / 16, m = l % 16;
    const int row = 16 * tile + m, lo = 32 * kb + 4 * hq;
    uint2 w0 = *reinterpret_cast<const uint2*>(&sm.a2[row][lo]);
    uint2 w1 = *reinterpret_cast<const uint2*>(&sm.a2[row][lo + 16]);
    a2_out[piece] = make_uint4(w0.x, w0.y, w1.x, w1.y);
  }
  // (diag(exp(c_C - c)) K)^T: rows = key channels, contraction over tokens
  for (int piece = tid; piece < 16 * 64; piece += 256) {
    const int f = piece / 64, l = piece % 64;
    const int tile = f / 2, kb = f % 2, hq = l / 16, m = l % 16;
    const int channel = 16 * tile + m, lo = 32 * kb + 4 * hq;
    uint16_t packed[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int token = lo + 16 * (e / 4) + (e % 4);
      const float factor = __expf(cum_last - sm.cum[token]) * sm.inv_k[token];
      packed[e] = float_to_bf16_bits(factor * bf16_bits_to_float(sm.k[token][channel]));
    }
    kt_out[piece] = *reinterpret_cast<const uint4*>(packed);
  }
  if (tid == 0) *reinterpret_cast<float*>(out + kGdnOffsetDecay) = __expf(cum_last);
}

__device__ inline floatx4 mfma16(bf16x8 a, bf16x8 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Two stacked accumulator tiles as the B operand of a 32-deep product.
__device__ inline bf16x8 tiles_to_operand(const floatx4& lo, const floatx4& hi) {
  bf16x8 out;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    out[e] = static_cast<__bf16>(lo[e]);
    out[4 + e] = static_cast<__bf16>(hi[e]);
  }
  return out;
}

__global__ void __launch_bounds__(64)
gdn_chunk_scan(GdnArgs a) {
  const int lane = threadIdx.x, hq = lane / 16, m = lane % 16;
  const int chunks = (a.length + C - 1) / C;
  // The 8 column slices of one (sequence, head) read the same operands: keep
  // them on one XCD so its L2 serves 7 of the 8 reads.
  int logical = blockIdx.x;
  if (gridDim.x % 8 == 0) logical = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
  const int slice = logical % SLICES;
  const int bh = logical / SLICES;
  const int head = bh % a.value_heads, seq = bh / a.value_heads;
  float* state = a.state + static_cast<size_t>(bh) * DK * DV;

  floatx4 s[8];  // rows 16t + 4hq + r, column 16*slice + m
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      s[t][r] = state[(16 * t + 4 * hq + r) * DV + 16 * slice + m];

  // Operands are fetched half an iteration ahead: the first-phase operands
  // (U, -W, cQ) of chunk c+1 are requested before the second phase of chunk c
  // runs, and the second-phase operands (A2, Kt) of chunk c before its first
  // phase, so the dependent matrix-core chain does not wait on memory.
  floatx4 u_reg[4];
  uint4 w_reg[16], q_reg[16], a2_reg[8], kt_reg[16];
  float decay = 1.0f;
  const char* base = a.workspace + static_cast<size_t>(bh) * chunks * kGdnChunkBytes;
  auto load_first = [&](int chunk) {
    const char* in = base + static_cast<size_t>(chunk) * kGdnChunkBytes;
    const floatx4* u_in = reinterpret_cast<const floatx4*>(in + kGdnOffsetU);
    const uint4* neg_w = reinterpret_cast<const uint4*>(in + kGdnOffsetW);
    const uint4* q_in = reinterpret_cast<const uint4*>(in + kGdnOffsetQ);
#pragma unroll
    for (int i = 0; i < 4; ++i) u_reg[i] = u_in[(i * SLICES + slice) * 64 + lane];
#pragma unroll
    for (int f = 0; f < 16; ++f) {
      w_reg[f] = neg_w[f * 64 + lane];
      q_reg[f] = q_in[f * 64 + lane];
    }
  };
  auto load_second = [&](int chunk) {
    const char* in = base + static_cast<size_t>(chunk) * kGdnChunkBytes;
    const uint4* a2_in = reinterpret_cast<const uint4*>(in + kGdnOffsetA2);
    const uint4* kt_in = reinterpret_cast<const uint4*>(in + kGdnOffsetKt);
#pragma unroll
    for (int f = 0; f < 8; ++f) a2_reg[f] = a2_in[f * 64 + lane];
#pragma unroll
    for (int f = 0; f < 16; ++f) kt_reg[f] = kt_in[f * 64 + lane];
    decay = *reinterpret_cast<const float*>(in + kGdnOffsetDecay);
  };
  load_first(0);
  for (int chunk = 0; chunk < chunks; ++chunk) {
    load_second(chunk);
    bf16x8 sb[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) sb[kb] = tiles_to_operand(s[2 * kb], s[2 * kb + 1]);
    // D = U - W S0 and the S0 part of O = exp(c) Q S0 + (M o Q K^T) D
    floatx4 d[4], o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      floatx4 acc = u_reg[i];
      floatx4 out_acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        acc = mfma16(bits_to_bf16x8(w_reg[4 * i + kb]), sb[kb], acc);
        out_acc = mfma16(bits_to_bf16x8(q_reg[4 * i + kb]), sb[kb], out_acc);
      }
      d[i] = acc;
      o[i] = out_acc;
    }
    if (chunk + 1 < chunks) load_first(chunk + 1);
    bf16x8 db[2];
    db[0] = tiles_to_operand(d[0], d[1]);
    db[1] = tiles_to_operand(d[2], d[3]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      floatx4 acc = o[i];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
        acc = mfma16(bits_to_bf16x8(a2_reg[2 * i + kb]), db[kb], acc);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int token = chunk * C + 16 * i + 4 * hq + r;
        if (token < a.length)
          a.out[((static_cast<long long>(seq) * a.length + token) * a.value_heads + head) * DV +
                16 * slice + m] = float_to_bf16_bits(acc[r]);
      }
    }
    // S = exp(c_C) S0 + (diag(exp(c_C - c)) K)^T D
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      floatx4 acc = s[t] * decay;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
        acc = mfma16(bits_to_bf16x8(kt_reg[2 * t + kb]), db[kb], acc);
      s[t] = acc;
    }
  }
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      state[(16 * t + 4 * hq + r) * DV + 16 * slice + m] = s[t][r];
}

// Token-by-token recurrence, any widths up to 128 x 256: one workgroup per
// (sequence, head), one thread per state column, the column's state in
// registers.  This is the reference's own loop structure
// (sequence_delta_net.cc:79-101); it serves shapes the chunked path does not
// specialise and cross-checks the chunked scan on the device.
__global__ void __launch_bounds__(256)
gdn_recurrence_kernel(GdnArgs a, int out_dtype) {
  __shared__ float ks[128];
  __shared__ float qs[128];
  const int bh = blockIdx.x;
  const int head = bh % a.value_heads, seq = bh / a.value_heads;
  const int key_head = head / (a.value_heads / a.key_heads);
  const int kd = a.key_dim, vd = a.value_dim;
  const int column = threadIdx.x;
  const bool active = column < vd;
  float* state = a.state + static_cast<size_t>(bh) * kd * vd;
  float s[128];
#pragma unroll
  for (int d = 0; d < 128; ++d) s[d] = (d < kd && active) ? state[d * vd + column] : 0.0f;
  for (int t = 0; t < a.length; ++t) {
    const long long token = static_cast<long long>(seq) * a.length + t;
    __syncthreads();
    if (threadIdx.x < 128) {
      const int d = threadIdx.x;
      ks[d] = d < kd ? load_element(a.k, token * a.k_token_stride + key_head * kd + d, a.in_dtype) : 0.0f;
      qs[d] = d < kd ? load_element(a.q, token * a.q_token_stride + key_head * kd + d, a.in_dtype) : 0.0f;
    }
    __syncthreads();
    float k_factor = 1.0f, q_factor = a.q_scale;
    if (a.normalize_qk) {
      float kk = 1e-6f, qq = 1e-6f;
      for (int d = 0; d < kd; ++d) {
        kk += ks[d] * ks[d];
        qq += qs[d] * qs[d];
      }
      k_factor = rsqrtf(kk);
      q_factor = a.q_scale * rsqrtf(qq);
    }
    const long long scalar = token * a.value_heads + head;
    const float decay = __expf(a.log_decay[scalar]);
    const float beta = a.beta[scalar];
    float value = 0.0f;
    if (active) value = load_element(a.v, token * a.v_token_stride + head * vd + column, a.in_dtype);
    float prediction = 0.0f;
#pragma unroll
    for (int d = 0; d < 128; ++d) {
      if (d < kd) {
        s[d] *= decay;
        prediction += s[d] * (ks[d] * k_factor);
      }
    }
    const float delta = (value - prediction) * beta;
    float output = 0.0f;
#pragma unroll
    for (int d = 0; d < 128; ++d) {
      if (d < kd) {
        s[d] += (ks[d] * k_factor) * delta;
        output += s[d] * (qs[d] * q_factor);
      }
    }
    if (active) {
      const long long at = (token * a.value_heads + head) * vd + column;
      if (out_dtype == PLUTO_HIP_BF16)
        static_cast<uint16_t*>(a.out_any)[at] = float_to_bf16_bits(output);
      else
        static_cast<float*>(a.out_any)[at] = a.round_output ? round_to_bf16(output) : output;
    }
  }
#pragma unroll
  for (int d = 0; d < 128; ++d)
    if (d < kd && active) state[d * vd + column] = s[d];
}

}  // namespace

bool gdn_chunked_supported(const GdnArgs& a, int chunk) {
  auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
  return chunk == C && a.key_dim == DK && a.value_dim == DV && a.in_dtype == PLUTO_HIP_BF16 &&
         a.q_token_stride % 8 == 0 && a.k_token_stride % 8 == 0 && a.v_token_stride % 8 == 0 &&
         aligned(a.q) && aligned(a.k) && aligned(a.v) && aligned(a.workspace);
}

int launch_gdn_chunked(hipStream_t stream, const GdnArgs& a) {
  const long long chunks = (a.length + C - 1) / C;
  const long long heads = static_cast<long long>(a.batch) * a.value_heads;
  if (heads * chunks > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  gdn_chunk_prepare<<<static_cast<unsigned>(heads * chunks), 256, 0, stream>>>(a);
  int status = launch_status();
  if (status != 0) return status;
  gdn_chunk_scan<<<static_cast<unsigned>(heads * SLICES), 64, 0, stream>>>(a);
  return launch_status();
}

int launch_gdn_recurrence(hipStream_t stream, const GdnArgs& a, int out_dtype) {
  if (a.key_dim > 128 || a.value_dim > 256) return PLUTO_HIP_EUNSUPPORTED;
  gdn_recurrence_kernel<<<a.batch * a.value_heads, 256, 0, stream>>>(a, out_dtype);
  return launch_status();
}

}  // namespace pluto_hip
