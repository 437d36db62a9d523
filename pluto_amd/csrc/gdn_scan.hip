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

// Two stacked accumulator tiles as a pair of B (or, read the other way, A)
// operands whose sum carries about 16 mantissa bits: hi = bf16(v), lo =
// bf16(v - hi).
__device__ inline void split_operand(const floatx4& first, const floatx4& second, bf16x8& hi,
                                     bf16x8& lo) {
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float v = e < 4 ? first[e] : second[e - 4];
    const __bf16 h = static_cast<__bf16>(v);
    hi[e] = h;
    lo[e] = static_cast<__bf16>(v - static_cast<float>(h));
  }
}

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

  // ---- (I + A) [U | W] = right-hand sides, by blocks of 16 rows on the matrix
  // cores.  With T_b the inverse of diagonal block b of I + A,
  //   X_b = T_b (R_b - sum_{k<b} A_bk X_k).
  // Every factor enters as a sum of two bf16 numbers (value = hi + lo, products
  // hi*hi + lo*hi + hi*lo), which keeps the result to about 2^-16 relative.
  //
  // T_b by forward substitution on the identity: wave b, lane = column; the
  // result replaces the diagonal block of A, which nothing else reads.
  if (lane < 16) {
    const int base = 16 * wave;
    float t[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float acc = (i == lane) ? 1.0f : 0.0f;
#pragma unroll
      for (int j4 = 0; j4 < (i + 3) / 4; ++j4) {
        const float4 row = *reinterpret_cast<const float4*>(&sm.a[base + i][base + 4 * j4]);
        acc -= row.x * t[4 * j4];
        if (4 * j4 + 1 < i) acc -= row.y * t[4 * j4 + 1];
        if (4 * j4 + 2 < i) acc -= row.z * t[4 * j4 + 2];
        if (4 * j4 + 3 < i) acc -= row.w * t[4 * j4 + 3];
      }
      t[i] = acc;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) sm.a[base + i][base + lane] = t[i];
  }
  __syncthreads();

  // Wave w solves columns 64 (w % 2) .. +63 of U (w < 2) or of W, four column
  // tiles of 16.  x[b][ct] is the 16x16 tile of block b in accumulator order:
  // lane (hq, m) holds rows 16 b + 4 hq + r of column 16 ct + m.
  floatx4 x[4][4];
  const bool is_u = wave < 2;
  const int col0 = 64 * (wave % 2);
  {
    const int hq = lane / 16, m = lane % 16;
    const uint16_t(*source)[DK + 8] = is_u ? sm.vw : sm.k;  // same row stride
    const float* factor = sm.rhs_factor[is_u ? 0 : 1];
    const floatx4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    bf16x8 pair_hi[4], pair_lo[4];  // blocks 0 and 1 stacked, as B operands
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      floatx4 r[4];
#pragma unroll
      for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int row = 16 * b + 4 * hq + e;
          r[ct][e] = factor[row] * bf16_bits_to_float(source[row][col0 + 16 * ct + m]);
        }
      // R_b -= [A_b,k0 | A_b,k1] [X_k0; X_k1]: contraction slot (hq, e) is row
      // 4 hq + e % 4 of block k0 (e < 4) or k1
#pragma unroll
      for (int k0 = 0; k0 < b; k0 += 2) {
        const bool both = k0 + 1 < b;
        const float4 first = *reinterpret_cast<const float4*>(&sm.a[16 * b + m][16 * k0 + 4 * hq]);
        float4 second = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (both) second = *reinterpret_cast<const float4*>(&sm.a[16 * b + m][16 * k0 + 16 + 4 * hq]);
        bf16x8 a_hi, a_lo;
        split_operand(floatx4{-first.x, -first.y, -first.z, -first.w},
                      floatx4{-second.x, -second.y, -second.z, -second.w}, a_hi, a_lo);
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) {
          bf16x8 b_hi, b_lo;
          if (k0 == 0 && both) {
            b_hi = pair_hi[ct];
            b_lo = pair_lo[ct];
          } else {
            split_operand(x[k0][ct], zero, b_hi, b_lo);
          }
          r[ct] = mfma16(a_hi, b_hi, r[ct]);
          r[ct] = mfma16(a_lo, b_hi, r[ct]);
          r[ct] = mfma16(a_hi, b_lo, r[ct]);
        }
      }
      // X_b = T_b R_b
      const float4 t4 = *reinterpret_cast<const float4*>(&sm.a[16 * b + m][16 * b + 4 * hq]);
      bf16x8 t_hi, t_lo;
      split_operand(floatx4{t4.x, t4.y, t4.z, t4.w}, zero, t_hi, t_lo);
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        bf16x8 r_hi, r_lo;
        split_operand(r[ct], zero, r_hi, r_lo);
        floatx4 acc = mfma16(t_hi, r_hi, zero);
        acc = mfma16(t_lo, r_hi, acc);
        x[b][ct] = mfma16(t_hi, r_lo, acc);
      }
      if (b == 1) {
#pragma unroll
        for (int ct = 0; ct < 4; ++ct) split_operand(x[0][ct], x[1][ct], pair_hi[ct], pair_lo[ct]);
      }
    }
  }
  char* out = a.workspace + (static_cast<size_t>(bh) * chunks + chunk) * kGdnChunkBytes;
  float* u_out = reinterpret_cast<float*>(out + kGdnOffsetU);
  __syncthreads();  // everyone is done reading V before -W overwrites it
  if (is_u) {
    // U in accumulator order: [block b][slice][lane = 16*hq + m][r], which is
    // how the tiles sit in registers
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int ct = 0; ct < 4; ++ct) {
        const int slice = col0 / 16 + ct;
        *reinterpret_cast<floatx4*>(u_out + ((b * SLICES + slice) * 64 + lane) * 4) = x[b][ct];
      }
  } else {
    const int hq = lane / 16, m = lane % 16;
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int ct = 0; ct < 4; ++ct)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          sm.vw[16 * b + 4 * hq + e][col0 + 16 * ct + m] = float_to_bf16_bits(-x[b][ct][e]);
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

// LDS stage of the sequential kernel: the chunk's -W | cQ | A2 | Kt fragments
// exactly as they sit in the scratch (56 KiB, contiguous there too) followed
// by the 4 KiB slice of U of each computing wave and the chunk's tail.
constexpr int kScanOperandBytes = static_cast<int>(kGdnOffsetDecay - kGdnOffsetW);  // 57344
// Column slices (computing waves) per workgroup: they would share the operand
// fragments of a stage, each with its own 4 KiB slice of U in it.
constexpr int kScanGroup = 1;
constexpr int kScanStageBytes = kScanOperandBytes + (4 * kScanGroup + 1) * 1024;
constexpr int kScanStages = 2;

typedef __attribute__((address_space(3))) unsigned char lds_byte;
typedef __attribute__((address_space(3))) const uint32x4 lds_u32x4;
typedef __attribute__((address_space(3))) const floatx4 lds_f32x4;
__device__ inline bf16x8 words_to_bf16x8(uint32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// One direct-to-LDS load of 16 bytes per lane: lane l fetches
// descriptor base + voffset(l) + soffset and the hardware writes it at LDS
// byte lds_address + 16 l.  Issued as inline assembly on purpose: the compiler
// does not see an LDS write, so it does not make later reads of the OTHER
// stage wait for this load; the kernel orders the accesses itself with
// s_waitcnt vmcnt (see gdn_chunk_scan).
__device__ inline void lds_dma_16(uint32x4 descriptor, uint32_t lds_address, uint32_t voffset,
                                  uint32_t soffset) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %1, %2, %3 offen lds"
      :
      : "s"(lds_address), "v"(voffset), "s"(descriptor), "s"(soffset)
      : "memory", "m0");
}

// The direct-to-LDS loads of one chunk: 56 + 4 * kScanGroup + 1 loads of 1 KiB
// (operand fragments, this workgroup's slices of U, the chunk's tail with its
// decay).
// Loader wave LOADER of LOADERS issues every LOADERS-th of them.
// `chunk_offset` is the byte offset of the chunk's scratch within the
// (sequence, head) region the descriptor covers.
constexpr int kScanFillLoads = kScanOperandBytes / 1024 + 4 * kScanGroup + 1;
template <int LOADER, int LOADERS>
__device__ __forceinline__ void scan_fill(uint32_t stage_address, uint32x4 descriptor,
                                          uint32_t chunk_offset, int slice, int lane) {
  const uint32_t lane_bytes = static_cast<uint32_t>(lane) * 16u;
  // fully unrolled: a lone wave issues a loop's scalar bookkeeping far slower
  // than the memory pipeline takes loads
#pragma unroll
  for (int f = LOADER; f < kScanFillLoads; f += LOADERS) {
    if (f < kScanOperandBytes / 1024) {
      lds_dma_16(descriptor, stage_address + f * 1024, lane_bytes,
                 chunk_offset + static_cast<uint32_t>(kGdnOffsetW) + f * 1024);
    } else if (f < kScanFillLoads - 1) {
      // `slice` is the first of the workgroup's kScanGroup slices
      const int j = f - kScanOperandBytes / 1024;
      lds_dma_16(descriptor, stage_address + f * 1024, lane_bytes,
                 chunk_offset + static_cast<uint32_t>(kGdnOffsetU) +
                     ((j % 4) * SLICES + slice + j / 4) * 1024);
    } else {
      // the tail is shorter than 1 KiB: its offset goes through the
      // bounds-checked lane offset so that lanes past the end of the scratch
      // read zeros
      lds_dma_16(descriptor, stage_address + f * 1024,
                 lane_bytes + chunk_offset + static_cast<uint32_t>(kGdnOffsetDecay), 0);
    }
  }
}

// Loader waves per workgroup, and what each needs at run time: the fill for its
// index, and a wait that lets exactly its share of one (the younger) fill stay
// in flight.
constexpr int kScanLoaders = 3;
static_assert(kScanLoaders == 2 || kScanLoaders == 3, "scan_fill_as and scan_wait_older_fill list the loaders");
constexpr int scan_fill_share(int loader) {
  return (kScanFillLoads - loader + kScanLoaders - 1) / kScanLoaders;
}
// (a wave whose two fills exceed the 63 operations its vector-memory counter
// holds merely stalls at the issue of the last few loads)
static_assert(scan_fill_share(0) <= 63, "the wait for the older fill must be encodable");
__device__ __forceinline__ void scan_fill_as(int loader, uint32_t stage_address, uint32x4 descriptor,
                                             uint32_t chunk_offset, int slice, int lane) {
  if (loader == 0) scan_fill<0, kScanLoaders>(stage_address, descriptor, chunk_offset, slice, lane);
  else if (loader == 1 || kScanLoaders == 2)
    scan_fill<1, kScanLoaders>(stage_address, descriptor, chunk_offset, slice, lane);
  else scan_fill<kScanLoaders - 1, kScanLoaders>(stage_address, descriptor, chunk_offset, slice, lane);
}
__device__ __forceinline__ void scan_wait_older_fill(int loader) {
  if (loader == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(scan_fill_share(0)) : "memory");
  else if (loader == 1 || kScanLoaders == 2)
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(scan_fill_share(1)) : "memory");
  else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(scan_fill_share(kScanLoaders - 1)) : "memory");
}

// Pulls this workgroup's eighth of a future chunk's scratch through L2 so that
// it is there by the time the workgroups of the (sequence, head) fetch it for
// real: the loader waves cannot keep enough real loads in flight to cover the
// latency of HBM.  These are full-width loads (1 KiB per instruction): what
// bounds a compute unit is the number of requests it has in flight, and a
// narrow load per cache sector is one request per lane.  They go straight to
// an LDS dump area nobody reads, so they need no registers and the issuing
// wave never waits for them.
constexpr int kScanTouchBytes = (static_cast<int>(kGdnChunkBytes) / SLICES + 1023) / 1024 * 1024;
constexpr int kScanTouchLoads = kScanTouchBytes / 1024;
constexpr int kScanAhead = 4;
__device__ inline void scan_touch(uint32x4 descriptor, uint32_t dump_address, uint32_t chunk_offset,
                                  int slice, int lane) {
  // the lane offset is the bounds-checked one: past the end of the scratch
  // the loads return zeros
  const uint32_t voffset = chunk_offset + static_cast<uint32_t>(slice) * (kGdnChunkBytes / SLICES) +
                           static_cast<uint32_t>(lane) * 16u;
#pragma unroll
  for (int i = 0; i < kScanTouchLoads; ++i) lds_dma_16(descriptor, dump_address, voffset, i * 1024);
}

// One workgroup per (sequence, head, kScanGroup slices of 16 state columns),
// one wave per SIMD so that a computing wave may use the whole register file:
// kScanGroup computing waves, one per slice, and kScanLoaders loader waves.
// A stage holds one chunk.  The computing wave moves the chunk's fragments into
// registers as its matrix instructions need them and releases the stage before
// the chunk's second phase; the loaders then stream chunk c+2 into it
// (asynchronous direct-to-LDS loads), so each loader has two fills in flight.
// Two workgroup barriers per chunk hand the stages over: "landed" and "free".
// A wave that issues long runs of loads stalls at issue while the memory
// pipeline digests them, which is why the computing wave issues only the few
// loads that warm L2.
//
// Measured on MI355X at 2 x 16 heads x 16384 tokens (256 chunks, one workgroup
// per compute unit), per chunk: the matrix instructions and the 60 KiB of LDS
// reads take about 0.85 us when nothing else runs, the fill of a stage 0.65 us
// when its data is in L2 and about 1 us when it comes from HBM; the two
// overlap only in part (1.3 us).  Two slices per workgroup halve the traffic
// from L2 but double the LDS reads of a compute unit, and measure slower.
constexpr int kScanThreads = 64 * (kScanGroup + kScanLoaders);
static_assert(kScanThreads <= 256, "one wave per SIMD");

// The workgroup barriers that hand an LDS stage over.  A loader arrives at the
// "landed" barrier once the stage's direct-to-LDS loads are complete (the
// caller waits for them); a computing wave arrives at the "free" barrier once
// its LDS reads are done, without waiting for its own vector-memory operations
// (output stores, L2 touches), which nobody in the workgroup depends on.
__device__ __forceinline__ void scan_barrier() { asm volatile("s_barrier" ::: "memory"); }
__device__ __forceinline__ void scan_handover_compute() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// One chunk of the sequential chain, computed from the operands in `stage`.
struct ScanContext {
  uint16_t* out;
  int length, value_heads;
  const char* base;
  int chunks, slice, lane, hq, m, seq, head;
};

__device__ __forceinline__ void scan_step(const ScanContext ctx, const uint32x4 descriptor,
                                          int chunk, const lds_byte* stage, floatx4 (&s)[8]) {
  struct {
    uint16_t* out;
    int length, value_heads;
  } a = {ctx.out, ctx.length, ctx.value_heads};
  const int slice = ctx.slice, lane = ctx.lane, hq = ctx.hq, m = ctx.m;
  const int seq = ctx.seq, head = ctx.head;
  const float decay = *(const __attribute__((address_space(3))) float*)(stage + kScanStageBytes - 1024);
  lds_u32x4* neg_w = (lds_u32x4*)(stage) + lane;
  lds_u32x4* q_in = (lds_u32x4*)(stage + (kGdnOffsetQ - kGdnOffsetW)) + lane;
  lds_u32x4* a2_in = (lds_u32x4*)(stage + (kGdnOffsetA2 - kGdnOffsetW)) + lane;
  lds_u32x4* kt_in = (lds_u32x4*)(stage + (kGdnOffsetKt - kGdnOffsetW)) + lane;
  lds_f32x4* u_in = (lds_f32x4*)(stage + kScanOperandBytes + 4096 * (slice % kScanGroup)) + lane;

  // LDS reads are issued well ahead of the matrix instructions that consume
  // them: the first-phase fragments (-W, cQ, U) one token tile ahead, the
  // second-phase fragments (Kt, A2) a quarter per token tile behind those.
  // Once the last of them is in registers, before the last token tile's
  // products, the stage goes back to the loaders.
  uint32x4 a2_reg[8], kt_reg[16];
  uint32x4 w_reg[2][4], q_reg[2][4];
  floatx4 u_reg[2];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    w_reg[0][kb] = neg_w[kb * 64];
    q_reg[0][kb] = q_in[kb * 64];
  }
  u_reg[0] = u_in[0];
  __builtin_amdgcn_sched_barrier(0);
  bf16x8 sb[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) sb[kb] = tiles_to_operand(s[2 * kb], s[2 * kb + 1]);
  // D = U - W S0 and the S0 part of O = exp(c) Q S0 + (M o Q K^T) D
  floatx4 d[4], o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (i + 1 < 4) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) {
        w_reg[(i + 1) % 2][kb] = neg_w[(4 * (i + 1) + kb) * 64];
        q_reg[(i + 1) % 2][kb] = q_in[(4 * (i + 1) + kb) * 64];
      }
      u_reg[(i + 1) % 2] = u_in[(i + 1) * 64];
#pragma unroll
      for (int f = 0; f < 8; ++f) {
        if (i < 2) kt_reg[8 * i + f] = kt_in[(8 * i + f) * 64];
        else a2_reg[f] = a2_in[f * 64];
      }
    } else {
      scan_handover_compute();
    }
    __builtin_amdgcn_sched_barrier(0);
    floatx4 acc = u_reg[i % 2];
    floatx4 out_acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      acc = mfma16(words_to_bf16x8(w_reg[i % 2][kb]), sb[kb], acc);
      out_acc = mfma16(words_to_bf16x8(q_reg[i % 2][kb]), sb[kb], out_acc);
    }
    d[i] = acc;
    o[i] = out_acc;
    __builtin_amdgcn_sched_barrier(0);
  }
  bf16x8 db[2];
  db[0] = tiles_to_operand(d[0], d[1]);
  db[1] = tiles_to_operand(d[2], d[3]);
  // S = exp(c_C) S0 + (diag(exp(c_C - c)) K)^T D, the chain the next chunk
  // waits for, goes first and the outputs follow; in both, products that depend
  // on each other are issued eight (four) instructions apart.
#pragma unroll
  for (int t = 0; t < 8; ++t) s[t] = s[t] * decay;
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
    for (int t = 0; t < 8; ++t) s[t] = mfma16(words_to_bf16x8(kt_reg[2 * t + kb]), db[kb], s[t]);
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = mfma16(words_to_bf16x8(a2_reg[2 * i + kb]), db[kb], o[i]);
    __builtin_amdgcn_sched_barrier(0);
  }
  // outputs: rows 16i + 4hq + r of the chunk, column 16*slice + m
  uint16_t* out_row = a.out +
      ((static_cast<long long>(seq) * a.length + chunk * C + 4 * hq) * a.value_heads + head) * DV +
      16 * slice + m;
  const long long row_step = static_cast<long long>(a.value_heads) * DV;
  if (chunk * C + C <= a.length) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) out_row[(16 * i + r) * row_step] = float_to_bf16_bits(o[i][r]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (chunk * C + 16 * i + 4 * hq + r < a.length)
          out_row[(16 * i + r) * row_step] = float_to_bf16_bits(o[i][r]);
  }
}

__global__ void __launch_bounds__(kScanThreads)
gdn_chunk_scan(GdnArgs a) {
  __shared__ __attribute__((aligned(1024))) unsigned char stage0[kScanStageBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char stage1[kScanStageBytes];
  __shared__ __attribute__((aligned(256))) unsigned char dump[1024];
  const int lane = threadIdx.x % 64, hq = lane / 16, m = lane % 16;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int chunks = (a.length + C - 1) / C;
  // The workgroups of one (sequence, head) read the same operands: keep them
  // on one XCD so that its L2 serves all but the first read.
  int logical = blockIdx.x;
  if (gridDim.x % 8 == 0) logical = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
  constexpr int kGroups = SLICES / kScanGroup;
  const int first_slice = (logical % kGroups) * kScanGroup;
  const int slice = first_slice + min(wave, kScanGroup - 1);
  const int bh = logical / kGroups;
  const int head = bh % a.value_heads, seq = bh / a.value_heads;
  float* state = a.state + static_cast<size_t>(bh) * DK * DV;
  const char* base = a.workspace + static_cast<size_t>(bh) * chunks * kGdnChunkBytes;
  // raw buffer descriptor: base address, no stride, size in bytes, data format
  const uint64_t address = reinterpret_cast<uint64_t>(base);
  const uint32x4 descriptor = {static_cast<uint32_t>(address),
                               static_cast<uint32_t>(address >> 32) & 0xffffu,
                               static_cast<uint32_t>(chunks * kGdnChunkBytes), 0x00020000u};
  const uint32_t stage0_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte*)stage0));
  const uint32_t stage1_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte*)stage1));

  // Every wave passes two barriers per chunk: "landed" (the chunk's stage is
  // complete) and "free" (the computing waves have copied it to registers).
  const uint32_t dump_address =
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte*)dump));
  if (wave >= kScanGroup) {
    const int loader = wave - kScanGroup;
    scan_fill_as(loader, stage0_address, descriptor, 0, first_slice, lane);
    if (chunks > 1)
      scan_fill_as(loader, stage1_address, descriptor, static_cast<uint32_t>(kGdnChunkBytes),
                   first_slice, lane);
    for (int chunk = 0; chunk < chunks; ++chunk) {
      // loads complete in issue order: all but the younger fill have landed
      if (chunk + 1 < chunks) scan_wait_older_fill(loader);
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      scan_barrier();  // landed
      scan_barrier();  // free
      if (chunk + 2 < chunks)
        scan_fill_as(loader, (chunk & 1) ? stage1_address : stage0_address, descriptor,
                     static_cast<uint32_t>(chunk + 2) * static_cast<uint32_t>(kGdnChunkBytes),
                     first_slice, lane);
    }
    return;
  }

  ScanContext ctx;
  ctx.out = a.out;
  ctx.length = a.length;
  ctx.value_heads = a.value_heads;
  ctx.base = base;
  ctx.chunks = chunks;
  ctx.slice = slice;
  ctx.lane = lane;
  ctx.hq = hq;
  ctx.m = m;
  ctx.seq = seq;
  ctx.head = head;
  floatx4 s[8];  // rows 16t + 4hq + r, column 16*slice + m
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      s[t][r] = state[(16 * t + 4 * hq + r) * DV + 16 * slice + m];
  for (int chunk = 2; chunk < min(kScanAhead + 2, chunks); ++chunk)
    scan_touch(descriptor, dump_address, static_cast<uint32_t>(chunk) * kGdnChunkBytes, slice, lane);
  for (int chunk = 0; chunk < chunks; ++chunk) {
    if (chunk + 2 + kScanAhead < chunks)
      scan_touch(descriptor, dump_address,
                 static_cast<uint32_t>(chunk + 2 + kScanAhead) * static_cast<uint32_t>(kGdnChunkBytes),
                 slice, lane);
    scan_barrier();  // landed
    // passes the "free" barrier once all of the chunk it still needs is in registers
    scan_step(ctx, descriptor, chunk, (chunk & 1) ? (lds_byte*)stage1 : (lds_byte*)stage0, s);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
  if (kernel_enabled(kAuxiliaryKernel))
    gdn_chunk_prepare<<<static_cast<unsigned>(heads * chunks), 256, 0, stream>>>(a);
  int status = launch_status();
  if (status != 0) return status;
  if (!kernel_enabled(kMainKernel)) return 0;
  gdn_chunk_scan<<<static_cast<unsigned>(heads * (SLICES / kScanGroup)), kScanThreads, 0, stream>>>(a);
  return launch_status();
}

int launch_gdn_recurrence(hipStream_t stream, const GdnArgs& a, int out_dtype) {
  if (a.key_dim > 128 || a.value_dim > 256) return PLUTO_HIP_EUNSUPPORTED;
  gdn_recurrence_kernel<<<a.batch * a.value_heads, 256, 0, stream>>>(a, out_dtype);
  return launch_status();
}

}  // namespace pluto_hip
