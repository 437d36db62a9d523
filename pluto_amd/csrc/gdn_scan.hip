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
// S0 = state entering the chunk, K and Q with their normalisation and scale):
//     A[i,j]  = b_i exp(c_i - c_j) (k_i . k_j)        for j <  i
//     T  = (I + A)^-1
//     D  = T diag(b) (V - diag(exp(c)) K S0)          (the d_t of the chunk)
//     O  = diag(exp(c)) Q S0 + (M o Q K^T) D,   M[i,j] = exp(c_i - c_j), j <= i
//     S  = exp(c_C) S0 + (diag(exp(c_C - c)) K)^T D
// Only differences c_i - c_j <= 0 are exponentiated, so nothing overflows.
// Every diagonal factor is applied in FP32 to matrix-core results, so the
// products themselves take the raw bf16 rows of K and Q as they lie in memory.
//
// Kernel 1 (gdn_chunk_prepare, one workgroup per chunk, fully parallel): the
// two Gram matrices on the matrix cores from the raw bf16 inputs, T by a block
// forward substitution on the matrix cores, and 14 KiB per chunk written out:
// T and M o (Q K^T) as bf16 matrix-core operands, and the per-token factors.
// Kernel 2 (gdn_chunk_scan, one workgroup per (sequence, head, 16 state
// columns)): walks the chunks with v_mfma_f32_16x16x32_bf16, the state in FP32
// accumulator registers of one wave, a second wave computing the outputs, two
// more streaming each chunk's 14 KiB and its raw K, Q and V rows into LDS.
// State columns are independent, which is what gives the sequential part
// 8 x batch x heads way parallelism.
#include "gdn.h"

namespace pluto_hip {
namespace {

constexpr int C = 64;     // tokens per chunk
constexpr int DK = 128;   // key width of the chunked path
constexpr int DV = 128;   // value width of the chunked path
constexpr int SLICES = DV / 16;

typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(4))) short shortx4;

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

// 35 KiB, so that four workgroups share a compute unit's LDS (the kernel is a
// chain of short, barrier-separated phases and lives on occupancy): once the
// Gram matrices are done the rows of K make room for A, and A in turn for the
// finished inverse; the rows of Q make room for the second bf16 result.
struct ChunkSmem {
  union {
    uint16_t k[C][DK + 8];  // raw K rows (bf16)
    float a[C][C + 4];      // then: strictly lower triangular A (FP32) and the blocks of its solve
    uint16_t t[C][C + 8];   // last: (I + A)^-1, bf16
  };
  union {
    uint16_t q[C][DK + 8];  // raw Q rows
    uint16_t a2[C][C + 8];  // later: M o (Q K^T) with all factors, bf16
  };
  float cum[C];             // inclusive cumulative log decay
  float beta[C];
  float inv_k[C];           // 1/|k| (or 1)
  float q_factor[C];        // q_scale / |q| (or q_scale)
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

  // ---- stage K and Q rows (16-byte pieces), zero beyond the sequence --------
  for (int piece = tid; piece < C * (DK / 8); piece += 256) {
    const int row = piece / (DK / 8), c8 = piece % (DK / 8);
    uint4 kb = make_uint4(0, 0, 0, 0), qb = kb;
    if (row < valid) {
      const long long token = static_cast<long long>(seq) * a.length + t0 + row;
      kb = *reinterpret_cast<const uint4*>(a.k + token * a.k_token_stride + key_head * DK + 8 * c8);
      qb = *reinterpret_cast<const uint4*>(a.q + token * a.q_token_stride + key_head * DK + 8 * c8);
    }
    *reinterpret_cast<uint4*>(&sm.k[row][8 * c8]) = kb;
    *reinterpret_cast<uint4*>(&sm.q[row][8 * c8]) = qb;
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
      sm.inv_k[row] = a.normalize_qk ? rsqrtf(kk + 1e-6f) : 1.0f;
      sm.q_factor[row] = a.normalize_qk ? a.q_scale * rsqrtf(qq + 1e-6f) : a.q_scale;
    }
  }
  __syncthreads();

  // ---- Gram matrices on the matrix cores: wave (ti, tj) owns a 32x32 tile --
  {
    const int ti = wave / 2, tj = wave % 2;
    const int h = lane / 32, n = lane % 32;
    float a2v[16], av[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      a2v[i] = 0.0f;
      av[i] = 0.0f;
    }
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
        if (col < row) av[i] = sm.beta[row] * decay * sm.inv_k[row] * inv_kj * gk[i];
        if (col <= row) a2v[i] = decay * sm.q_factor[row] * inv_kj * gq[i];
      }
    }
    __syncthreads();  // nobody reads the rows of K and Q any more
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = 32 * ti + 8 * (i / 4) + 4 * h + (i % 4);
      sm.a[row][32 * tj + n] = av[i];  // the tile above the diagonal is zero
      sm.a2[row][32 * tj + n] = float_to_bf16_bits(a2v[i]);
    }
  }
  __syncthreads();

  // ---- T = (I + A)^-1 by blocks of 16 rows on the matrix cores.  With T_b the
  // inverse of diagonal block b of I + A, block row b of the solve X of
  // (I + A) X = R is  X_b = T_b (R_b - sum_{k<b} A_bk X_k).
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

  // Wave w solves columns 16 w .. 16 w + 15 of X for R = I: X_b = 0 above the
  // diagonal block, X_w = T_w, and the blocks below follow from the recurrence.
  // x[b] is the 16x16 tile of block row b in accumulator order: lane (hq, m)
  // holds rows 16 b + 4 hq + r of column 16 w + m.
  {
    const int hq = lane / 16, m = lane % 16;
    const floatx4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    floatx4 x[4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      x[b] = zero;
      if (b < wave) continue;  // uniform over the wave
      floatx4 r = zero;
      if (b == wave) {
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = (4 * hq + e == m) ? 1.0f : 0.0f;
      }
      // R_b -= [A_b,k0 | A_b,k1] [X_k0; X_k1]: contraction slot (hq, e) is row
      // 4 hq + e % 4 of block k0 (e < 4) or k1
#pragma unroll
      for (int k0 = 0; k0 < b; k0 += 2) {
        if (k0 + 1 < wave) continue;  // both blocks of X are zero
        const bool both = k0 + 1 < b;
        const float4 first = *reinterpret_cast<const float4*>(&sm.a[16 * b + m][16 * k0 + 4 * hq]);
        float4 second = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (both) second = *reinterpret_cast<const float4*>(&sm.a[16 * b + m][16 * k0 + 16 + 4 * hq]);
        bf16x8 a_hi, a_lo, b_hi, b_lo;
        split_operand(floatx4{-first.x, -first.y, -first.z, -first.w},
                      floatx4{-second.x, -second.y, -second.z, -second.w}, a_hi, a_lo);
        split_operand(x[k0], both ? x[k0 + 1] : zero, b_hi, b_lo);
        r = mfma16(a_hi, b_hi, r);
        r = mfma16(a_lo, b_hi, r);
        r = mfma16(a_hi, b_lo, r);
      }
      // X_b = T_b R_b
      const float4 t4 = *reinterpret_cast<const float4*>(&sm.a[16 * b + m][16 * b + 4 * hq]);
      bf16x8 t_hi, t_lo, r_hi, r_lo;
      split_operand(floatx4{t4.x, t4.y, t4.z, t4.w}, zero, t_hi, t_lo);
      split_operand(r, zero, r_hi, r_lo);
      floatx4 acc = mfma16(t_hi, r_hi, zero);
      acc = mfma16(t_lo, r_hi, acc);
      x[b] = mfma16(t_hi, r_lo, acc);
    }
    __syncthreads();  // every wave has read what it needs of A: T takes its place
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        sm.t[16 * b + 4 * hq + e][16 * wave + m] = float_to_bf16_bits(x[b][e]);
  }
  __syncthreads();

  // ---- what the sequential kernel reads of this chunk -------------------------
  char* out = a.workspace + (static_cast<size_t>(bh) * chunks + chunk) * kGdnChunkBytes;
  uint4* t_out = reinterpret_cast<uint4*>(out + kGdnOffsetT);
  uint4* a2_out = reinterpret_cast<uint4*>(out + kGdnOffsetA2);
  // T and M o (Q K^T) as matrix-core operands over tokens j: fragment
  // (tile, kb), lane (hq, m) = row 16 tile + m, slot (hq, e) = column
  // 32 kb + 16 (e / 4) + 4 hq + e % 4; the two fragments above the diagonal
  // are zero and are not stored
  for (int piece = tid; piece < 6 * 64; piece += 256) {
    const int f = piece / 64, l = piece % 64;
    const int tile = f < 2 ? f : 2 + (f - 2) / 2, kb = f < 2 ? 0 : (f - 2) % 2;
    const int hq = l / 16, m = l % 16;
    const int row = 16 * tile + m, lo = 32 * kb + 4 * hq;
    uint2 w0 = *reinterpret_cast<const uint2*>(&sm.t[row][lo]);
    uint2 w1 = *reinterpret_cast<const uint2*>(&sm.t[row][lo + 16]);
    t_out[piece] = make_uint4(w0.x, w0.y, w1.x, w1.y);
    w0 = *reinterpret_cast<const uint2*>(&sm.a2[row][lo]);
    w1 = *reinterpret_cast<const uint2*>(&sm.a2[row][lo + 16]);
    a2_out[piece] = make_uint4(w0.x, w0.y, w1.x, w1.y);
  }
  // per-token factors, and the decay of the whole chunk
  float* factors = reinterpret_cast<float*>(out + kGdnOffsetFactors);
  const float cum_last = sm.cum[C - 1];
  if (tid < C) {
    const float grown = __expf(sm.cum[tid]);
    factors[tid] = sm.beta[tid];
    factors[C + tid] = sm.beta[tid] * grown * sm.inv_k[tid];
    factors[2 * C + tid] = sm.q_factor[tid] * grown;
    factors[3 * C + tid] = __expf(cum_last - sm.cum[tid]) * sm.inv_k[tid];
  } else if (tid < 2 * C) {
    // the rest of the block is loaded with it: keep it defined
    factors[4 * C + tid - C] = tid == C ? __expf(cum_last) : 0.0f;
  }
}

// LDS stage of the sequential kernel for one chunk: the chunk's scratch as it
// sits in memory (T | A2 | factors, 14 KiB), the raw K and Q rows gathered
// into matrix-core operand order (16 KiB each), and the 16 value columns of the
// workgroup's slice (2 KiB).
constexpr int kStageScratch = 0;
constexpr int kStageK = static_cast<int>(kGdnChunkBytes);
constexpr int kStageQ = kStageK + 16384;
constexpr int kStageV = kStageQ + 16384;
constexpr int kScanStageBytes = kStageV + 2048;
constexpr int kScanStages = 2;

typedef __attribute__((address_space(3))) unsigned char lds_byte;
typedef __attribute__((address_space(3))) const uint32x4 lds_u32x4;
typedef __attribute__((address_space(3))) const floatx4 lds_f32x4;
__device__ inline bf16x8 words_to_bf16x8(uint32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// One direct-to-LDS load of 16 bytes per lane: lane l fetches
// descriptor base + voffset(l) + soffset and the hardware writes it at LDS
// byte lds_address + 16 l.  Only voffset is checked against the size in the
// descriptor (a lane beyond it reads zeros).  Issued as inline assembly on
// purpose: the compiler does not see an LDS write, so it does not make later
// reads of the OTHER stage wait for this load; the kernel orders the accesses
// itself with s_waitcnt vmcnt (see gdn_chunk_scan).
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

// LDS transpose read of four 16-bit elements per lane (ds_read_b64_tr_b16):
// within every group of 16 lanes, source lane 4 kk + b supplies the 8 bytes at
// its address, and lane 4 b + e receives element e of source lanes b, b + 4,
// b + 8, b + 12 (kk = 0..3, in that order).
__device__ inline uint2 lds_transposed(const lds_byte* address) {
  const shortx4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) shortx4*)(address));
  return __builtin_bit_cast(uint2, v);
}

// K and Q operands sit in the stage in fragments of 64 slots of 16 bytes,
// fragment 4 tile + kb: logical lane (hq, m) holds token 16 tile + m, channels
// 32 kb + 8 hq .. + 7.  A token's four pieces occupy four consecutive slots, so
// the four lanes that fill them fetch 64 contiguous bytes; the pieces are
// rotated by m / 4 within those slots, which spreads both the operand reads
// (16 tokens at a fixed piece) and the transpose reads of K (four tokens at
// each of the four pieces) over the LDS banks.
__device__ inline int operand_slot(int hq, int m) { return 4 * m + ((hq + m / 4) & 3); }

// Where the loaders fetch a chunk from: one buffer descriptor per source, and
// the lane's own byte offset into each.
struct ScanSources {
  uint32x4 scratch, k, q, v;
  uint32_t k_lane, q_lane, v_lane;
  uint32_t k_row_bytes, q_row_bytes, v_row_bytes;
};

// The direct-to-LDS loads of one chunk, 1 KiB each: 14 of scratch, 16 of K,
// 16 of Q, 2 of V.  Loader wave LOADER of LOADERS issues every LOADERS-th.
constexpr int kFillScratch = static_cast<int>(kGdnChunkBytes) / 1024;
constexpr int kScanFillLoads = kFillScratch + 16 + 16 + 2;
template <int LOADER, int LOADERS>
__device__ __forceinline__ void scan_fill(uint32_t stage_address, const ScanSources& src, int chunk,
                                          int lane) {
  const uint32_t lane_bytes = static_cast<uint32_t>(lane) * 16u;
  const uint32_t row0 = static_cast<uint32_t>(chunk) * C;
  // fully unrolled: a lone wave issues a loop's scalar bookkeeping far slower
  // than the memory pipeline takes loads
#pragma unroll
  for (int f = LOADER; f < kScanFillLoads; f += LOADERS) {
    if (f < kFillScratch) {
      lds_dma_16(src.scratch, stage_address + f * 1024, lane_bytes,
                 static_cast<uint32_t>(chunk) * static_cast<uint32_t>(kGdnChunkBytes) + f * 1024);
    } else if (f < kFillScratch + 32) {
      // rows past the end of the sequence lie beyond the descriptor's size and
      // read zeros: the whole offset goes through the checked lane offset
      const int g = (f - kFillScratch) % 16, tile = g / 4, kb = g % 4;
      if (f < kFillScratch + 16)
        lds_dma_16(src.k, stage_address + kStageK + g * 1024,
                   src.k_lane + (row0 + 16 * tile) * src.k_row_bytes + 64 * kb, 0);
      else
        lds_dma_16(src.q, stage_address + kStageQ + g * 1024,
                   src.q_lane + (row0 + 16 * tile) * src.q_row_bytes + 64 * kb, 0);
    } else {
      const int half = f - kFillScratch - 32;
      lds_dma_16(src.v, stage_address + kStageV + half * 1024,
                 src.v_lane + (row0 + 32 * half) * src.v_row_bytes, 0);
    }
  }
}

// Loader waves per workgroup, and what each needs at run time: the fill for its
// index, and a wait that lets exactly its share of one (the younger) fill stay
// in flight.
constexpr int kScanLoaders = 2;
static_assert(kScanLoaders == 2 || kScanLoaders == 3, "scan_fill_as and scan_wait_older_fill list the loaders");
constexpr int scan_fill_share(int loader) {
  return (kScanFillLoads - loader + kScanLoaders - 1) / kScanLoaders;
}
// (a wave whose two fills exceed the 63 operations its vector-memory counter
// holds merely stalls at the issue of the last few loads)
static_assert(scan_fill_share(0) <= 63, "the wait for the older fill must be encodable");
__device__ __forceinline__ void scan_fill_as(int loader, uint32_t stage_address,
                                             const ScanSources& src, int chunk, int lane) {
  if (loader == 0) scan_fill<0, kScanLoaders>(stage_address, src, chunk, lane);
  else if (loader == 1 || kScanLoaders == 2) scan_fill<1, kScanLoaders>(stage_address, src, chunk, lane);
  else scan_fill<kScanLoaders - 1, kScanLoaders>(stage_address, src, chunk, lane);
}
__device__ __forceinline__ void scan_wait_older_fill(int loader) {
  if (loader == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(scan_fill_share(0)) : "memory");
  else if (loader == 1 || kScanLoaders == 2)
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(scan_fill_share(1)) : "memory");
  else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(scan_fill_share(kScanLoaders - 1)) : "memory");
}

// Pulls this workgroup's eighth of a future chunk (its scratch, its K rows and
// its Q rows; the eight workgroups of a (sequence, head) share all three) and
// its own V columns through L2 so that it is there by the time the workgroups fetch it for real:
// the loader waves cannot keep enough real loads in flight to cover the latency
// of HBM.  These are full-width loads (1 KiB per instruction): what bounds a
// compute unit is the number of requests it has in flight, and a narrow load
// per cache sector is one request per lane.  They go straight to an LDS dump
// area nobody reads, so they need no registers and the issuing wave never waits
// for them.
constexpr int kScanAhead = 4;
__device__ inline void scan_touch(const ScanSources& src, uint32_t dump_address, int chunk,
                                  int slice, int lane) {
  const uint32_t lane_bytes = static_cast<uint32_t>(lane) * 16u;
  // scratch: 14 KiB / 8 = 1792 bytes, two loads (the second runs into the
  // next slice's share, or past the end of the scratch, where it reads zeros)
  const uint32_t scratch = static_cast<uint32_t>(chunk) * static_cast<uint32_t>(kGdnChunkBytes) +
                           static_cast<uint32_t>(slice) * (kGdnChunkBytes / SLICES) + lane_bytes;
#pragma unroll
  for (int i = 0; i < 2; ++i) lds_dma_16(src.scratch, dump_address, scratch + i * 1024, 0);
  // K and Q: eight token rows of 256 bytes each, four rows a load
  const uint32_t row = static_cast<uint32_t>(chunk) * C + 8 * slice + lane / 16;
  const uint32_t piece = (lane % 16) * 16u;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    lds_dma_16(src.k, dump_address, (row + 4 * i) * src.k_row_bytes + piece, 0);
    lds_dma_16(src.q, dump_address, (row + 4 * i) * src.q_row_bytes + piece, 0);
  }
  // V: the slice's 16 columns belong to this workgroup alone
#pragma unroll
  for (int half = 0; half < 2; ++half)
    lds_dma_16(src.v, dump_address,
               src.v_lane + (static_cast<uint32_t>(chunk) * C + 32 * half) * src.v_row_bytes, 0);
}

// One workgroup per (sequence, head, slice of 16 state columns), one wave per
// SIMD so that each may use the whole register file: the chain wave (the
// sequential dependence from state to state: P = K S0, D, the state update),
// the output wave (Q S0, the causal product with D, the stores, and the loads
// that warm L2), and kScanLoaders loader waves.  A stage holds one chunk.  The
// two computing waves move the chunk's operands into registers as their matrix
// instructions need them; once the last read is issued the stage goes back to
// the loaders, which stream chunk c+2 into it (asynchronous direct-to-LDS
// loads), so each loader has two fills in flight.  Two workgroup barriers per
// chunk order everything: "landed" (the stage is complete, and the chain wave
// has published the state entering the chunk as a bf16 operand) and "free" (both
// computing waves are done with the stage, and the chain wave has published D).
// A wave that issues long runs of loads stalls at issue while the memory
// pipeline digests them, which is why the chain wave issues none.
constexpr int kScanThreads = 64 * (2 + kScanLoaders);
static_assert(kScanThreads <= 256, "one wave per SIMD");

// The workgroup barriers that hand an LDS stage over.  A loader arrives at the
// "landed" barrier once the stage's direct-to-LDS loads are complete (the
// caller waits for them); the computing wave arrives at the "free" barrier once
// its LDS reads are done, without waiting for its own vector-memory operations
// (output stores, L2 touches), which nobody in the workgroup depends on.
__device__ __forceinline__ void scan_barrier() { asm volatile("s_barrier" ::: "memory"); }
__device__ __forceinline__ void scan_handover_compute() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

struct ScanContext {
  uint16_t* out;
  int length, value_heads;
  int slice, lane, hq, m, seq, head;
};

__device__ inline float bf16_half(uint32_t word, int upper) {
  return __builtin_bit_cast(float, upper ? (word & 0xffff0000u) : (word << 16));
}

// What the chain wave hands to the output wave through LDS, one 16-byte slot a
// lane: the state entering the chunk as four operands, D as two.
struct ScanExchange {
  uint32x4 state[4][64];
  uint32x4 d[2][64];
};
typedef __attribute__((address_space(3))) ScanExchange lds_exchange;

__device__ inline uint32x4 bf16x8_to_words(bf16x8 v) { return __builtin_bit_cast(uint32x4, v); }

// The chain wave's share of one chunk.  The state s[t] holds rows
// 16 t + 4 hq + r of the slice's column m, where row rho stands for key channel
// 32 (rho / 32) + 8 ((rho % 16) / 4) + 4 ((rho / 16) % 2) + rho % 4: with that
// order the raw rows of K and Q are matrix-core operands as they are (eight
// consecutive channels per lane).  `sb` is the state as operands, which the
// caller has already published; on return it is the next chunk's.
__device__ __forceinline__ void chain_step(const ScanContext ctx, const lds_byte* stage,
                                           lds_exchange* exchange, floatx4 (&s)[8],
                                           bf16x8 (&sb)[4]) {
  const int lane = ctx.lane, hq = ctx.hq, m = ctx.m;
  const int slot = operand_slot(hq, m);
  lds_u32x4* k_in = (lds_u32x4*)(stage + kStageK) + slot;
  lds_u32x4* t_in = (lds_u32x4*)(stage + kStageScratch + kGdnOffsetT) + lane;
  // factor n of rows 16 i + 4 hq .. + 3: four consecutive floats
  lds_f32x4* factor_in = (lds_f32x4*)(stage + kStageScratch + kGdnOffsetFactors) + hq;
  const float decay =
      *(const __attribute__((address_space(3))) float*)(stage + kStageScratch + kGdnOffsetFactors + 4 * C * 4);
  // as a source lane of the transpose reads: token row kk of a group of four,
  // 8-byte piece b of the row
  const int kk = m / 4, piece = m % 4;
  const floatx4 zero = {0.0f, 0.0f, 0.0f, 0.0f};

  // LDS reads are issued well ahead of the matrix instructions that consume
  // them (a read takes about as long as four matrix instructions): the K
  // fragments one token tile ahead, everything the later phases need during the
  // phase before.
  uint32x4 k_reg[2][4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) k_reg[0][kb] = k_in[kb * 64];
  uint2 v_reg[4];
  floatx4 f1[4], f2[4], f4[4];
  uint32x4 t_reg[6];  // (i, kb) = (0,0) (1,0) (2,0) (2,1) (3,0) (3,1): T is lower triangular
  floatx4 p[4];
  // P = K S0, token tile by token tile
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (i + 1 < 4) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) k_reg[(i + 1) % 2][kb] = k_in[(4 * (i + 1) + kb) * 64];
    }
    if (i == 0) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v_reg[j] = lds_transposed(stage + kStageV + (16 * j + 4 * hq + kk) * 32 + 8 * piece);
        f1[j] = factor_in[4 * j];
      }
    } else if (i == 1) {
#pragma unroll
      for (int j = 0; j < 4; ++j) f2[j] = factor_in[16 + 4 * j];
      t_reg[0] = t_in[0 * 64];
      t_reg[1] = t_in[1 * 64];
      t_reg[2] = t_in[2 * 64];
    } else if (i == 2) {
      t_reg[3] = t_in[3 * 64];
      t_reg[4] = t_in[4 * 64];
      t_reg[5] = t_in[5 * 64];
#pragma unroll
      for (int j = 0; j < 4; ++j) f4[j] = factor_in[48 + 4 * j];
    }
    __builtin_amdgcn_sched_barrier(0);
    floatx4 acc = zero;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) acc = mfma16(words_to_bf16x8(k_reg[i % 2][kb]), sb[kb], acc);
    p[i] = acc;
    __builtin_amdgcn_sched_barrier(0);
  }
  // S = exp(c_C) S0 + K^T (diag(exp(c_C - c) / |k|) D): row tile t = 2 kb + j
  // of the state is channels 32 kb + 8 b + 4 j + e for operand row 4 b + e,
  // read from the K fragments through the transposing LDS path; tokens
  // 32 tb + 16 jt + 4 hq + kk, jt = 0, 1
  uint2 kt_reg[2][8][2];
  auto read_kt = [&](int tb) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int kb = t / 2, j = t % 2;
      const lds_byte* base = stage + kStageK + 8 * j;
#pragma unroll
      for (int jt = 0; jt < 2; ++jt)
        kt_reg[tb][t][jt] = lds_transposed(
            base + (((2 * tb + jt) * 4 + kb) * 64 + operand_slot(piece, 4 * hq + kk)) * 16);
    }
  };
  read_kt(0);
  __builtin_amdgcn_sched_barrier(0);
  // R = diag(beta) V - diag(beta exp(c) / |k|) P, then D = T R
  floatx4 rt[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint2 v = v_reg[i];
    rt[i][0] = f1[i][0] * bf16_half(v.x, 0) - f2[i][0] * p[i][0];
    rt[i][1] = f1[i][1] * bf16_half(v.x, 1) - f2[i][1] * p[i][1];
    rt[i][2] = f1[i][2] * bf16_half(v.y, 0) - f2[i][2] * p[i][2];
    rt[i][3] = f1[i][3] * bf16_half(v.y, 1) - f2[i][3] * p[i][3];
  }
  bf16x8 r_op[2];
  r_op[0] = tiles_to_operand(rt[0], rt[1]);
  r_op[1] = tiles_to_operand(rt[2], rt[3]);
  __builtin_amdgcn_sched_barrier(0);
  read_kt(1);
  __builtin_amdgcn_sched_barrier(0);
  floatx4 d[4];
  {
    constexpr int first[4] = {0, 1, 2, 4};  // index of (i, 0) in t_reg
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      floatx4 acc = zero;
#pragma unroll
      for (int kb = 0; kb < (i < 2 ? 1 : 2); ++kb)
        acc = mfma16(words_to_bf16x8(t_reg[first[i] + kb]), r_op[kb], acc);
      d[i] = acc;
    }
  }
  // the two roles of D: as it is for the outputs (published for the output
  // wave), scaled by exp(c_C - c) / |k| for the state
  bf16x8 ds[2];
  {
    floatx4 scaled[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) scaled[i] = d[i] * f4[i];
    exchange->d[0][lane] = bf16x8_to_words(tiles_to_operand(d[0], d[1]));
    exchange->d[1][lane] = bf16x8_to_words(tiles_to_operand(d[2], d[3]));
    ds[0] = tiles_to_operand(scaled[0], scaled[1]);
    ds[1] = tiles_to_operand(scaled[2], scaled[3]);
  }
  // every read of the stage has been issued, D is on its way to LDS
  scan_handover_compute();
#pragma unroll
  for (int t = 0; t < 8; ++t) s[t] = s[t] * decay;
#pragma unroll
  for (int tb = 0; tb < 2; ++tb) {
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const uint32x4 words = {kt_reg[tb][t][0].x, kt_reg[tb][t][0].y, kt_reg[tb][t][1].x,
                              kt_reg[tb][t][1].y};
      s[t] = mfma16(words_to_bf16x8(words), ds[tb], s[t]);
    }
  }
  // the next chunk's operands, published before its "landed" barrier
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    sb[kb] = tiles_to_operand(s[2 * kb], s[2 * kb + 1]);
    exchange->state[kb][lane] = bf16x8_to_words(sb[kb]);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}

// The output wave's share of one chunk:
// O = diag(q_scale exp(c) / |q|) Q S0 + (M o Q K^T) D.
__device__ __forceinline__ void output_step(const ScanContext ctx, int chunk, const lds_byte* stage,
                                            const lds_exchange* exchange) {
  const int slice = ctx.slice, lane = ctx.lane, hq = ctx.hq, m = ctx.m;
  lds_u32x4* q_in = (lds_u32x4*)(stage + kStageQ) + operand_slot(hq, m);
  lds_u32x4* a2_in = (lds_u32x4*)(stage + kStageScratch + kGdnOffsetA2) + lane;
  lds_f32x4* factor_in = (lds_f32x4*)(stage + kStageScratch + kGdnOffsetFactors) + hq;
  const floatx4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
  bf16x8 sb[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) sb[kb] = words_to_bf16x8(exchange->state[kb][lane]);
  uint32x4 q_reg[2][4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) q_reg[0][kb] = q_in[kb * 64];
  uint32x4 a2_reg[6];  // (i, kb) = (0,0) (1,0) (2,0) (2,1) (3,0) (3,1): causal
  floatx4 f3[4];
  floatx4 o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (i + 1 < 4) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb) q_reg[(i + 1) % 2][kb] = q_in[(4 * (i + 1) + kb) * 64];
    }
    if (i == 1) {
      a2_reg[0] = a2_in[0 * 64];
      a2_reg[1] = a2_in[1 * 64];
      a2_reg[2] = a2_in[2 * 64];
    } else if (i == 2) {
      a2_reg[3] = a2_in[3 * 64];
      a2_reg[4] = a2_in[4 * 64];
      a2_reg[5] = a2_in[5 * 64];
#pragma unroll
      for (int j = 0; j < 4; ++j) f3[j] = factor_in[32 + 4 * j];
    }
    __builtin_amdgcn_sched_barrier(0);
    floatx4 acc = zero;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) acc = mfma16(words_to_bf16x8(q_reg[i % 2][kb]), sb[kb], acc);
    o[i] = acc;
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = o[i] * f3[i];
  // done with the stage; D follows the barrier
  scan_handover_compute();
  bf16x8 db[2];
  db[0] = words_to_bf16x8(exchange->d[0][lane]);
  db[1] = words_to_bf16x8(exchange->d[1][lane]);
  {
    constexpr int first[4] = {0, 1, 2, 4};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int kb = 0; kb < (i < 2 ? 1 : 2); ++kb)
        o[i] = mfma16(words_to_bf16x8(a2_reg[first[i] + kb]), db[kb], o[i]);
    }
  }
  // outputs: rows 16i + 4hq + r of the chunk, column 16*slice + m
  uint16_t* out_row = ctx.out +
      ((static_cast<long long>(ctx.seq) * ctx.length + chunk * C + 4 * hq) * ctx.value_heads + ctx.head) * DV +
      16 * slice + m;
  const long long row_step = static_cast<long long>(ctx.value_heads) * DV;
  if (chunk * C + C <= ctx.length) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) out_row[(16 * i + r) * row_step] = float_to_bf16_bits(o[i][r]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (chunk * C + 16 * i + 4 * hq + r < ctx.length)
          out_row[(16 * i + r) * row_step] = float_to_bf16_bits(o[i][r]);
  }
}

__device__ inline uint32x4 raw_descriptor(const void* base, uint32_t bytes) {
  const uint64_t address = reinterpret_cast<uint64_t>(base);
  // base address, no stride, size in bytes, data format
  return uint32x4{static_cast<uint32_t>(address), static_cast<uint32_t>(address >> 32) & 0xffffu,
                  bytes, 0x00020000u};
}

__global__ void __launch_bounds__(kScanThreads)
gdn_chunk_scan(GdnArgs a) {
  __shared__ __attribute__((aligned(1024))) unsigned char stages[kScanStages * kScanStageBytes];
  __shared__ __attribute__((aligned(256))) unsigned char dump[1024];
  __shared__ __attribute__((aligned(16))) ScanExchange exchange;
  const int lane = threadIdx.x % 64, hq = lane / 16, m = lane % 16;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
  const int chunks = (a.length + C - 1) / C;
  // The workgroups of one (sequence, head) read the same operands: keep them
  // on one XCD so that its L2 serves all but the first read.
  int logical = blockIdx.x;
  if (gridDim.x % 8 == 0) logical = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
  const int slice = logical % SLICES;
  const int bh = logical / SLICES;
  const int head = bh % a.value_heads, seq = bh / a.value_heads;
  const int key_head = head / (a.value_heads / a.key_heads);
  float* state = a.state + static_cast<size_t>(bh) * DK * DV;

  ScanSources src;
  src.scratch = raw_descriptor(a.workspace + static_cast<size_t>(bh) * chunks * kGdnChunkBytes,
                               static_cast<uint32_t>(chunks * kGdnChunkBytes));
  const long long first_token = static_cast<long long>(seq) * a.length;
  src.k_row_bytes = static_cast<uint32_t>(a.k_token_stride * 2);
  src.q_row_bytes = static_cast<uint32_t>(a.q_token_stride * 2);
  src.v_row_bytes = static_cast<uint32_t>(a.v_token_stride * 2);
  src.k = raw_descriptor(a.k + first_token * a.k_token_stride + key_head * DK,
                         static_cast<uint32_t>(a.length - 1) * src.k_row_bytes + DK * 2);
  src.q = raw_descriptor(a.q + first_token * a.q_token_stride + key_head * DK,
                         static_cast<uint32_t>(a.length - 1) * src.q_row_bytes + DK * 2);
  src.v = raw_descriptor(a.v + first_token * a.v_token_stride + head * DV + 16 * slice,
                         static_cast<uint32_t>(a.length - 1) * src.v_row_bytes + 16 * 2);
  {
    // LDS slot `lane` of a K or Q fragment belongs to the logical lane whose
    // operand_slot it is: token lane / 4 of the tile, piece (lane % 4 - token / 4) mod 4
    const uint32_t token = static_cast<uint32_t>(lane / 4);
    const uint32_t part = static_cast<uint32_t>((lane % 4 - lane / 16) & 3);
    src.k_lane = token * src.k_row_bytes + 16u * part;
    src.q_lane = token * src.q_row_bytes + 16u * part;
    // V: two slots a token (16 columns = 32 bytes)
    src.v_lane = static_cast<uint32_t>(lane / 2) * src.v_row_bytes + 16u * (lane % 2);
  }
  // chunk c lives in stage c % 2; every address within a stage is then the
  // stage's base plus a constant
  const uint32_t stage0_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte*)stages));
  const uint32_t stage1_address = stage0_address + kScanStageBytes;
  const uint32_t dump_address =
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_byte*)dump));

  // Every wave passes two barriers per chunk: "landed" and "free".
  if (wave >= 2) {
    const int loader = wave - 2;
    scan_fill_as(loader, stage0_address, src, 0, lane);
    if (chunks > 1) scan_fill_as(loader, stage1_address, src, 1, lane);
    for (int chunk = 0; chunk < chunks; ++chunk) {
      // loads complete in issue order: all but the younger fill have landed
      if (chunk + 1 < chunks) scan_wait_older_fill(loader);
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      scan_barrier();  // landed
      scan_barrier();  // free
      if (chunk + 2 < chunks)
        scan_fill_as(loader, (chunk & 1) ? stage1_address : stage0_address, src, chunk + 2, lane);
    }
    return;
  }

  ScanContext ctx;
  ctx.out = a.out;
  ctx.length = a.length;
  ctx.value_heads = a.value_heads;
  ctx.slice = slice;
  ctx.lane = lane;
  ctx.hq = hq;
  ctx.m = m;
  ctx.seq = seq;
  ctx.head = head;
  if (wave == 1) {
    for (int chunk = 2; chunk < min(kScanAhead + 2, chunks); ++chunk)
      scan_touch(src, dump_address, chunk, slice, lane);
    for (int chunk = 0; chunk < chunks; ++chunk) {
      if (chunk + 2 + kScanAhead < chunks)
        scan_touch(src, dump_address, chunk + 2 + kScanAhead, slice, lane);
      scan_barrier();  // landed
      // passes the "free" barrier once it has read all it needs of the stage,
      // and has read D by the time it returns
      output_step(ctx, chunk, (lds_byte*)stages + (chunk & 1) * kScanStageBytes,
                  (const lds_exchange*)&exchange);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    return;
  }

  // state rows in operand order (see chain_step)
  floatx4 s[8];
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      s[t][r] = state[(32 * (t / 2) + 8 * hq + 4 * (t % 2) + r) * DV + 16 * slice + m];
  bf16x8 sb[4];
#pragma unroll
  for (int kb = 0; kb < 4; ++kb) {
    sb[kb] = tiles_to_operand(s[2 * kb], s[2 * kb + 1]);
    exchange.state[kb][lane] = bf16x8_to_words(sb[kb]);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  for (int chunk = 0; chunk < chunks; ++chunk) {
    scan_barrier();  // landed
    // passes the "free" barrier once it has read all it needs of the stage
    chain_step(ctx, (lds_byte*)stages + (chunk & 1) * kScanStageBytes, (lds_exchange*)&exchange, s,
               sb);
  }
#pragma unroll
  for (int t = 0; t < 8; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      state[(32 * (t / 2) + 8 * hq + 4 * (t % 2) + r) * DV + 16 * slice + m] = s[t][r];
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
  // the sequential kernel addresses a sequence's rows through 32-bit offsets
  auto in_range = [&](long long token_stride) {
    return token_stride > 0 && token_stride * 2 * a.length < (1LL << 31);
  };
  if (!in_range(a.q_token_stride) || !in_range(a.k_token_stride) || !in_range(a.v_token_stride))
    return false;
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
  gdn_chunk_scan<<<static_cast<unsigned>(heads * SLICES), kScanThreads, 0, stream>>>(a);
  return launch_status();
}

int launch_gdn_recurrence(hipStream_t stream, const GdnArgs& a, int out_dtype) {
  if (a.key_dim > 128 || a.value_dim > 256) return PLUTO_HIP_EUNSUPPORTED;
  gdn_recurrence_kernel<<<a.batch * a.value_heads, 256, 0, stream>>>(a, out_dtype);
  return launch_status();
}

}  // namespace pluto_hip
