// Causal flash attention backward for bf16 activations on gfx950 matrix cores.
//
// Contract of AttentionLayer::bwd_impl (src/llm/layers/attention.cc:509-596):
// packed bf16 Q|K|V and stored bf16 output, FP32 upstream gradient, FP32 packed
// gradient out; query-owned dQ and key-owned dK/dV with a fixed reduction
// order and no atomics, hence bitwise repeatable.
//
// Two kernels:
//   dq    one workgroup per 128 queries, loops over 64-key tiles.  Its
//         prologue also does what the reference's delta pass does
//         (attention.cc:283-291): delta = sum(dO * O) per (row, head), plus the
//         row's log2-sum-exp and a bf16 copy of dO, all three left in the
//         workspace for the second kernel.
//   dkv   one workgroup per 128 keys, loops over query tiles in ascending
//         order.
// Streamed tiles are row major in LDS, filled by direct-to-LDS buffer loads;
// the same tile feeds the score product through 16-byte row reads and the
// gradient product through LDS transpose reads (mfma_tile.h).  All products
// use v_mfma_f32_32x32x16_bf16 in the orientation that keeps the score tile's
// accumulator directly usable as the B operand of the gradient product: dq
// works on S^T (lane = query), dkv on S (lane = key).  Deviation, within the
// stated bf16 tolerance: P, dS and dO are rounded to bf16 for the matrix
// products (the reference keeps them FP32).
#include "flash_bwd_mfma.h"

#include "mfma_tile.h"

namespace pluto_hip {
namespace {

constexpr int kThreads = 256;
// Schedules (see BackwardUnit).  The 64-wide dQ kernel keeps three
// workgroups per CU resident, which holds the whole paired grid of the
// training shape at once; the other three kernels hold two per CU and drain
// faster unpaired (1554 -> 1177 us for dK/dV and 754 -> 644 us for dQ at
// T = 8192, 24 heads of 128; 99 -> 94 us for dK/dV at T = 1024, 12 heads of
// 64, 16 sequences; the 64-wide dQ kernel is 8 % slower unpaired).
constexpr int kWideFromRows = 4096;
constexpr bool kDqPaired64 = true;
constexpr bool kOtherPaired = false;

// Which tile(s) a workgroup owns.  Paired: the workgroup takes tile `pair`
// and tile tiles-1-pair, which together carry the same work for every pair
// under the causal mask -- perfect balance when the whole grid is resident.
// Unpaired: one tile per workgroup, handed out from the heavy end of the
// sequence to the light one (`pair` counts from the light end for dQ, where
// the last query tile is the heaviest, and from the heavy end for dK/dV,
// where key tile 0 is), so that a grid larger than the resident set drains
// evenly.  A (sequence, head) unit keeps its XCD across tiles whenever the
// number of units is a multiple of 8.
struct BackwardUnit {
  int pair, head, seq;
};

template <bool PAIRED>
__device__ inline BackwardUnit backward_unit(int tiles, int heads) {
  BackwardUnit u;
  if constexpr (PAIRED) {
    const int pairs = (tiles + 1) / 2;
    const int logical = xcd_logical_block();
    u.pair = logical % pairs;
    u.head = (logical / pairs) % heads;
    u.seq = logical / (pairs * heads);
  } else {
    const int units = gridDim.x / tiles;
    u.pair = blockIdx.x / units;
    u.head = (blockIdx.x % units) % heads;
    u.seq = (blockIdx.x % units) / heads;
  }
  return u;
}

// dQ^T[d, query] = sum_keys K^T[d, key] dS^T[key, query]
template <int D, bool PAIRED>
__global__ void __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(D == 64 ? 3 : 2, D == 64 ? 3 : 2)))
flash_dq_kernel(GenericBackwardArgs a, float* __restrict__ lse2,
                uint16_t* __restrict__ d_out_bf16) {
  constexpr int BM = 128, BN = 64;
  constexpr int KCH = D / 8, KS = D / 16, DB = D / 32, KB = BN / 32;
  constexpr int LOADS = BN * KCH / kThreads;
  constexpr int kTileBytes = BN * D * 2, kStageBytes = 2 * kTileBytes;
  constexpr int kBlockBytes = 32 * D * 2;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];
  // 4 KiB a wave that no other wave touches (64-wide heads, where three
  // workgroups of 48 KiB still share a compute unit): rows on their way out are
  // reordered here without a barrier
  constexpr bool kOwnArea = D == 64;
  __shared__ __attribute__((aligned(16))) uint4 own_area[kOwnArea ? 4 * 256 : 1];

  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int T = a.context_length, H = a.num_heads, E = a.embedding_dim;
  const int q_tiles = (T + BM - 1) / BM;
  const BackwardUnit unit = backward_unit<PAIRED>(q_tiles, H);
  const int pair = unit.pair, head = unit.head, seq = unit.seq;
  const long long seq_row0 = static_cast<long long>(seq) * T;
  const long long stats_base = (static_cast<long long>(seq) * H + head) * T;
  const uint16_t* qkv = static_cast<const uint16_t*>(a.qkv);
  const uint16_t* q_base = qkv + seq_row0 * 3 * E + head * D;
  const uint16_t* k_base = q_base + E;
  const uint16_t* v_base = q_base + 2 * E;
  const uint16_t* o_base = static_cast<const uint16_t*>(a.out) + seq_row0 * E + head * D;
  const float* g_base = a.d_out + seq_row0 * E + head * D;
  uint16_t* gb_base = d_out_bf16 + seq_row0 * E + head * D;
  const float scale2 = a.scale * kLog2e;

  // K and V rows share the packed row stride, hence one set of fill offsets.
  uint32_t fill[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i)
    fill[i] = tile_fill_offset<D>((wave * LOADS + i) * 64 + lane, 3LL * E);
  int row_read[KS], tr_read[DB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) row_read[ks] = tile_row_read<D>(n, 2 * ks + h);
#pragma unroll
  for (int db = 0; db < DB; ++db) tr_read[db] = tile_transpose_read<D>(lane, db);

  // Query tiles (q_tiles-1-pair) and (pair) together see the same number of
  // keys for every pair: equal work per workgroup under the causal mask.
  for (int pass = 0; pass < (PAIRED ? 2 : 1); ++pass) {
    const int q_tile = pass == 0 ? q_tiles - 1 - pair : pair;
    if (pass == 1 && q_tile == q_tiles - 1 - pair) break;
    const int q0 = q_tile * BM;
    const int last_row = min(q0 + BM, T) - 1;
    const int tiles = last_row / BN + 1;
    tile_fill<D, LOADS>(lds, wave, k_base, 3LL * E, 0, T, fill);
    tile_fill<D, LOADS>(lds + kTileBytes, wave, v_base, 3LL * E, 0, T, fill);

    const int wave_first_row = q0 + 32 * wave;
    const int q_row = wave_first_row + n;
    uint4* copy_area = kOwnArea ? own_area + wave * 256
                                : reinterpret_cast<uint4*>(lds + kStageBytes) + wave * 32 * KCH;
    // Rows beyond the sequence are clamped to its last row and never stored.
    const int q_load = min(q_row, T - 1);
    bf16x8 qf[KS], gf[KS];
    float partial = 0.0f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c = 16 * ks + 8 * h;
      qf[ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
          q_base + static_cast<long long>(q_load) * 3 * E + c));
      const float4 g0 = *reinterpret_cast<const float4*>(g_base + static_cast<long long>(q_load) * E + c);
      const float4 g1 = *reinterpret_cast<const float4*>(g_base + static_cast<long long>(q_load) * E + c + 4);
      const uint4 o = *reinterpret_cast<const uint4*>(o_base + static_cast<long long>(q_load) * E + c);
      const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
      const uint32_t ow[4] = {o.x, o.y, o.z, o.w};
      uint32_t packed[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        partial += g[2 * i] * __uint_as_float(ow[i] << 16);
        partial += g[2 * i + 1] * __uint_as_float(ow[i] & 0xffff0000u);
        packed[i] = pack_bf16(g[2 * i], g[2 * i + 1]);
      }
      const uint4 bits = make_uint4(packed[0], packed[1], packed[2], packed[3]);
      gf[ks] = as_bf16x8(bits);
      copy_area[n * KCH + ((2 * ks + h) ^ (n & 7))] = bits;
    }
    // The bf16 copy of dO leaves through LDS (the wave's slice of the stage
    // that no fill has been issued into yet): a lane holds 16-byte pieces of its
    // own row, and stored from there a store instruction touches 32 lines;
    // from LDS it writes whole rows (25 MB in 17 us against 5 us).
#pragma unroll
    for (int i = 0; i < 32 * KCH / 64; ++i) {
      const int at = i * 64 + lane, row = at / KCH, chunk = at % KCH;
      const uint4 bits = copy_area[row * KCH + (chunk ^ (row & 7))];
      if (wave_first_row + row < T)
        *reinterpret_cast<uint4*>(gb_base + static_cast<long long>(wave_first_row + row) * E +
                                  8 * chunk) = bits;
    }
    // delta of attention.cc:283-291 (uses the stored, rounded output)
    const float row_delta = half_swap_sum(partial);
    const float normalizer = a.normalizers[stats_base + q_load];
    const float row_lse2 = a.maxima[stats_base + q_load] * kLog2e +
                           __log2f(normalizer > 0.0f ? normalizer : 1.0f);
    if (h == 0 && q_row < T) {
      // the key-owned kernel starts its accumulators from these
      a.deltas[stats_base + q_row] = -row_delta;
      lse2[stats_base + q_row] = -row_lse2 / scale2;
    }
    floatx16 dq_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) dq_acc[db][i] = 0.0f;

    const int wave_last_key = wave_first_row + 31;

    for (int tile = 0; tile < tiles; ++tile) {
      const int k0 = tile * BN;
      // this tile has landed; every wave is done with the other stage
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tile + 1 < tiles) {
        unsigned char* stage = lds + ((tile + 1) & 1) * kStageBytes;
        tile_fill<D, LOADS>(stage, wave, k_base + static_cast<long long>(k0 + BN) * 3 * E,
                            3LL * E, k0 + BN, T, fill);
        tile_fill<D, LOADS>(stage + kTileBytes, wave,
                            v_base + static_cast<long long>(k0 + BN) * 3 * E, 3LL * E, k0 + BN, T,
                            fill);
      }
      const unsigned char* k_tile = lds + (tile & 1) * kStageBytes;
      const unsigned char* v_tile = k_tile + kTileBytes;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int kb0 = k0 + 32 * kb;
        if (kb0 > wave_last_key) continue;
        const unsigned char* k_block = k_tile + kb * kBlockBytes;
        const unsigned char* v_block = v_tile + kb * kBlockBytes;
        bf16x8 ktf[2][DB];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int db = 0; db < DB; ++db)
            ktf[s2][db] = tile_transposed_operand<D>(k_block, tr_read[db], s2);
        floatx16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          s[i] = 0.0f;
          dp[i] = 0.0f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 kf = as_bf16x8(*reinterpret_cast<const uint4*>(k_block + row_read[ks]));
          const bf16x8 vf = as_bf16x8(*reinterpret_cast<const uint4*>(v_block + row_read[ks]));
          s = mfma32(kf, qf[ks], s);
          dp = mfma32(vf, gf[ks], dp);
        }
        // dS^T = P^T o (dP^T - delta), without the 1/sqrt(d) factor (applied
        // once at the end)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], scale2, -row_lse2));
          s[i] = p * (dp[i] - row_delta);
        }
        if (kb0 + 31 > wave_first_row) {  // diagonal block: hide future keys
          const int limit = q_row - kb0 - 4 * h;
#pragma unroll
          for (int i = 0; i < 16; ++i) s[i] = (8 * (i / 4) + (i % 4) > limit) ? 0.0f : s[i];
        }
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const bf16x8 dsf = accumulator_to_operand(s, s2);
#pragma unroll
          for (int db = 0; db < DB; ++db) dq_acc[db] = mfma32(ktf[s2][db], dsf, dq_acc[db]);
        }
      }
    }
    if constexpr (kOwnArea) {
      // dQ leaves through the wave's own area, 32 columns at a time: a store
      // instruction then writes eight whole 128-byte half rows instead of
      // 32-byte pieces of 32 rows
      float4* area = reinterpret_cast<float4*>(own_area) + wave * 256;
      float* dst = a.d_qkv + (seq_row0 + wave_first_row) * 3 * E + head * D;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float4 value;
          value.x = dq_acc[db][4 * j + 0] * a.scale;
          value.y = dq_acc[db][4 * j + 1] * a.scale;
          value.z = dq_acc[db][4 * j + 2] * a.scale;
          value.w = dq_acc[db][4 * j + 3] * a.scale;
          area[n * 8 + ((2 * j + h) ^ (n & 7))] = value;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = 8 * i + lane / 8, piece = lane % 8;
          const float4 value = area[row * 8 + (piece ^ (row & 7))];
          if (wave_first_row + row < T)
            *reinterpret_cast<float4*>(dst + static_cast<long long>(row) * 3 * E + 32 * db +
                                       4 * piece) = value;
        }
      }
    } else if (q_row < T) {
      float* dst = a.d_qkv + (seq_row0 + q_row) * 3 * E + head * D;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float4 value;
          value.x = dq_acc[db][4 * j + 0] * a.scale;
          value.y = dq_acc[db][4 * j + 1] * a.scale;
          value.z = dq_acc[db][4 * j + 2] * a.scale;
          value.w = dq_acc[db][4 * j + 3] * a.scale;
          *reinterpret_cast<float4*>(dst + 32 * db + 8 * j + 4 * h) = value;
        }
    }
    __syncthreads();  // the next pass refills stage 0
  }
}

// Stage of the key-owned kernel: Q tile | dO tile | lse2[64] | -delta[64] for
// query rows q0.. .  Waves 0 and 1 also fetch the row statistics, one float
// per lane.
template <int D, int BQ, int LOADS>
__device__ inline void dkv_fill_stage(unsigned char* stage, int wave, int lane,
                                      const uint16_t* q_base, const uint16_t* g_base,
                                      const float* lse2_base, const float* delta_base, int E,
                                      int q0, int T, const uint32_t* q_fill,
                                      const uint32_t* g_fill) {
  constexpr int kTileBytes = BQ * D * 2;
  tile_fill<D, LOADS>(stage, wave, q_base + static_cast<long long>(q0) * 3 * E, 3LL * E, q0, T,
                      q_fill);
  tile_fill<D, LOADS>(stage + kTileBytes, wave, g_base + static_cast<long long>(q0) * E, 1LL * E,
                      q0, T, g_fill);
  if (wave < 2) {
    const float* source = wave == 0 ? lse2_base : delta_base;
    const int left = T - q0;
    const int32x4 rsrc =
        make_rsrc(source + q0, left <= 0 ? 0u : static_cast<uint32_t>(left) * 4u);
    lds_fill<4>(rsrc, stage + 2 * kTileBytes + wave * 256, lane * 4);
  }
}

// dK^T[d, key] = sum_q Q^T[d, q] dS[q, key];  dV^T[d, key] = sum_q dO^T[d, q] P[q, key]
template <int D, bool PAIRED>
__global__ void __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(2, 2)))
flash_dkv_kernel(GenericBackwardArgs a, const float* __restrict__ lse2,
                 const uint16_t* __restrict__ d_out_bf16) {
  constexpr int BNK = 128;
  constexpr int BQ = D == 64 ? 64 : 32;  // query rows per LDS tile
  constexpr int KCH = D / 8, KS = D / 16, DB = D / 32, QB = BQ / 32;
  constexpr int LOADS = BQ * KCH / kThreads;
  constexpr int kTileBytes = BQ * D * 2;
  constexpr int kStatBytes = 256;  // 64 floats
  constexpr int kStageBytes = 2 * kTileBytes + 2 * kStatBytes;
  constexpr int kBlockBytes = 32 * D * 2;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];

  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int T = a.context_length, H = a.num_heads, E = a.embedding_dim;
  const int key_tiles = (T + BNK - 1) / BNK;
  const BackwardUnit unit = backward_unit<PAIRED>(key_tiles, H);
  const int pair = unit.pair, head = unit.head, seq = unit.seq;
  const long long seq_row0 = static_cast<long long>(seq) * T;
  const long long stats_base = (static_cast<long long>(seq) * H + head) * T;
  const uint16_t* qkv = static_cast<const uint16_t*>(a.qkv);
  const uint16_t* q_base = qkv + seq_row0 * 3 * E + head * D;
  const uint16_t* k_base = q_base + E;
  const uint16_t* v_base = q_base + 2 * E;
  const uint16_t* g_base = d_out_bf16 + seq_row0 * E + head * D;
  const float* lse2_base = lse2 + stats_base;
  const float* delta_base = a.deltas + stats_base;  // holds -delta
  const float scale2 = a.scale * kLog2e;
  const int tiles = (T + BQ - 1) / BQ;

  uint32_t q_fill[LOADS], g_fill[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    q_fill[i] = tile_fill_offset<D>((wave * LOADS + i) * 64 + lane, 3LL * E);
    g_fill[i] = tile_fill_offset<D>((wave * LOADS + i) * 64 + lane, 1LL * E);
  }
  int row_read[KS], tr_read[DB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) row_read[ks] = tile_row_read<D>(n, 2 * ks + h);
#pragma unroll
  for (int db = 0; db < DB; ++db) tr_read[db] = tile_transpose_read<D>(lane, db);

  // Key tiles (pair) and (key_tiles-1-pair) together visit the same number of
  // query tiles for every pair.  Query tiles are visited in ascending order
  // within each key tile (fixed reduction order).
  for (int pass = 0; pass < (PAIRED ? 2 : 1); ++pass) {
    const int key_tile = pass == 0 ? pair : key_tiles - 1 - pair;
    if (pass == 1 && key_tile == pair) break;
    const int k0 = key_tile * BNK;
    const int first_tile = k0 / BQ;
    if (first_tile < tiles)
      dkv_fill_stage<D, BQ, LOADS>(lds + ((first_tile) & 1) * kStageBytes, wave, lane, q_base, g_base,
                                   lse2_base, delta_base, E, (first_tile) * BQ, T, q_fill, g_fill);
    const int key_row = k0 + 32 * wave + n;
    const int key_load = min(key_row, T - 1);
    bf16x8 kf[KS], vf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
          k_base + static_cast<long long>(key_load) * 3 * E + 16 * ks + 8 * h));
      vf[ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
          v_base + static_cast<long long>(key_load) * 3 * E + 16 * ks + 8 * h));
    }
    floatx16 dk_acc[DB], dv_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        dk_acc[db][i] = 0.0f;
        dv_acc[db][i] = 0.0f;
      }
    const int wave_first_key = k0 + 32 * wave;

    for (int tile = first_tile; tile < tiles; ++tile) {
      const int q0 = tile * BQ;
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tile + 1 < tiles)
        dkv_fill_stage<D, BQ, LOADS>(lds + ((tile + 1) & 1) * kStageBytes, wave, lane, q_base, g_base,
                                     lse2_base, delta_base, E, (tile + 1) * BQ, T, q_fill, g_fill);
      const unsigned char* q_tile = lds + (tile & 1) * kStageBytes;
      const unsigned char* g_tile = q_tile + kTileBytes;
      const float* stat_lse2 = reinterpret_cast<const float*>(q_tile + 2 * kTileBytes);
      const float* stat_delta = stat_lse2 + kStatBytes / 4;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const int qb0 = q0 + 32 * qb;
        if (qb0 + 31 < wave_first_key) continue;  // every query precedes my keys
        const unsigned char* q_block = q_tile + qb * kBlockBytes;
        const unsigned char* g_block = g_tile + qb * kBlockBytes;
        // transposed operands: requested up front when the register budget
        // allows (64-wide heads), otherwise just before their products
        constexpr bool kHoist = D == 64;
        bf16x8 qt[2][DB], gt[2][DB];
        if constexpr (kHoist) {
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
            for (int db = 0; db < DB; ++db) {
              gt[s2][db] = tile_transposed_operand<D>(g_block, tr_read[db], s2);
              qt[s2][db] = tile_transposed_operand<D>(q_block, tr_read[db], s2);
            }
        }
        // accumulator register i = (query qb0 + 8(i/4) + 4h + i%4, key n); the
        // score accumulator starts from -lse/scale of its query, the dP
        // accumulator from -delta
        floatx16 s, dp;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 l2 = *reinterpret_cast<const float4*>(&stat_lse2[32 * qb + 8 * j + 4 * h]);
          const float4 dl = *reinterpret_cast<const float4*>(&stat_delta[32 * qb + 8 * j + 4 * h]);
          s[4 * j + 0] = l2.x; s[4 * j + 1] = l2.y; s[4 * j + 2] = l2.z; s[4 * j + 3] = l2.w;
          dp[4 * j + 0] = dl.x; dp[4 * j + 1] = dl.y; dp[4 * j + 2] = dl.z; dp[4 * j + 3] = dl.w;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 qa = as_bf16x8(*reinterpret_cast<const uint4*>(q_block + row_read[ks]));
          const bf16x8 ga = as_bf16x8(*reinterpret_cast<const uint4*>(g_block + row_read[ks]));
          s = mfma32(qa, kf[ks], s);
          dp = mfma32(ga, vf[ks], dp);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float p = __builtin_amdgcn_exp2f(s[i] * scale2);
          s[i] = p;
          dp[i] = p * dp[i];
        }
        if (qb0 < wave_first_key + 31 || qb0 + 32 > T) {
          // diagonal block (queries before this lane's key) or sequence tail
          const int first = key_row - qb0 - 4 * h;   // visible: local query >= first
          const int last = T - 1 - qb0 - 4 * h;      //          local query <= last
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int local = 8 * (i / 4) + (i % 4);
            const bool hidden = (local < first) | (local > last);
            s[i] = hidden ? 0.0f : s[i];
            dp[i] = hidden ? 0.0f : dp[i];
          }
        }
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          const bf16x8 pf = accumulator_to_operand(s, s2);
          const bf16x8 dsf = accumulator_to_operand(dp, s2);
          if constexpr (!kHoist) {
#pragma unroll
            for (int db = 0; db < DB; ++db) {
              gt[s2][db] = tile_transposed_operand<D>(g_block, tr_read[db], s2);
              qt[s2][db] = tile_transposed_operand<D>(q_block, tr_read[db], s2);
            }
          }
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            dv_acc[db] = mfma32(gt[s2][db], pf, dv_acc[db]);
            dk_acc[db] = mfma32(qt[s2][db], dsf, dk_acc[db]);
          }
        }
      }
    }
    // dK and dV leave through LDS so that every store instruction writes whole
    // rows (16 lanes x 16 bytes): written straight from the accumulators, a
    // lane's 16-byte pieces lie 9 KiB apart and each store touches 32 lines.
    // One tensor at a time, 32 keys x D floats a wave, pieces swizzled by row.
    __syncthreads();  // every wave is done with the tile stages
    {
      // 64 columns of one tensor at a time: 32 keys x 64 floats a wave, 32 KiB
      static_assert(4 * 32 * 64 * 4 <= 2 * kStageBytes, "the stages hold one step of the workgroup");
      constexpr int kPieces = 16;  // 16-byte pieces in 64 columns
      float4* area = reinterpret_cast<float4*>(lds) + wave * 32 * kPieces;
      const int out_piece = lane % kPieces, out_row = lane / kPieces;
#pragma unroll
      for (int step = 0; step < 2 * (D / 64); ++step) {
        const int tensor = step / (D / 64), half = step % (D / 64);
#pragma unroll
        for (int d2 = 0; d2 < 2; ++d2)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const floatx16& acc = tensor == 0 ? dk_acc[2 * half + d2] : dv_acc[2 * half + d2];
            const float factor = tensor == 0 ? a.scale : 1.0f;
            float4 value;
            value.x = acc[4 * j + 0] * factor;
            value.y = acc[4 * j + 1] * factor;
            value.z = acc[4 * j + 2] * factor;
            value.w = acc[4 * j + 3] * factor;
            const int piece = 8 * d2 + 2 * j + h;
            area[n * kPieces + (piece ^ (n % kPieces))] = value;
          }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wave reads what its own lanes wrote
        float* dst = a.d_qkv + (seq_row0 + k0 + 32 * wave) * 3 * E + (1 + tensor) * E + head * D +
                     64 * half;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int row = 4 * i + out_row;
          const float4 value = area[row * kPieces + (out_piece ^ (row % kPieces))];
          if (k0 + 32 * wave + row < T)
            *reinterpret_cast<float4*>(dst + static_cast<long long>(row) * 3 * E + 4 * out_piece) = value;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // before the area is overwritten
      }
    }
    __syncthreads();  // the next pass refills a stage
  }
}

}  // namespace

bool flash_backward_supported(const GenericBackwardArgs& a) {
  const int dim = a.embedding_dim / a.num_heads;
  if (a.dtype != PLUTO_HIP_BF16 || (dim != 64 && dim != 128)) return false;
  auto aligned = [](const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
  };
  // tiles of one sequence are addressed through 32-bit buffer offsets and a
  // 32-bit descriptor size: a sequence's rows of the packed operand (the
  // widest, 3E bf16 per row) must stay below 2 GiB
  if (static_cast<long long>(a.context_length) * 3 * a.embedding_dim * 2 >= (1LL << 31))
    return false;
  return aligned(a.qkv) && aligned(a.out) && aligned(a.d_out) && aligned(a.d_qkv);
}

int launch_flash_backward(hipStream_t stream, const GenericBackwardArgs& a,
                          float* lse2, uint16_t* d_out_bf16) {
  const int dim = a.embedding_dim / a.num_heads;
  const int sequences = a.rows / a.context_length;
  int status = 0;
  const long long tiles128 = (a.context_length + 127) / 128;
  const long long units = 1LL * a.num_heads * sequences;
  if (tiles128 * units > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  const dim3 paired(static_cast<unsigned>(((tiles128 + 1) / 2) * units));
  const dim3 unpaired(static_cast<unsigned>(tiles128 * units));
  if (!kernel_enabled(kQueryKernel)) {
  } else if (dim == 64)
    flash_dq_kernel<64, kDqPaired64><<<kDqPaired64 ? paired : unpaired, kThreads, 0, stream>>>(
        a, lse2, d_out_bf16);
  else
    flash_dq_kernel<128, kOtherPaired><<<kOtherPaired ? paired : unpaired, kThreads, 0, stream>>>(
        a, lse2, d_out_bf16);
  status = launch_status();
  if (status != 0) return status;
  if (!kernel_enabled(kMainKernel)) return 0;
  // The hand-scheduled kernel (one wave a SIMD, 64 keys a wave) gives the same
  // bits; it is level with the kernel below at 2048 rows and 6 % ahead at 4096.
  if (dim == 64 && kernel_enabled(kEightWave) &&
      (a.context_length >= kWideFromRows || !kernel_enabled(kFromLength)))
    return launch_flash_dkv_wide(stream, a, lse2, d_out_bf16);
  if (dim == 64)
    flash_dkv_kernel<64, kOtherPaired><<<kOtherPaired ? paired : unpaired, kThreads, 0, stream>>>(
        a, lse2, d_out_bf16);
  else
    flash_dkv_kernel<128, kOtherPaired><<<kOtherPaired ? paired : unpaired, kThreads, 0, stream>>>(
        a, lse2, d_out_bf16);
  return launch_status();
}

}  // namespace pluto_hip
