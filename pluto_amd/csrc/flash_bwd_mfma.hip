// Causal flash attention backward for bf16 activations on gfx950 matrix cores.
//
// Contract of AttentionLayer::bwd_impl (src/llm/layers/attention.cc:509-596):
// packed bf16 Q|K|V and stored bf16 output, FP32 upstream gradient, FP32 packed
// gradient out; query-owned dQ and key-owned dK/dV with a fixed reduction
// order and no atomics, hence bitwise repeatable.
//
// Three kernels:
//   prepare   delta = sum(dO * O) per (row, head) (attention.cc:283-291), the
//             row's log2-sum-exp, and a bf16 copy of dO for the matrix cores.
//   dq        one workgroup per 128 queries, loops over 64-key tiles.
//   dkv       one workgroup per 128 keys, loops over 64-query tiles in
//             ascending order.
// All products use v_mfma_f32_32x32x16_bf16 in the orientation that keeps the
// score tile's accumulator directly usable as the B operand of the gradient
// product (see mfma_tile.h): dq works on S^T (lane = query), dkv on S
// (lane = key).  Deviation, within the stated bf16 tolerance: P, dS and dO are
// rounded to bf16 for the matrix products (the reference keeps them FP32).
#include "flash_bwd_mfma.h"

#include "mfma_tile.h"

namespace pluto_hip {
namespace {

constexpr int kThreads = 256;
constexpr int kTileRows = 64;  // rows of the streamed operand per LDS tile

// 8 channels per thread (16-byte loads of O, 2 x 16 bytes of dO); the D/8
// threads of one (row, head) are neighbouring lanes and reduce with shuffles.
template <int D>
__global__ void __launch_bounds__(256)
backward_prepare_kernel(GenericBackwardArgs a, float* lse2, uint16_t* d_out_bf16) {
  constexpr int LANES = D / 8;
  const long long piece = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  const long long pieces = static_cast<long long>(a.rows) * a.embedding_dim / 8;
  if (piece >= pieces) return;  // whole (row, head) groups drop out together
  const long long base = piece * 8;
  const float4 g0 = *reinterpret_cast<const float4*>(a.d_out + base);
  const float4 g1 = *reinterpret_cast<const float4*>(a.d_out + base + 4);
  const uint4 o = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(a.out) + base);
  const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
  const uint32_t ow[4] = {o.x, o.y, o.z, o.w};
  float sum = 0.0f;
  uint32_t packed[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    sum += g[2 * i] * __uint_as_float(ow[i] << 16);
    sum += g[2 * i + 1] * __uint_as_float(ow[i] & 0xffff0000u);
    packed[i] = pack_bf16(g[2 * i], g[2 * i + 1]);
  }
  *reinterpret_cast<uint4*>(d_out_bf16 + base) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
#pragma unroll
  for (int offset = 1; offset < LANES; offset <<= 1) sum += __shfl_xor(sum, offset, 64);
  if (piece % LANES == 0) {
    const long long unit = piece / LANES;  // row * H + head
    const int row = static_cast<int>(unit / a.num_heads);
    const int head = static_cast<int>(unit % a.num_heads);
    const int seq = row / a.context_length, pos = row % a.context_length;
    const long long stat =
        (static_cast<long long>(seq) * a.num_heads + head) * a.context_length + pos;
    a.deltas[stat] = sum;
    const float normalizer = a.normalizers[stat];
    lse2[stat] = a.maxima[stat] * kLog2e + __log2f(normalizer > 0.0f ? normalizer : 1.0f);
  }
}

template <int D>
struct DqSmem {
  static constexpr int KCH = D / 8;
  uint4 k_rm[kTileRows * KCH];       // K tile, row major
  uint4 v_rm[kTileRows * KCH];       // V tile, row major
  uint4 k_tr[D * (kTileRows / 8)];   // K tile, transposed, accumulator order
};

// dQ^T[d, query] = sum_keys K^T[d, key] dS^T[key, query]
template <int D>
__global__ void __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(D == 64 ? 3 : 1, D == 64 ? 3 : 2)))
flash_dq_kernel(GenericBackwardArgs a, const float* __restrict__ lse2,
                const uint16_t* __restrict__ d_out_bf16) {
  constexpr int BM = 128, BN = kTileRows;
  constexpr int KCH = D / 8, KS = D / 16, DB = D / 32, KB = BN / 32;
  constexpr int LOADS = BN * KCH / 128;
  __shared__ DqSmem<D> sm;

  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int T = a.context_length, H = a.num_heads, E = a.embedding_dim;
  const int q_tiles = (T + BM - 1) / BM;
  const int pairs = (q_tiles + 1) / 2;
  const int logical = xcd_logical_block();
  const int pair = logical % pairs;
  const int head = (logical / pairs) % H;
  const int seq = logical / (pairs * H);
  const long long seq_row0 = static_cast<long long>(seq) * T;
  const long long stats_base = (static_cast<long long>(seq) * H + head) * T;
  const uint16_t* qkv = static_cast<const uint16_t*>(a.qkv);
  const uint16_t* q_base = qkv + seq_row0 * 3 * E + head * D;
  const uint16_t* k_base = q_base + E;
  const uint16_t* v_base = q_base + 2 * E;
  const uint16_t* g_base = d_out_bf16 + seq_row0 * E + head * D;
  const float scale2 = a.scale * kLog2e;

  uint4 staged[LOADS];
  const int ltid = tid % 128;
  const bool loads_k = tid < 128;
  // Rows beyond the sequence are clamped to its last row; every product they
  // enter is masked (keys) or never stored (queries).
  auto fetch = [&](int tile) {
    const int k0 = tile * BN;
    if (loads_k) {
#pragma unroll
      for (int u = 0; u < LOADS / 4; ++u) {
        const int unit = ltid + 128 * u;
        const int quad = unit / KCH, g = unit % KCH;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int key = min(k0 + 4 * quad + r, T - 1);
          staged[4 * u + r] = *reinterpret_cast<const uint4*>(
              k_base + static_cast<long long>(key) * 3 * E + 8 * g);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < LOADS; ++i) {
        const int c = ltid + 128 * i;
        const int key = min(k0 + c / KCH, T - 1);
        staged[i] = *reinterpret_cast<const uint4*>(
            v_base + static_cast<long long>(key) * 3 * E + 8 * (c % KCH));
      }
    }
  };
  auto commit = [&]() {
    if (loads_k) {
#pragma unroll
      for (int u = 0; u < LOADS / 4; ++u) {
        const int unit = ltid + 128 * u;
        const int quad = unit / KCH, g = unit % KCH;
#pragma unroll
        for (int r = 0; r < 4; ++r)
          sm.k_rm[row_major_index<KCH>(4 * quad + r, g)] = staged[4 * u + r];
        transposed_store<BN>(sm.k_tr, quad, g, staged[4 * u + 0], staged[4 * u + 1],
                             staged[4 * u + 2], staged[4 * u + 3]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < LOADS; ++i) {
        const int c = ltid + 128 * i;
        sm.v_rm[row_major_index<KCH>(c / KCH, c % KCH)] = staged[i];
      }
    }
  };

  // Query tiles (q_tiles-1-pair) and (pair) together see the same number of
  // keys for every pair: equal work per workgroup under the causal mask.
  for (int pass = 0; pass < 2; ++pass) {
    const int q_tile = pass == 0 ? q_tiles - 1 - pair : pair;
    if (pass == 1 && q_tile == q_tiles - 1 - pair) break;
    const int q0 = q_tile * BM;
    const int q_row = q0 + 32 * wave + n;
    const int q_load = min(q_row, T - 1);
    bf16x8 qf[KS], gf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
          q_base + static_cast<long long>(q_load) * 3 * E + 16 * ks + 8 * h));
      gf[ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
          g_base + static_cast<long long>(q_load) * E + 16 * ks + 8 * h));
    }
    const float row_lse2 = lse2[stats_base + q_load];
    const float row_delta = a.deltas[stats_base + q_load];
    floatx16 dq_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) dq_acc[db][i] = 0.0f;

    const int last_row = min(q0 + BM, T) - 1;
    const int tiles = last_row / BN + 1;
    const int wave_first_row = q0 + 32 * wave;
    const int wave_last_key = wave_first_row + 31;

    fetch(0);
    for (int tile = 0; tile < tiles; ++tile) {
      const int k0 = tile * BN;
      __syncthreads();
      commit();
      __syncthreads();
      if (tile + 1 < tiles) fetch(tile + 1);
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int kb0 = k0 + 32 * kb;
        if (kb0 > wave_last_key) continue;
        floatx16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          s[i] = 0.0f;
          dp[i] = 0.0f;
        }
        const int key = 32 * kb + n;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 kf = as_bf16x8(sm.k_rm[row_major_index<KCH>(key, 2 * ks + h)]);
          const bf16x8 vf = as_bf16x8(sm.v_rm[row_major_index<KCH>(key, 2 * ks + h)]);
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
          const int chunk = 4 * kb + 2 * s2 + h;
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const int d = 32 * db + n;
            const bf16x8 ktf = as_bf16x8(sm.k_tr[transposed_index<BN>(d, chunk)]);
            dq_acc[db] = mfma32(ktf, dsf, dq_acc[db]);
          }
        }
      }
    }
    if (q_row < T) {
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
  }
}

template <int D>
struct DkvSmem {
  static constexpr int KCH = D / 8;
  uint4 q_rm[kTileRows * KCH];       // Q tile, row major
  uint4 g_rm[kTileRows * KCH];       // dO tile, row major
  uint4 q_tr[D * (kTileRows / 8)];   // Q tile, transposed, accumulator order
  uint4 g_tr[D * (kTileRows / 8)];   // dO tile, transposed, accumulator order
  float lse2[kTileRows];
  float delta[kTileRows];
};

// dK^T[d, key] = sum_q Q^T[d, q] dS[q, key];  dV^T[d, key] = sum_q dO^T[d, q] P[q, key]
template <int D>
__global__ void __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(D == 64 ? 2 : 1, D == 64 ? 2 : 2)))
flash_dkv_kernel(GenericBackwardArgs a, const float* __restrict__ lse2,
                 const uint16_t* __restrict__ d_out_bf16) {
  constexpr int BNK = 128, BQ = kTileRows;
  constexpr int KCH = D / 8, KS = D / 16, DB = D / 32, QB = BQ / 32;
  constexpr int LOADS = BQ * KCH / 128;
  __shared__ DkvSmem<D> sm;

  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int T = a.context_length, H = a.num_heads, E = a.embedding_dim;
  const int key_tiles = (T + BNK - 1) / BNK;
  const int pairs = (key_tiles + 1) / 2;
  const int logical = xcd_logical_block();
  const int pair = logical % pairs;
  const int head = (logical / pairs) % H;
  const int seq = logical / (pairs * H);
  const long long seq_row0 = static_cast<long long>(seq) * T;
  const long long stats_base = (static_cast<long long>(seq) * H + head) * T;
  const uint16_t* qkv = static_cast<const uint16_t*>(a.qkv);
  const uint16_t* q_base = qkv + seq_row0 * 3 * E + head * D;
  const uint16_t* k_base = q_base + E;
  const uint16_t* v_base = q_base + 2 * E;
  const uint16_t* g_base = d_out_bf16 + seq_row0 * E + head * D;
  const float scale2 = a.scale * kLog2e;
  const int tiles = (T + BQ - 1) / BQ;

  uint4 staged[LOADS];
  float staged_stat = 0.0f;
  const int ltid = tid % 128;
  const bool loads_q = tid < 128;
  // Query rows beyond the sequence are clamped to its last row and masked.
  auto fetch = [&](int tile) {
    const int q0 = tile * BQ;
    const uint16_t* base = loads_q ? q_base : g_base;
    const long long stride = loads_q ? 3LL * E : 1LL * E;
#pragma unroll
    for (int u = 0; u < LOADS / 4; ++u) {
      const int unit = ltid + 128 * u;
      const int quad = unit / KCH, g = unit % KCH;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = min(q0 + 4 * quad + r, T - 1);
        staged[4 * u + r] = *reinterpret_cast<const uint4*>(base + row * stride + 8 * g);
      }
    }
    if (ltid < BQ) {
      const int row = min(q0 + ltid, T - 1);
      staged_stat = loads_q ? lse2[stats_base + row] : a.deltas[stats_base + row];
    }
  };
  auto commit = [&]() {
    uint4* rm = loads_q ? sm.q_rm : sm.g_rm;
    uint4* tr = loads_q ? sm.q_tr : sm.g_tr;
#pragma unroll
    for (int u = 0; u < LOADS / 4; ++u) {
      const int unit = ltid + 128 * u;
      const int quad = unit / KCH, g = unit % KCH;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        rm[row_major_index<KCH>(4 * quad + r, g)] = staged[4 * u + r];
      transposed_store<BQ>(tr, quad, g, staged[4 * u + 0], staged[4 * u + 1],
                           staged[4 * u + 2], staged[4 * u + 3]);
    }
    if (ltid < BQ) (loads_q ? sm.lse2 : sm.delta)[ltid] = staged_stat;
  };

  // Key tiles (pair) and (key_tiles-1-pair) together visit the same number of
  // query tiles for every pair.  Query tiles are visited in ascending order
  // within each key tile (fixed reduction order).
  for (int pass = 0; pass < 2; ++pass) {
    const int key_tile = pass == 0 ? pair : key_tiles - 1 - pair;
    if (pass == 1 && key_tile == pair) break;
    const int k0 = key_tile * BNK;
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
    const int first_tile = k0 / BQ;
    const int wave_first_key = k0 + 32 * wave;

    if (first_tile < tiles) fetch(first_tile);
    for (int tile = first_tile; tile < tiles; ++tile) {
      const int q0 = tile * BQ;
      __syncthreads();
      commit();
      __syncthreads();
      if (tile + 1 < tiles) fetch(tile + 1);
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const int qb0 = q0 + 32 * qb;
        if (qb0 + 31 < wave_first_key) continue;  // every query precedes my keys
        floatx16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          s[i] = 0.0f;
          dp[i] = 0.0f;
        }
        const int q_local = 32 * qb + n;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 qa = as_bf16x8(sm.q_rm[row_major_index<KCH>(q_local, 2 * ks + h)]);
          const bf16x8 ga = as_bf16x8(sm.g_rm[row_major_index<KCH>(q_local, 2 * ks + h)]);
          s = mfma32(qa, kf[ks], s);
          dp = mfma32(ga, vf[ks], dp);
        }
        // accumulator register i = (query qb0 + 8(i/4) + 4h + i%4, key n)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 l2 = *reinterpret_cast<const float4*>(&sm.lse2[32 * qb + 8 * j + 4 * h]);
          const float4 dl = *reinterpret_cast<const float4*>(&sm.delta[32 * qb + 8 * j + 4 * h]);
          const float l2v[4] = {l2.x, l2.y, l2.z, l2.w};
          const float dlv[4] = {dl.x, dl.y, dl.z, dl.w};
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int i = 4 * j + r;
            const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], scale2, -l2v[r]));
            s[i] = p;
            dp[i] = p * (dp[i] - dlv[r]);
          }
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
          const int chunk = 4 * qb + 2 * s2 + h;
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const int d = 32 * db + n;
            const bf16x8 gt = as_bf16x8(sm.g_tr[transposed_index<BQ>(d, chunk)]);
            const bf16x8 qt = as_bf16x8(sm.q_tr[transposed_index<BQ>(d, chunk)]);
            dv_acc[db] = mfma32(gt, pf, dv_acc[db]);
            dk_acc[db] = mfma32(qt, dsf, dk_acc[db]);
          }
        }
      }
    }
    if (key_row < T) {
      float* dk = a.d_qkv + (seq_row0 + key_row) * 3 * E + E + head * D;
      float* dv = dk + E;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float4 kv, vv;
          kv.x = dk_acc[db][4 * j + 0] * a.scale;
          kv.y = dk_acc[db][4 * j + 1] * a.scale;
          kv.z = dk_acc[db][4 * j + 2] * a.scale;
          kv.w = dk_acc[db][4 * j + 3] * a.scale;
          vv.x = dv_acc[db][4 * j + 0];
          vv.y = dv_acc[db][4 * j + 1];
          vv.z = dv_acc[db][4 * j + 2];
          vv.w = dv_acc[db][4 * j + 3];
          *reinterpret_cast<float4*>(dk + 32 * db + 8 * j + 4 * h) = kv;
          *reinterpret_cast<float4*>(dv + 32 * db + 8 * j + 4 * h) = vv;
        }
    }
  }
}

}  // namespace

bool flash_backward_supported(const GenericBackwardArgs& a) {
  const int dim = a.embedding_dim / a.num_heads;
  if (a.dtype != PLUTO_HIP_BF16 || (dim != 64 && dim != 128)) return false;
  auto aligned = [](const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
  };
  return aligned(a.qkv) && aligned(a.out) && aligned(a.d_out) && aligned(a.d_qkv);
}

int launch_flash_backward(hipStream_t stream, const GenericBackwardArgs& a,
                          float* lse2, uint16_t* d_out_bf16) {
  const int dim = a.embedding_dim / a.num_heads;
  const int sequences = a.rows / a.context_length;
  const long long pieces = static_cast<long long>(a.rows) * a.embedding_dim / 8;
  const unsigned prepare_blocks = static_cast<unsigned>((pieces + 255) / 256);
  if (dim == 64)
    backward_prepare_kernel<64><<<prepare_blocks, 256, 0, stream>>>(a, lse2, d_out_bf16);
  else
    backward_prepare_kernel<128><<<prepare_blocks, 256, 0, stream>>>(a, lse2, d_out_bf16);
  int status = launch_status();
  if (status != 0) return status;
  const long long tiles128 = (a.context_length + 127) / 128;
  const long long blocks = ((tiles128 + 1) / 2) * a.num_heads * sequences;
  if (blocks > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  dim3 grid(static_cast<unsigned>(blocks));
  if (dim == 64)
    flash_dq_kernel<64><<<grid, kThreads, 0, stream>>>(a, lse2, d_out_bf16);
  else
    flash_dq_kernel<128><<<grid, kThreads, 0, stream>>>(a, lse2, d_out_bf16);
  status = launch_status();
  if (status != 0) return status;
  if (dim == 64)
    flash_dkv_kernel<64><<<grid, kThreads, 0, stream>>>(a, lse2, d_out_bf16);
  else
    flash_dkv_kernel<128><<<grid, kThreads, 0, stream>>>(a, lse2, d_out_bf16);
  return launch_status();
}

}  // namespace pluto_hip
