// Causal flash attention forward for bf16 activations on gfx950 matrix cores.
//
// One workgroup (4 wave64) owns 128 query rows of one (sequence, head); wave w
// owns rows 32w..32w+31.  Key/value tiles of 64 rows are staged through LDS.
// Both products are computed transposed with v_mfma_f32_32x32x16_bf16:
//
//   S^T[key, query] = K[key, :] . Q[query, :]      A = K (LDS), B = Q (regs)
//   O^T[d,   query] = V^T[d, key] . P^T[key, query] A = V^T (LDS), B = P^T
//
// In the 32x32 accumulator layout lane l holds column (l % 32), i.e. ONE query,
// so the softmax row statistics are per-lane scalars and need a single
// cross-lane exchange (lane ^ 32) per tile, and the probabilities leave the
// accumulator registers already laid out as the B operand of the second
// product: no shuffle, no LDS round trip.  The contraction index of an MFMA
// may be enumerated in any order as long as A and B agree, so V^T is written to
// LDS with its keys permuted to the order in which the accumulator registers
// hold them.
//
// Semantics follow FlashAttentionForwardKernel (src/llm/layers/attention.cc:
// 98-170) and, with the gate epilogue, ForwardKernel
// (src/llm/layers/qwen_attention.cc:68-119).  Deviation, within the stated
// bf16 tolerance: probabilities are rounded to bf16 for the P.V product (the
// reference keeps them FP32, attention.cc:151-156).
#include "flash_fwd_mfma.h"

#include "mfma_tile.h"

namespace pluto_hip {
namespace {

constexpr int BM = 128;  // query rows per workgroup
constexpr int BN = 64;   // keys per LDS tile
constexpr int kThreads = 256;

template <int D>
struct Smem {
  static constexpr int KCH = D / 8;  // 16-byte chunks per K row
  // K tile, row major: chunk (key, ch) at key*KCH + (ch ^ (key & 7)).
  uint4 k[BN * KCH];
  // V^T tile: row d holds BN keys as 8 chunks of 8 keys in accumulator order;
  // chunk c of row d at d*(BN/8) + (c ^ swizzle_d(d)).
  uint4 vt[D * (BN / 8)];
};

// Register budget: 4 waves per SIMD for 64-wide heads (128 VGPRs), 2 for
// 128-wide heads, so that several workgroups per CU overlap their matrix-core
// and vector phases.
template <int D>
__global__ void __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(D == 64 ? 3 : 2, D == 64 ? 3 : 2)))
flash_forward_kernel(FlashForwardArgs a) {
  constexpr int KCH = D / 8;
  constexpr int KS = D / 16;      // contraction steps of S^T
  constexpr int DB = D / 32;      // 32-row blocks of O^T
  constexpr int KB = BN / 32;     // 32-key blocks per tile
  constexpr int OSTRIDE = D * 2 + 16;  // bytes per staged output row
  __shared__ __attribute__((aligned(16))) unsigned char raw[
      sizeof(Smem<D>) > BM * OSTRIDE ? sizeof(Smem<D>) : BM * OSTRIDE];
  Smem<D>& sm = *reinterpret_cast<Smem<D>*>(raw);

  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int q_tiles = (a.q_rows + BM - 1) / BM;
  const int pairs = (q_tiles + 1) / 2;
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.
  // Renumber them so that the workgroups sharing one (sequence, kv head) K/V
  // stream run on the same XCD.
  const int logical = xcd_logical_block();
  const int pair = logical % pairs;
  const int head = (logical / pairs) % a.query_heads;
  const int seq = logical / (pairs * a.query_heads);
  const int kv_head = head / a.group;

  const uint16_t* q_base = a.q + seq * a.q_seq_stride + head * a.q_head_stride;
  const uint16_t* k_base = a.k + seq * a.k_seq_stride + kv_head * a.k_head_stride;
  const uint16_t* v_base = a.v + seq * a.v_seq_stride + kv_head * a.v_head_stride;
  uint16_t* o_base = a.out + seq * a.o_seq_stride + head * a.o_head_stride;
  const uint16_t* gate_base =
      a.gate ? a.gate + seq * a.gate_seq_stride + head * a.gate_head_stride : nullptr;
  const float scale2 = a.scale * kLog2e;
  bf16x8 ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = static_cast<__bf16>(1.0f);

  // Loader roles: waves 0-1 fetch K (row major), waves 2-3 fetch V and
  // transpose it in registers.  Both move BN*D*2 bytes per tile with
  // 16-byte loads.
  constexpr int LOADS = BN * KCH / 128;  // 16-byte loads per loader thread
  uint4 staged[LOADS];
  const int ltid = tid % 128;
  const bool loads_k = tid < 128;

  auto fetch = [&](int tile) {
    const int k0 = tile * BN;
    if (loads_k) {
#pragma unroll
      for (int i = 0; i < LOADS; ++i) {
        const int c = ltid + 128 * i;
        const int key = c / KCH, ch = c % KCH;
        // rows beyond the valid prefix are clamped to its last row: their
        // scores are masked, and a finite row keeps 0 * V finite
        const int row = min(k0 + key, a.kv_rows - 1);
        staged[i] = *reinterpret_cast<const uint4*>(
            k_base + static_cast<long long>(row) * a.k_row_stride + 8 * ch);
      }
    } else {
      // unit = (key quad, channel group); 4 loads (one per key) per unit.
#pragma unroll
      for (int u = 0; u < LOADS / 4; ++u) {
        const int unit = ltid + 128 * u;
        const int quad = unit / KCH, g = unit % KCH;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = min(k0 + 4 * quad + r, a.kv_rows - 1);
          staged[4 * u + r] = *reinterpret_cast<const uint4*>(
              v_base + static_cast<long long>(row) * a.v_row_stride + 8 * g);
        }
      }
    }
  };

  auto commit = [&]() {
    if (loads_k) {
#pragma unroll
      for (int i = 0; i < LOADS; ++i) {
        const int c = ltid + 128 * i;
        const int key = c / KCH, ch = c % KCH;
        sm.k[row_major_index<KCH>(key, ch)] = staged[i];
      }
    } else {
#pragma unroll
      for (int u = 0; u < LOADS / 4; ++u) {
        const int unit = ltid + 128 * u;
        transposed_store<BN>(sm.vt, unit / KCH, unit % KCH, staged[4 * u + 0],
                             staged[4 * u + 1], staged[4 * u + 2],
                             staged[4 * u + 3]);
      }
    }
  };

  // A workgroup processes query tile (q_tiles-1-pair) and then tile `pair`:
  // under the causal mask their key counts add up to the same total for every
  // pair, so all workgroups carry equal work.
  for (int pass = 0; pass < 2; ++pass) {
    const int q_tile = pass == 0 ? q_tiles - 1 - pair : pair;
    if (pass == 1 && q_tile == q_tiles - 1 - pair) break;
    const int q0 = q_tile * BM;
    const int q_row = q0 + 32 * wave + n;

    // Q fragments (B operand of S^T): row q_row, channels 16ks + 8h .. +7.
    bf16x8 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int row = min(q_row, a.q_rows - 1);
      qf[ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
          q_base + static_cast<long long>(row) * a.q_row_stride + 16 * ks + 8 * h));
    }
    floatx16 o_acc[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o_acc[db][i] = 0.0f;
    // Online softmax in the log2 domain with a lazily updated reference
    // point: probabilities are 2^(s*scale2 - m_used); m_used follows the
    // running row maximum only when that has grown by more than kLazy, so
    // the accumulator rescale is rare.  The true maximum is tracked
    // separately and the saved statistics are converted to it at the end.
    constexpr float kLazy = 8.0f;
    float m_used = kMasked;   // reference point, score * scale * log2(e) units
    float m_true = kMasked;   // running maximum of the raw scores
    // Row sums come out of the matrix cores: an all-ones A operand makes
    // every row of this accumulator the sum over keys of the bf16
    // probabilities.
    floatx16 l_acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) l_acc[i] = 0.0f;

    const int last_row = min(q0 + BM, a.q_rows) - 1;
    const int visible = min(a.kv_rows, a.start_position + last_row + 1);
    const int tiles = (visible + BN - 1) / BN;
    const int wave_last_key = a.start_position + q0 + 32 * wave + 31;
    // keys up to `row_limit` are visible to this lane's query
    const int row_limit = min(a.start_position + q_row, a.kv_rows - 1);

    if (tiles > 0) fetch(0);
    for (int tile = 0; tile < tiles; ++tile) {
      const int k0 = tile * BN;
      __syncthreads();  // everyone finished reading the previous tile
      commit();
      __syncthreads();
      if (tile + 1 < tiles) fetch(tile + 1);
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int kb0 = k0 + 32 * kb;
        if (kb0 > wave_last_key) continue;  // nothing visible to this wave's rows
        // ---- S^T = K Q^T for 32 keys ------------------------------------
        floatx16 s;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = 0.0f;
        const int key = 32 * kb + n;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const bf16x8 kf = as_bf16x8(sm.k[row_major_index<KCH>(key, 2 * ks + h)]);
          s = mfma32(kf, qf[ks], s);
        }
        // ---- mask (diagonal and tail blocks only), row maximum ----------
        if (kb0 + 31 > a.start_position + q0 + 32 * wave || kb0 + 32 > a.kv_rows) {
          const int limit = row_limit - kb0 - 4 * h;
#pragma unroll
          for (int i = 0; i < 16; ++i) s[i] = (8 * (i / 4) + (i % 4) > limit) ? kMasked : s[i];
        }
        float row_max = fmaxf(s[0], s[1]);
#pragma unroll
        for (int i = 2; i < 16; i += 2) row_max = fmaxf(row_max, fmaxf(s[i], s[i + 1]));
        row_max = fmaxf(row_max, __shfl_xor(row_max, 32, 64));
        m_true = fmaxf(m_true, row_max);
        const float candidate = m_true * scale2;
        if (__any(candidate > m_used + kLazy)) {
          const float m_new = candidate > m_used + kLazy ? candidate : m_used;
          const float alpha = __builtin_amdgcn_exp2f(m_used - m_new);
          m_used = m_new;
          l_acc[0] *= alpha;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) o_acc[db][i] *= alpha;
        }
        // ---- P^T = 2^(S^T scale2 - m_used); O^T += V^T P^T; l += 1^T P^T
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
          uint32_t packed[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            floatx2 two;
            two[0] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[8 * s2 + 2 * e], scale2, -m_used));
            two[1] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[8 * s2 + 2 * e + 1], scale2, -m_used));
            packed[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(two, bf16x2));
          }
          const bf16x8 pf =
              __builtin_bit_cast(bf16x8, make_uint4(packed[0], packed[1], packed[2], packed[3]));
          const int chunk = 4 * kb + 2 * s2 + h;
          l_acc = mfma32(ones, pf, l_acc);
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const int d = 32 * db + n;
            const bf16x8 vf = as_bf16x8(sm.vt[transposed_index<BN>(d, chunk)]);
            o_acc[db] = mfma32(vf, pf, o_acc[db]);
          }
        }
      }
    }

    // ---- epilogue ----------------------------------------------------------
    // l_acc holds the sum over all keys (both lane halves contract into the
    // same accumulator column).
    const float l_used = l_acc[0] > 0.0f ? l_acc[0] : 1.0f;
    const float inverse = 1.0f / l_used;
    __syncthreads();  // LDS is reused to transpose the output tile
    {
      unsigned char* row = raw + (32 * wave + n) * OSTRIDE;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int d = 32 * db + 8 * j + 4 * h;
          floatx2 lo = {o_acc[db][4 * j] * inverse, o_acc[db][4 * j + 1] * inverse};
          floatx2 hi = {o_acc[db][4 * j + 2] * inverse, o_acc[db][4 * j + 3] * inverse};
          uint2 packed;
          packed.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(lo, bf16x2));
          packed.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, bf16x2));
          *reinterpret_cast<uint2*>(row + 2 * d) = packed;
        }
    }
    if (h == 0 && q_row < a.q_rows) {
      // statistics relative to the true maximum: attention.cc:161-168
      const float normalizer = l_used * __builtin_amdgcn_exp2f(m_used - m_true * scale2);
      const float maximum = m_true * a.scale;
      const long long stat =
          (static_cast<long long>(seq) * a.query_heads + head) * a.q_rows + q_row;
      if (a.maxima) a.maxima[stat] = maximum;
      if (a.normalizers) a.normalizers[stat] = normalizer;
      if (a.lse)
        a.lse[(static_cast<long long>(seq) * a.q_rows + q_row) * a.query_heads + head] =
            maximum + __logf(normalizer);
    }
    __syncthreads();
    for (int c = tid; c < BM * KCH; c += kThreads) {
      const int r = c / KCH, ch = c % KCH;
      const int row = q0 + r;
      if (row >= a.q_rows) continue;
      uint4 bits = *reinterpret_cast<const uint4*>(raw + r * OSTRIDE + 16 * ch);
      if (gate_base) {
        // out = bf16(bf16(core) * bf16(sigmoid(gate))): qwen_attention.cc:103-108
        const uint4 gate_bits = *reinterpret_cast<const uint4*>(
            gate_base + static_cast<long long>(row) * a.gate_row_stride + 8 * ch);
        const uint32_t cw[4] = {bits.x, bits.y, bits.z, bits.w};
        const uint32_t gw[4] = {gate_bits.x, gate_bits.y, gate_bits.z, gate_bits.w};
        uint32_t ow[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float c0 = __uint_as_float(cw[e] << 16), c1 = __uint_as_float(cw[e] & 0xffff0000u);
          const float g0 = __uint_as_float(gw[e] << 16), g1 = __uint_as_float(gw[e] & 0xffff0000u);
          const float s0 = round_to_bf16(1.0f / (1.0f + expf(-g0)));
          const float s1 = round_to_bf16(1.0f / (1.0f + expf(-g1)));
          ow[e] = static_cast<uint32_t>(float_to_bf16_bits(c0 * s0)) |
                  (static_cast<uint32_t>(float_to_bf16_bits(c1 * s1)) << 16);
        }
        bits = make_uint4(ow[0], ow[1], ow[2], ow[3]);
      }
      *reinterpret_cast<uint4*>(o_base + static_cast<long long>(row) * a.o_row_stride +
                                8 * ch) = bits;
    }
  }
}

}  // namespace

bool flash_forward_supported(const FlashForwardArgs& a, int head_dim) {
  if (head_dim != 64 && head_dim != 128) return false;
  auto aligned = [](const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
  };
  auto mult8 = [](long long s) { return (s % 8) == 0; };
  if (!aligned(a.q) || !aligned(a.k) || !aligned(a.v) || !aligned(a.out))
    return false;
  if (a.gate && !aligned(a.gate)) return false;
  return mult8(a.q_seq_stride) && mult8(a.q_row_stride) && mult8(a.q_head_stride) &&
         mult8(a.k_seq_stride) && mult8(a.k_row_stride) && mult8(a.k_head_stride) &&
         mult8(a.v_seq_stride) && mult8(a.v_row_stride) && mult8(a.v_head_stride) &&
         mult8(a.o_seq_stride) && mult8(a.o_row_stride) && mult8(a.o_head_stride) &&
         mult8(a.gate_seq_stride) && mult8(a.gate_row_stride) &&
         mult8(a.gate_head_stride);
}

int launch_flash_forward(hipStream_t stream, const FlashForwardArgs& a,
                         int head_dim, int sequences) {
  if (!flash_forward_supported(a, head_dim)) return PLUTO_HIP_EUNSUPPORTED;
  const long long q_tiles = (a.q_rows + BM - 1) / BM;
  const long long blocks = ((q_tiles + 1) / 2) * a.query_heads * sequences;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  dim3 grid(static_cast<unsigned>(blocks));
  if (head_dim == 64)
    flash_forward_kernel<64><<<grid, kThreads, 0, stream>>>(a);
  else
    flash_forward_kernel<128><<<grid, kThreads, 0, stream>>>(a);
  return launch_status();
}

}  // namespace pluto_hip
