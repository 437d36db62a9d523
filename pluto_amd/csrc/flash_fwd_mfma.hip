// Causal flash attention forward for bf16 activations on gfx950 matrix cores.
//
// A workgroup of WAVES wave64 owns BM = 32*G*WAVES query rows of one
// (sequence, head); a wave owns G groups of 32 consecutive rows.  Key/value
// tiles of 64 rows are double-buffered in LDS, both row major, and are filled
// by buffer loads that write LDS directly (no VGPR round trip, out-of-range
// rows read as zero).  Both products are computed transposed with
// v_mfma_f32_32x32x16_bf16:
//
//   S^T[key, query] = K[key, :] . Q[query, :]      A = K (LDS), B = Q (regs)
//   O^T[d,   query] = V^T[d, key] . P^T[key, query] A = V^T (LDS), B = P^T
//
// In the 32x32 accumulator layout lane l holds column (l % 32), i.e. ONE query,
// so the softmax row statistics are per-lane scalars and need a single
// exchange between the two lane halves per block, and the probabilities leave
// the accumulator registers already laid out as the B operand of the second
// product: no shuffle, no LDS round trip.  The contraction index of an MFMA
// may be enumerated in any order as long as A and B agree, so the V^T operand
// gathers its keys in the order in which the accumulator registers hold them;
// the gather itself is done by the LDS transpose read (ds_read_b64_tr_b16),
// which hands each lane four keys of one channel from a row-major tile.
//
// Semantics follow FlashAttentionForwardKernel (src/llm/layers/attention.cc:
// 98-170) and, with the gate epilogue, ForwardKernel
// (src/llm/layers/qwen_attention.cc:68-119).  Deviation, within the stated
// bf16 tolerance: probabilities are rounded to bf16 for the P.V product (the
// reference keeps them FP32, attention.cc:151-156).
#include "flash_fwd_mfma.h"

#include "mfma_tile.h"

#include <algorithm>

namespace pluto_hip {
namespace {

constexpr int BN = 64;  // keys per LDS tile
// measured on both head widths: level with the four-wave kernel at 2048 rows,
// 10-15 % ahead from 4096, behind it at 1024 (few, short tiles per workgroup)
constexpr int kPipelinedFromRows = 2048;
constexpr int kPipelined256FromRows = 256;

// Queues the loads of one K tile and one V tile (keys k0..k0+63) into an LDS
// stage.  Lane l of load i of a wave writes 16 bytes at chunk
// (wave*LOADS + i)*64 + l of the tile; k_fill/v_fill say which global bytes it
// fetches.  Rows at or beyond kv_rows read as zero.
template <int D, int LOADS>
__device__ inline void fill_stage(unsigned char* stage, int wave, const uint16_t* k_base,
                                  const uint16_t* v_base, long long k_row_stride,
                                  long long v_row_stride, int k0, int kv_rows,
                                  const uint32_t* k_fill, const uint32_t* v_fill) {
  constexpr int kTileBytes = BN * D * 2;
  const long long rows_left = kv_rows - 1 - k0;
  const int32x4 k_rsrc =
      make_rsrc(k_base + static_cast<long long>(k0) * k_row_stride,
                static_cast<uint32_t>((rows_left * k_row_stride + D) * 2));
  const int32x4 v_rsrc =
      make_rsrc(v_base + static_cast<long long>(k0) * v_row_stride,
                static_cast<uint32_t>((rows_left * v_row_stride + D) * 2));
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int at = (wave * LOADS + i) * 1024;
    lds_fill<16>(k_rsrc, stage + at, k_fill[i]);
    lds_fill<16>(v_rsrc, stage + kTileBytes + at, v_fill[i]);
  }
}

template <int D, int G, int WAVES>
struct Config {
  static constexpr int kThreads = 64 * WAVES;
  static constexpr int BM = 32 * G * WAVES;
  static constexpr int KCH = D / 8;                // 16-byte chunks per row
  static constexpr int kTileBytes = BN * D * 2;    // one K or V tile
  static constexpr int kStageBytes = 2 * kTileBytes;
  static constexpr int kLoads = BN * KCH / kThreads;  // 16-byte loads per lane per tensor
  // waves per SIMD the register budget is sized for
  static constexpr int kOccupancy = (D == 64 && G == 1) ? 3 : (D == 256 ? 1 : 2);
};

template <int D, int G, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
__attribute__((amdgpu_waves_per_eu(Config<D, G, WAVES>::kOccupancy,
                                   Config<D, G, WAVES>::kOccupancy)))
flash_forward_kernel(FlashForwardArgs a_in, int unit_count) {
  struct Args : FlashForwardArgs {
    int unit_count;
  } a;
  static_cast<FlashForwardArgs&>(a) = a_in;
  a.unit_count = unit_count;
  using C = Config<D, G, WAVES>;
  constexpr int KCH = C::KCH;
  constexpr int KS = D / 16;   // contraction steps of S^T
  constexpr int DB = D / 32;   // 32-row blocks of O^T
  constexpr int KB = BN / 32;  // 32-key blocks per tile
  constexpr int BM = C::BM;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * C::kStageBytes];

  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int q_tiles = (a.q_rows + BM - 1) / BM;
  const int pairs = (q_tiles + 1) / 2;
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.
  // Renumber them so that the workgroups sharing one (sequence, kv head) K/V
  // stream run on the same XCD.
  // Two schedules.  Paired (kPaired): a workgroup processes query tile
  // q_tiles-1-pair and then tile pair; under the causal mask every pair
  // carries the same work, which balances perfectly when all workgroups are
  // resident at once.  Unpaired: one tile per workgroup, heaviest tiles first,
  // for kernels whose resident workgroups are fewer than the grid (the greedy
  // dispatch of ever lighter tiles then fills the machine evenly).
  constexpr bool kPaired = D == 64;
  int pair, head, seq;
  if constexpr (kPaired) {
    const int logical = xcd_logical_block();
    pair = logical % pairs;
    head = (logical / pairs) % a.query_heads;
    seq = logical / (pairs * a.query_heads);
  } else {
    // The `group` query heads that share a (sequence, kv head) at one query
    // tile form a unit u; XCD x works on u = x, x + 8, ... in that order, so
    // the heads that stream the same K/V rows do so from the same L2 at the
    // same time.  u counts query tiles from the heaviest (last) down, kv heads
    // fastest; the grid is padded to a multiple of 8 units.
    const int kv_heads = a.query_heads / a.group;
    const int kv_units = a.unit_count / q_tiles;  // (sequence, kv head) pairs
    const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
    const int u = 8 * (slot / a.group) + xcd;
    if (u >= a.unit_count) return;
    pair = q_tiles - 1 - u / kv_units;
    const int kv_unit = u % kv_units;
    head = (kv_unit % kv_heads) * a.group + slot % a.group;
    seq = kv_unit / kv_heads;
  }
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

  // ---- loop-invariant lane addresses ---------------------------------------
  // Tile fill: load i of this lane lands at LDS chunk p = (wave*kLoads+i)*64 +
  // lane of the tile (the hardware writes lane l at base + 16 l); which global
  // chunk it fetches is chosen so that the tile ends up swizzled:
  //   K: chunk c of row r at r*KCH + (c ^ (r & 7))        (16-byte row reads)
  //   V: chunk c of row r at r*KCH + (c ^ (2 * (r & 3)))  (transpose reads)
  uint32_t k_fill[C::kLoads], v_fill[C::kLoads];
#pragma unroll
  for (int i = 0; i < C::kLoads; ++i) {
    const int p = (wave * C::kLoads + i) * 64 + lane;
    const int row = p / KCH, slot = p % KCH;
    k_fill[i] = static_cast<uint32_t>(row * a.k_row_stride * 2 + (slot ^ (row & 7)) * 16);
    v_fill[i] = static_cast<uint32_t>(row * a.v_row_stride * 2 + (slot ^ (2 * (row & 3))) * 16);
  }
  // K operand of key block kb, step ks: row 32kb + n, chunk 2ks + h.
  int k_read[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_read[ks] = (n * KCH + ((2 * ks + h) ^ (n & 7))) * 16;
  // V^T operand: the 16 lanes of group gq = lane/16 receive channels
  // 32db + 16(gq%2) + (lane%16) and keys 4(gq/2) + (0..3) of the addressed
  // rows; as a source, lane (kk = (lane%16)/4, b = lane%4) supplies row kk,
  // channels 4b..4b+3 of that 16-channel span.
  int v_read[DB];
  {
    const int gq = lane / 16, kk = (lane % 16) / 4, b = lane % 4;
    const int row = 4 * (gq / 2) + kk;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int chunk = 4 * db + 2 * (gq % 2) + b / 2;
      v_read[db] = (row * KCH + (chunk ^ (2 * kk))) * 16 + (b % 2) * 8;
    }
  }

  // A workgroup processes query tile (q_tiles-1-pair) and then tile `pair`:
  // under the causal mask their key counts add up to the same total for every
  // pair, so all workgroups carry equal work.
  for (int pass = 0; pass < 2; ++pass) {
    const int q_tile = (kPaired && pass == 0) ? q_tiles - 1 - pair : pair;
    if (pass == 1 && (!kPaired || q_tile == q_tiles - 1 - pair)) break;
    const int q0 = q_tile * BM;
    const int wave_q0 = q0 + 32 * G * wave;

    // Q fragments (B operand of S^T): row, channels 16ks + 8h .. +7.
    bf16x8 qf[G][KS];
    int q_row[G], row_limit[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      q_row[g] = wave_q0 + 32 * g + n;
      const int row = min(q_row[g], a.q_rows - 1);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qf[g][ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
            q_base + static_cast<long long>(row) * a.q_row_stride + 16 * ks + 8 * h));
      // keys up to row_limit are visible to this lane's query
      row_limit[g] = min(a.start_position + q_row[g], a.kv_rows - 1);
    }
    floatx16 o_acc[G][DB];
    // Row sums come out of the matrix cores: an all-ones A operand makes every
    // row of this accumulator the sum over keys of the bf16 probabilities.
    floatx16 l_acc[G];
    // Online softmax in the log2 domain with a lazily updated reference
    // point: probabilities are 2^(s*scale2 - m_used); m_used follows the
    // running row maximum only when that has grown by more than kLazy, so the
    // accumulator rescale is rare.  The true maximum is tracked separately and
    // the saved statistics are converted to it at the end.
    constexpr float kLazy = 8.0f;
    float m_used[G], m_true[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      m_used[g] = kMasked;
      m_true[g] = kMasked;
#pragma unroll
      for (int i = 0; i < 16; ++i) l_acc[g][i] = 0.0f;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[g][db][i] = 0.0f;
    }

    const int last_row = min(q0 + BM, a.q_rows) - 1;
    const int visible = min(a.kv_rows, a.start_position + last_row + 1);
    const int tiles = (visible + BN - 1) / BN;

    if (tiles > 0)
      fill_stage<D, C::kLoads>(lds + (0 & 1) * C::kStageBytes, wave, k_base, v_base,
                                 a.k_row_stride, a.v_row_stride, (0) * BN, a.kv_rows, k_fill,
                                 v_fill);
    for (int tile = 0; tile < tiles; ++tile) {
      const int k0 = tile * BN;
      // The tile's loads have landed; every wave is done with the other stage.
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
      if (tile + 1 < tiles)
        fill_stage<D, C::kLoads>(lds + ((tile + 1) & 1) * C::kStageBytes, wave, k_base, v_base,
                                 a.k_row_stride, a.v_row_stride, (tile + 1) * BN, a.kv_rows, k_fill,
                                 v_fill);
      const unsigned char* k_tile = lds + (tile & 1) * C::kStageBytes;
      const unsigned char* v_tile = k_tile + C::kTileBytes;
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const int kb0 = k0 + 32 * kb;
        // nothing of this block is visible to any of the wave's rows
        if (kb0 > a.start_position + wave_q0 + 32 * G - 1) continue;
        // ---- S^T = K Q^T for 32 keys ------------------------------------
        bf16x8 kf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          kf[ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
              k_tile + k_read[ks] + kb * 32 * KCH * 16));
        // V^T operands of this block are requested now, so that their LDS
        // latency passes under the first product and the softmax
        bf16x8 vf[2][DB];
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            // keys 16 s2 + 4h + (0..3), then 16 s2 + 8 + 4h + (0..3)
            const int at = v_read[db] + (32 * kb + 16 * s2) * KCH * 16;
            const uint2 lo = lds_transpose_read(v_tile, at);
            const uint2 hi = lds_transpose_read(v_tile, at + 8 * KCH * 16);
            vf[s2][db] = __builtin_bit_cast(bf16x8, make_uint4(lo.x, lo.y, hi.x, hi.y));
          }
        __builtin_amdgcn_sched_barrier(0);
        floatx16 s[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
          for (int i = 0; i < 16; ++i) s[g][i] = 0.0f;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) s[g] = mfma32(kf[ks], qf[g][ks], s[g]);
        }
        bf16x8 pf[G][2];
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int group_q0 = a.start_position + wave_q0 + 32 * g;
          // ---- mask (diagonal and tail blocks only), row maximum ----------
          if (kb0 + 31 > group_q0 || kb0 + 32 > a.kv_rows) {
            const int limit = row_limit[g] - kb0 - 4 * h;
#pragma unroll
            for (int i = 0; i < 16; ++i)
              s[g][i] = (8 * (i / 4) + (i % 4) > limit) ? kMasked : s[g][i];
          }
          float row_max = fmaxf(fmaxf(s[g][0], s[g][1]), s[g][2]);
#pragma unroll
          for (int i = 3; i < 15; i += 2) row_max = fmaxf(fmaxf(row_max, s[g][i]), s[g][i + 1]);
          row_max = fmaxf(row_max, s[g][15]);
          m_true[g] = fmaxf(m_true[g], half_swap_max(row_max));
          const float candidate = m_true[g] * scale2;
          if (__any(candidate > m_used[g] + kLazy)) {
            const float m_new = candidate > m_used[g] + kLazy ? candidate : m_used[g];
            const float alpha = __builtin_amdgcn_exp2f(m_used[g] - m_new);
            m_used[g] = m_new;
            l_acc[g][0] *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
              for (int i = 0; i < 16; ++i) o_acc[g][db][i] *= alpha;
          }
          // ---- P^T = 2^(S^T scale2 - m_used) as bf16 B operands -----------
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            uint32_t packed[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              packed[e] = pack_bf16(
                  __builtin_amdgcn_exp2f(__builtin_fmaf(s[g][8 * s2 + 2 * e], scale2, -m_used[g])),
                  __builtin_amdgcn_exp2f(
                      __builtin_fmaf(s[g][8 * s2 + 2 * e + 1], scale2, -m_used[g])));
            pf[g][s2] = __builtin_bit_cast(
                bf16x8, make_uint4(packed[0], packed[1], packed[2], packed[3]));
          }
        }
        // ---- O^T += V^T P^T; l += 1^T P^T ----------------------------------
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
          for (int g = 0; g < G; ++g) {
            l_acc[g] = mfma32(ones, pf[g][s2], l_acc[g]);
#pragma unroll
            for (int db = 0; db < DB; ++db)
              o_acc[g][db] = mfma32(vf[s2][db], pf[g][s2], o_acc[g][db]);
          }
        }
      }
    }

    // ---- epilogue ----------------------------------------------------------
    // A lane owns, for its query, channels 32db + 8j + 4h .. +3: four bf16 =
    // one 8-byte store; the eight stores of a lane pair cover the row's bytes.
#pragma unroll
    for (int g = 0; g < G; ++g) {
      // l_acc holds the sum over all keys (both lane halves contract into the
      // same accumulator column).
      const float l_used = l_acc[g][0] > 0.0f ? l_acc[g][0] : 1.0f;
      const float inverse = 1.0f / l_used;
      const int row = q_row[g];
      if (row < a.q_rows) {
        uint16_t* o_row = o_base + static_cast<long long>(row) * a.o_row_stride;
        uint16_t* core_row = a.core ? a.core + (o_row - a.out) : nullptr;
        const uint16_t* gate_row =
            gate_base ? gate_base + static_cast<long long>(row) * a.gate_row_stride : nullptr;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int d = 32 * db + 8 * j + 4 * h;
            float c[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) c[e] = o_acc[g][db][4 * j + e] * inverse;
            if (core_row) {
              uint2 plain;
              plain.x = pack_bf16(c[0], c[1]);
              plain.y = pack_bf16(c[2], c[3]);
              *reinterpret_cast<uint2*>(core_row + d) = plain;
            }
            if (gate_row) {
              // out = bf16(bf16(core) * bf16(sigmoid(gate))): qwen_attention.cc:103-108
              const uint2 gate_bits = *reinterpret_cast<const uint2*>(gate_row + d);
              const uint32_t gw[2] = {gate_bits.x, gate_bits.y};
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float logit = __uint_as_float(
                    (e & 1) ? (gw[e / 2] & 0xffff0000u) : (gw[e / 2] << 16));
                c[e] = round_to_bf16(c[e]) * round_to_bf16(gate_sigmoid(logit));
              }
            }
            uint2 packed;
            packed.x = pack_bf16(c[0], c[1]);
            packed.y = pack_bf16(c[2], c[3]);
            *reinterpret_cast<uint2*>(o_row + d) = packed;
          }
        if (h == 0) {
          // statistics relative to the true maximum: attention.cc:161-168
          const float normalizer =
              l_used * __builtin_amdgcn_exp2f(m_used[g] - m_true[g] * scale2);
          const float maximum = m_true[g] * a.scale;
          const long long stat =
              (static_cast<long long>(seq) * a.query_heads + head) * a.q_rows + row;
          if (a.maxima) a.maxima[stat] = maximum;
          if (a.normalizers) a.normalizers[stat] = normalizer;
          if (a.lse)
            a.lse[(static_cast<long long>(seq) * a.q_rows + row) * a.query_heads + head] =
                maximum + __logf(normalizer);
        }
      }
    }
    // the next pass refills stage 0 while slower waves may still read a stage
    __syncthreads();
  }
}

long long grid_blocks(const FlashForwardArgs& a, int block_rows, int sequences, bool paired) {
  const long long q_tiles = (a.q_rows + block_rows - 1) / block_rows;
  return (paired ? (q_tiles + 1) / 2 : q_tiles) * a.query_heads * sequences;
}

}  // namespace

bool flash_forward_supported(const FlashForwardArgs& a, int head_dim) {
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return false;
  auto aligned = [](const void* p) {
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
  };
  auto mult8 = [](long long s) { return (s % 8) == 0; };
  if (!aligned(a.q) || !aligned(a.k) || !aligned(a.v) || !aligned(a.out))
    return false;
  if (a.gate && !aligned(a.gate)) return false;
  // K and V of one (sequence, head) are addressed through 32-bit buffer offsets
  const long long limit = 1LL << 31;
  if (a.kv_rows * a.k_row_stride * 2 >= limit || a.kv_rows * a.v_row_stride * 2 >= limit)
    return false;
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
  long long blocks = grid_blocks(a, 128, sequences, head_dim == 64);
  // unpaired schedule: units of `group` heads, dealt to the 8 XCDs
  const long long q_tiles = (a.q_rows + 127) / 128;
  const long long units = q_tiles * sequences * (a.query_heads / a.group);
  if (head_dim != 64) blocks = (units + 7) / 8 * 8 * a.group;
  if (blocks <= 0 || blocks > 0x7fffffffLL || units > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  const dim3 grid(static_cast<unsigned>(blocks));
  const int unit_count = static_cast<int>(units);
  if (!kernel_enabled(kMainKernel)) return 0;
  // Long sequences take the kernel with the hand-scheduled loop
  // (flash_fwd_pipelined.hip): tiles of 256 rows (128 at head widths 64 and
  // 256), which short sequences do not fill.  Its epilogue addresses a head's rows through
  // 32-bit buffer offsets.
  // (a test lifts the threshold at head width 256 to compare the two kernels on small shapes)
  const int from_rows = head_dim != 256 ? kPipelinedFromRows
                        : kernel_enabled(kFromLength) ? kPipelined256FromRows : 1;
  if (a.q_rows >= from_rows && kernel_enabled(kEightWave)) {
    const long long widest = a.gate ? std::max(a.o_row_stride, a.gate_row_stride) : a.o_row_stride;
    if (a.q_rows * widest * 2 < (1LL << 31) - 4096)
      return launch_flash_forward_pipelined(stream, a, head_dim, sequences);
  }
  if (head_dim == 256)
    flash_forward_kernel<256, 1, 4><<<grid, 256, 0, stream>>>(a, unit_count);
  else if (head_dim == 128)
    flash_forward_kernel<128, 1, 4><<<grid, 256, 0, stream>>>(a, unit_count);
  else
    flash_forward_kernel<64, 1, 4><<<grid, 256, 0, stream>>>(a, unit_count);
  return launch_status();
}

}  // namespace pluto_hip
