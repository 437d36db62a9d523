// Key-owned half of the causal attention backward for bf16 heads of 64
// channels: dK^T[d, key] = sum_q Q^T[d, q] dS[q, key], dV^T[d, key] = sum_q
// dO^T[d, q] P[q, key] (src/llm/layers/attention.cc:293-396, the key side of
// bwd_impl's loops), with the main loop as a hand-scheduled instruction stream
// (gen_flash_dkv_loop.py describes the schedule).
//
// Same arithmetic and the same reduction order over queries as
// flash_dkv_kernel<64> (flash_bwd_mfma.hip): the score accumulator starts from
// -lse / scale and the dP accumulator from -delta, both left in the workspace
// by the query-owned kernel; P, dS and dO enter the matrix products as bf16.
//
// A workgroup of two waves owns 128 keys, a wave 64 of them as two halves of
// 32 (lane = key).  Query blocks of 32 rows stream through a ring of LDS
// stages; the waves walk them in ascending order.  One wave a SIMD: 256
// vector registers and 192 accumulator registers.
#include "flash_bwd_mfma.h"

#include "flash_dkv_loop.inc"
#include "mfma_tile.h"

namespace pluto_hip {
namespace {

constexpr int kWideThreads = 128;
constexpr int kRing = FLASH_DKV_D64_RING;
constexpr int kStageBytes = FLASH_DKV_D64_STAGE_BYTES;
constexpr int kTileBytes = FLASH_DKV_D64_TILE_BYTES;

__global__ void __launch_bounds__(kWideThreads) __attribute__((amdgpu_waves_per_eu(1, 1)))
flash_dkv_wide_kernel(GenericBackwardArgs a, const float* __restrict__ lse2,
                      const uint16_t* __restrict__ d_out_bf16) {
  constexpr int D = 64, BNK = 128, KS = D / 16, DB = D / 32;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[kRing * kStageBytes];
  static_assert(kTileBytes == 32 * D * 2);

  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int T = a.context_length, H = a.num_heads, E = a.embedding_dim;
  const int key_tiles = (T + BNK - 1) / BNK;
  // one tile per workgroup, the tiles that see the most queries first; a
  // (sequence, head) unit keeps its XCD across tiles whenever the number of
  // units is a multiple of 8
  const int units = gridDim.x / key_tiles;
  const int key_tile = blockIdx.x / units;
  const int head = (blockIdx.x % units) % H, seq = (blockIdx.x % units) / H;
  const long long seq_row0 = static_cast<long long>(seq) * T;
  const long long stats_base = (static_cast<long long>(seq) * H + head) * T;
  const uint16_t* qkv = static_cast<const uint16_t*>(a.qkv);
  const uint16_t* q_base = qkv + seq_row0 * 3 * E + head * D;
  const uint16_t* k_base = q_base + E;
  const uint16_t* v_base = q_base + 2 * E;
  const uint16_t* g_base = d_out_bf16 + seq_row0 * E + head * D;
  const int k0 = key_tile * BNK;
  const int first_block = k0 / 32;                       // query blocks first_block .. last_block
  const int steps = (T - 1) / 32 - first_block + 1;      // see some key of this tile
  const int wave_first_key = k0 + 64 * wave;

  // K and V of the wave's keys as B operands
  bf16x8 kf[2][KS], vf[2][KS];
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int key_load = min(wave_first_key + 32 * c + n, T - 1);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[c][ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
          k_base + static_cast<long long>(key_load) * 3 * E + 16 * ks + 8 * h));
      vf[c][ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
          v_base + static_cast<long long>(key_load) * 3 * E + 16 * ks + 8 * h));
    }
  }

  // What the loop statement takes.  Requests: chunk (2 wave + i) 64 + lane of a
  // tile of 32 rows; the second of a pair lands 1024 bytes further on in LDS
  // through the instruction's offset, which also moves its global address:
  // taken out of the lane's offset again.  Statistics: one float a lane of the
  // lower half, wave 0 the scaled log-sum-exp, wave 1 minus delta; the upper
  // half asks beyond the descriptor and gets zeros.
  const int row_read[KS] = {tile_row_read<D>(n, 0 + h), tile_row_read<D>(n, 2 + h),
                            tile_row_read<D>(n, 4 + h), tile_row_read<D>(n, 6 + h)};
  const int tr_read[DB] = {tile_transpose_read<D>(lane, 0), tile_transpose_read<D>(lane, 1)};
  const int stat_read = 2 * kTileBytes + 16 * h;
  const uint32_t q_fill0 = tile_fill_offset<D>((wave * 2 + 0) * 64 + lane, 3LL * E);
  const uint32_t q_fill1 = tile_fill_offset<D>((wave * 2 + 1) * 64 + lane, 3LL * E) - 1024u;
  const uint32_t g_fill0 = tile_fill_offset<D>((wave * 2 + 0) * 64 + lane, 1LL * E);
  const uint32_t g_fill1 = tile_fill_offset<D>((wave * 2 + 1) * 64 + lane, 1LL * E) - 1024u;
  const uint32_t s_fill = lane < 32 ? lane * 4u : 0x40000000u;
  const int rows_left = T - 1 - 32 * first_block;  // >= 0
  const int32x4 q_rsrc = make_rsrc(q_base + static_cast<long long>(32 * first_block) * 3 * E,
                                   static_cast<uint32_t>((static_cast<long long>(rows_left) * 3 * E + D) * 2));
  const int32x4 g_rsrc = make_rsrc(g_base + static_cast<long long>(32 * first_block) * E,
                                   static_cast<uint32_t>((static_cast<long long>(rows_left) * E + D) * 2));
  const float* stat_source = (wave == 0 ? lse2 : a.deltas) + stats_base + 32 * first_block;
  const int32x4 s_rsrc = make_rsrc(stat_source, static_cast<uint32_t>(rows_left + 1) * 4u);
  const uint32_t lds_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void*)lds));
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(lds_address);
  const uint32_t lds_q = __builtin_amdgcn_readfirstlane(lds_address + wave * 2048);
  const uint32_t lds_s = __builtin_amdgcn_readfirstlane(lds_address + 2 * kTileBytes + wave * 256);
  const uint32_t q_step = static_cast<uint32_t>(32LL * 3 * E * 2), g_step = static_cast<uint32_t>(32LL * E * 2);
  const float scale2 = a.scale * kLog2e;
  const uint32_t scale2_bits = __builtin_amdgcn_readfirstlane(__float_as_uint(scale2));
  // a wave's blocks start two steps after the workgroup's per 64 keys of offset
  const int wave_blocks_signed = steps - 2 * wave;
  const uint32_t wave_blocks =
      __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(wave_blocks_signed > 0 ? wave_blocks_signed : 0));
  uint32_t idle_steps = __builtin_amdgcn_readfirstlane(
      wave_blocks > 0 ? static_cast<uint32_t>(2 * wave) : static_cast<uint32_t>(steps + 1));
  // query 32 b + 8 (i / 4) + 4 h + i % 4 of the wave's block b, key n of half c:
  // hidden where the query precedes the key or lies beyond the sequence
  const int first_bound = n - 4 * h;
  const int last_bound = T - 1 - wave_first_key - 4 * h;
  uint32_t q_offset = 0, g_offset = 0, s_offset = 0, steps_done = 0, block_count = 0;
  uint32_t saved_m0, temp0, temp1;
  unsigned long long mask_pair;
  floatx16 dk[2][DB], dv[2][DB];
  asm volatile(FLASH_DKV_D64_ASM
               : FLASH_DKV_D64_DK00(dk[0][0]), FLASH_DKV_D64_DK01(dk[0][1]),
                 FLASH_DKV_D64_DK10(dk[1][0]), FLASH_DKV_D64_DK11(dk[1][1]),
                 FLASH_DKV_D64_DV00(dv[0][0]), FLASH_DKV_D64_DV01(dv[0][1]),
                 FLASH_DKV_D64_DV10(dv[1][0]), FLASH_DKV_D64_DV11(dv[1][1]),
                 FLASH_DKV_D64_K00(kf[0][0]), FLASH_DKV_D64_K01(kf[0][1]),
                 FLASH_DKV_D64_K02(kf[0][2]), FLASH_DKV_D64_K03(kf[0][3]),
                 FLASH_DKV_D64_K10(kf[1][0]), FLASH_DKV_D64_K11(kf[1][1]),
                 FLASH_DKV_D64_K12(kf[1][2]), FLASH_DKV_D64_K13(kf[1][3]),
                 FLASH_DKV_D64_V00(vf[0][0]), FLASH_DKV_D64_V01(vf[0][1]),
                 FLASH_DKV_D64_V02(vf[0][2]), FLASH_DKV_D64_V03(vf[0][3]),
                 FLASH_DKV_D64_V10(vf[1][0]), FLASH_DKV_D64_V11(vf[1][1]),
                 FLASH_DKV_D64_V12(vf[1][2]), FLASH_DKV_D64_V13(vf[1][3]),
                 [qoff] "+&s"(q_offset), [goff] "+&s"(g_offset), [soff] "+&s"(s_offset),
                 [tcount] "+&s"(steps_done), [idle] "+&s"(idle_steps), [bcount] "+&s"(block_count),
                 [m0save] "=&s"(saved_m0), [t0] "=&s"(temp0), [t1] "=&s"(temp1),
                 [mpair] "=&s"(mask_pair)
               : FLASH_DKV_D64_ROWADDR0(row_read[0]), FLASH_DKV_D64_ROWADDR1(row_read[1]),
                 FLASH_DKV_D64_ROWADDR2(row_read[2]), FLASH_DKV_D64_ROWADDR3(row_read[3]),
                 FLASH_DKV_D64_TRADDR0(tr_read[0]), FLASH_DKV_D64_TRADDR1(tr_read[1]),
                 FLASH_DKV_D64_STATADDR(stat_read),
                 FLASH_DKV_D64_QFILL0(q_fill0), FLASH_DKV_D64_QFILL1(q_fill1),
                 FLASH_DKV_D64_GFILL0(g_fill0), FLASH_DKV_D64_GFILL1(g_fill1),
                 FLASH_DKV_D64_SFILL(s_fill), FLASH_DKV_D64_N4(first_bound),
                 FLASH_DKV_D64_TL4(last_bound),
                 [qrsrc] "s"(q_rsrc), [grsrc] "s"(g_rsrc), [srsrc] "s"(s_rsrc),
                 [scale2] "s"(scale2_bits), [qstep] "s"(q_step), [gstep] "s"(g_step),
                 [ldsbase] "s"(lds_base), [ldsq] "s"(lds_q), [ldss] "s"(lds_s),
                 [nblk] "s"(wave_blocks)
               : FLASH_DKV_D64_CLOBBERS);

  // dK and dV leave through LDS so that every store instruction writes whole
  // rows (16 lanes x 16 bytes): written straight from the accumulators, a
  // lane's 16-byte pieces lie 9 KiB apart and each store touches 32 lines.
  // One tensor and half at a time, 32 keys x 64 floats a wave, pieces swizzled
  // by row.  The loop statement ends with a barrier behind every LDS access.
  {
    static_assert(2 * 32 * 64 * 4 <= kRing * kStageBytes, "the ring holds one step of the workgroup");
    constexpr int kPieces = 16;  // 16-byte pieces in 64 columns
    float4* area = reinterpret_cast<float4*>(lds) + wave * 32 * kPieces;
    const int out_piece = lane % kPieces, out_row = lane / kPieces;
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      const int tensor = step / 2, c = step % 2;
#pragma unroll
      for (int d2 = 0; d2 < 2; ++d2)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const floatx16& acc = tensor == 0 ? dk[c][d2] : dv[c][d2];
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
      const int key0 = wave_first_key + 32 * c;
      float* dst = a.d_qkv + (seq_row0 + key0) * 3 * E + (1 + tensor) * E + head * D;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int row = 4 * i + out_row;
        const float4 value = area[row * kPieces + (out_piece ^ (row % kPieces))];
        if (key0 + row < T)
          *reinterpret_cast<float4*>(dst + static_cast<long long>(row) * 3 * E + 4 * out_piece) = value;
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // before the area is overwritten
    }
  }
}

}  // namespace

int launch_flash_dkv_wide(hipStream_t stream, const GenericBackwardArgs& a, const float* lse2,
                          const uint16_t* d_out_bf16) {
  const long long tiles = (a.context_length + 127) / 128;
  const long long units = 1LL * a.num_heads * (a.rows / a.context_length);
  if (tiles * units > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  flash_dkv_wide_kernel<<<dim3(static_cast<unsigned>(tiles * units)), kWideThreads, 0, stream>>>(
      a, lse2, d_out_bf16);
  return launch_status();
}

}  // namespace pluto_hip
