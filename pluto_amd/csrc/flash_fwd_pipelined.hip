// Causal flash attention forward for bf16 sequences on gfx950: the kernel
// whose main loop is a hand-scheduled instruction stream.
//
// Same mathematics, operand layouts and results as flash_forward_kernel
// (flash_fwd_mfma.hip; semantics of FlashAttentionForwardKernel,
// src/llm/layers/attention.cc:98-170, and with the gate epilogue of
// ForwardKernel, src/llm/layers/qwen_attention.cc:68-119).  What differs is who
// orders the instructions.  A wave owns 32 query rows; all the key blocks it
// sees, the ones the causal mask or the end of the keys cuts included, are
// processed by ONE asm statement (flash_fwd_loop.inc for head widths 64 and
// 128, flash_fwd_loop256.inc for 256, written by gen_flash_fwd_loop*.py): per
// 32-key block a wave issues the S^T products of the next block, the softmax
// arithmetic of the current one and the O^T products of the previous one
// interleaved instruction by instruction, with its own LDS reads, waits and
// global->LDS requests, on fixed registers.  Around the statement this file
// loads Q, writes the output (through LDS, whole rows) and the row statistics,
// and walks the list of tiles the launcher packed for the workgroup.
#include "flash_fwd_mfma.h"
#include "flash_fwd_loop.inc"
#include "flash_fwd_loop256.inc"
#include "mfma_tile.h"

#include <algorithm>
#include <vector>

namespace pluto_hip {
namespace {

constexpr int BN = 64;

// Which query tiles a workgroup processes.  The causal mask makes tiles
// unequal (tile t costs about t + 1 units plus a fixed part) and a long
// sequence yields only a few tiles per compute unit, so handing tiles out in
// launch order leaves compute units idle at the end (measured at 8192 rows, 24
// heads: 12 % of the kernel).  Instead the launcher packs the tiles into one
// list per workgroup, equal in cost, and launches one workgroup a compute
// unit; the lists travel in the kernel arguments.  slots == 0: no lists,
// workgroup i processes the single tile the XCD-aware numbering gives it.
constexpr int kScheduleEntries = 1536;
constexpr uint16_t kNoItem = 0xffff;
struct Schedule {
  int slots = 0;  // entries per workgroup; its list ends at kNoItem or after `slots`
  uint16_t item[kScheduleEntries];  // (sequence * heads + head) * q_tiles + q_tile
};

// Head width 128: eight waves, 256 query rows and 128 KiB of key/value stages
// a workgroup, one workgroup a compute unit.  Head width 64: four waves, 128
// rows, 64 KiB, two workgroups a compute unit, so that one computes while the
// other waits for its first tiles or writes its output (at 1024 rows a tile's
// loop is short against those).
// Head width 256: four waves, 128 rows, one wave a SIMD (448 registers: O^T and
// Q^T in AGPRs), 128 KiB of stages that hold single blocks of 32 keys, one
// workgroup a compute unit.
template <int D>
constexpr int kWaves = D == 256 ? FLASH_LOOP_D256_WAVES
                                : (D == 128 ? FLASH_LOOP_D128_WAVES : FLASH_LOOP_D64_WAVES);

template <int D>
__global__ void __launch_bounds__(64 * kWaves<D>)
__attribute__((amdgpu_waves_per_eu(D == 256 ? 1 : 2, D == 256 ? 1 : 2)))
flash_forward_pipelined_kernel(FlashForwardArgs a_in, int unit_count, Schedule schedule) {
  struct Args : FlashForwardArgs {
    int unit_count;
  } a;
  static_cast<FlashForwardArgs&>(a) = a_in;
  a.unit_count = unit_count;
  constexpr int WAVES = kWaves<D>, KCH = D / 8, KS = D / 16, DB = D / 32;
  constexpr int BM = 32 * WAVES;
  // keys of a K or V tile in an LDS stage: a tile of 64 at the narrower widths, one block at 256
  constexpr int kTileKeys = D == 256 ? 32 : BN;
  constexpr int kTileBytes = kTileKeys * D * 2, kStageBytes = 2 * kTileBytes, kStages = 4;
  constexpr int kLoads = kTileKeys * KCH / (64 * WAVES);
  static_assert(D == 256 || D == 128 || D == 64, "the loop text is instantiated for these head widths");
  static_assert(D == 256 ? (kLoads == FLASH_LOOP_D256_LOADS && kStageBytes == FLASH_LOOP_D256_STAGE_BYTES)
                : D == 128 ? (kLoads == FLASH_LOOP_D128_LOADS && kStageBytes == FLASH_LOOP_D128_STAGE_BYTES)
                           : (kLoads == FLASH_LOOP_D64_LOADS && kStageBytes == FLASH_LOOP_D64_STAGE_BYTES));
  __shared__ __attribute__((aligned(1024))) unsigned char lds[kStages * kStageBytes];

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int q_tiles = (a.q_rows + BM - 1) / BM;
  const int list_length = schedule.slots > 0 ? schedule.slots : 1;
  for (int entry = 0; entry < list_length; ++entry) {
  int q_tile, head, seq;
  if (schedule.slots > 0) {
    const int item = schedule.item[blockIdx.x * schedule.slots + entry];
    if (item == kNoItem) break;
    q_tile = item % q_tiles;
    const int column = item / q_tiles;
    head = column % a.query_heads;
    seq = column / a.query_heads;
  } else {
    // The query heads of a kv head at one query tile run on one XCD (workgroup
    // i lands on XCD i mod 8, each with a private L2), heaviest tiles first.
    const int kv_heads = a.query_heads / a.group;
    const int kv_units = a.unit_count / q_tiles;
    const int xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
    const int u = 8 * (slot / a.group) + xcd;
    if (u >= a.unit_count) return;  // the whole workgroup
    q_tile = q_tiles - 1 - u / kv_units;
    const int kv_unit = u % kv_units;
    head = (kv_unit % kv_heads) * a.group + slot % a.group;
    seq = kv_unit / kv_heads;
  }
  const int kv_head = head / a.group;
  const uint16_t* q_base = a.q + seq * a.q_seq_stride + head * a.q_head_stride;
  const uint16_t* k_base = a.k + seq * a.k_seq_stride + kv_head * a.k_head_stride;
  const uint16_t* v_base = a.v + seq * a.v_seq_stride + kv_head * a.v_head_stride;
  const float scale2 = a.scale * kLog2e;
  // the loop statement takes the factor as a scalar operand
  const uint32_t scale2_bits = __builtin_amdgcn_readfirstlane(__float_as_uint(scale2));
  bf16x8 ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = static_cast<__bf16>(1.0f);

  // lane addresses: the tile layouts of flash_forward_kernel
  uint32_t k_fill[kLoads], v_fill[kLoads];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const int p = (wave * kLoads + i) * 64 + lane;
    const int row = p / KCH, slot = p % KCH;
    k_fill[i] = static_cast<uint32_t>(row * a.k_row_stride * 2 + (slot ^ (row & 7)) * 16);
    v_fill[i] = static_cast<uint32_t>(row * a.v_row_stride * 2 + (slot ^ (2 * (row & 3))) * 16);
  }
  int k_read[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) k_read[ks] = (n * KCH + ((2 * ks + h) ^ (n & 7))) * 16;
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

  const int q0 = q_tile * BM;
  const int wave_q0 = q0 + 32 * wave;
  const int q_row = wave_q0 + n;
  bf16x8 qf[KS];
  {
    const int row = min(q_row, a.q_rows - 1);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      qf[ks] = as_bf16x8(*reinterpret_cast<const uint4*>(
          q_base + static_cast<long long>(row) * a.q_row_stride + 16 * ks + 8 * h));
  }
  const int row_limit = min(a.start_position + q_row, a.kv_rows - 1);
  floatx16 o_acc[DB], l_acc;
  constexpr float kLazy = 8.0f;
  float m_used = kMasked, m_true = kMasked;
#pragma unroll
  for (int i = 0; i < 16; ++i) l_acc[i] = 0.0f;
  if constexpr (D != 256) {  // at 256 the loop statement keeps O^T in AGPRs and hands it out at its end
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o_acc[db][i] = 0.0f;
  }

  // Blocks of 32 keys this wave walks: up to the last key its last row sees.  A
  // wave's last two blocks may be cut by the causal mask or by the end of the
  // keys; the loop statement masks those two and no others.
  const int32x4 k_all = make_rsrc(
      k_base, static_cast<uint32_t>(((a.kv_rows - 1) * a.k_row_stride + D) * 2));
  const int32x4 v_all = make_rsrc(
      v_base, static_cast<uint32_t>(((a.kv_rows - 1) * a.v_row_stride + D) * 2));
  const uint32_t lds_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void*)lds));
  auto blocks_of = [&](int first_row) {
    return min(a.start_position + first_row + 31, a.kv_rows - 1) / 32 + 1;
  };
  const uint32_t wave_blocks =
      __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(blocks_of(wave_q0)));
  // Every wave passes the same number of step barriers, the last wave's: a step
  // (two blocks) starts with one.
  const uint32_t total_steps = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(blocks_of(q0 + BM - 32)) / (D == 256 ? 1 : 2));
  {
    // ---- the hand-scheduled loop ----------------------------------------------------
    const uint32_t k_tile_step = static_cast<uint32_t>(BN * a.k_row_stride * 2);
    const uint32_t v_tile_step = static_cast<uint32_t>(BN * a.v_row_stride * 2);
    uint32_t iterations = __builtin_amdgcn_readfirstlane(wave_blocks > 3 ? wave_blocks - 3 : 0),
             flag = 0, k_offset = 0, v_offset = 0, steps_done = 0, v_block = 0,
             idle_steps = __builtin_amdgcn_readfirstlane(total_steps - wave_blocks / 2);
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(lds_address + wave * kLoads * 1024);
    uint32_t saved_m0, scalar_temp0, scalar_temp1;
    float threshold = m_used + kLazy;
    const int row_limit_lane = row_limit - 4 * h;
    if constexpr (D == 256) {
      // one step a block: the waves with fewer blocks idle for the difference
      uint32_t idle_256 = __builtin_amdgcn_readfirstlane(total_steps - wave_blocks), block_count = 0;
      uint32_t scalar_temp2;
      const uint32_t lds_base = __builtin_amdgcn_readfirstlane(lds_address);
      const uint32_t k_block_step = static_cast<uint32_t>(32 * a.k_row_stride * 2);
      const uint32_t v_block_step = static_cast<uint32_t>(32 * a.v_row_stride * 2);
      // load i of a lane lands 1024 i bytes further on in LDS through the
      // instruction's offset, which also moves its global address: taken out of
      // the lane's offset again
      const uint32_t k1 = k_fill[1] - 1024u, k2 = k_fill[2] - 2048u, k3 = k_fill[3] - 3072u;
      const uint32_t v1 = v_fill[1] - 1024u, v2 = v_fill[2] - 2048u, v3 = v_fill[3] - 3072u;
      asm volatile(FLASH_LOOP_D256_ASM
                   : FLASH_LOOP_D256_O0(o_acc[0]), FLASH_LOOP_D256_O1(o_acc[1]),
                     FLASH_LOOP_D256_O2(o_acc[2]), FLASH_LOOP_D256_O3(o_acc[3]),
                     FLASH_LOOP_D256_O4(o_acc[4]), FLASH_LOOP_D256_O5(o_acc[5]),
                     FLASH_LOOP_D256_O6(o_acc[6]), FLASH_LOOP_D256_O7(o_acc[7]),
                     FLASH_LOOP_D256_L(l_acc), FLASH_LOOP_D256_MUSED(m_used),
                     FLASH_LOOP_D256_MTRUE(m_true), FLASH_LOOP_D256_THR(threshold),
                     FLASH_LOOP_D256_QF0(qf[0]), FLASH_LOOP_D256_QF1(qf[1]),
                     FLASH_LOOP_D256_QF2(qf[2]), FLASH_LOOP_D256_QF3(qf[3]),
                     FLASH_LOOP_D256_QF4(qf[4]), FLASH_LOOP_D256_QF5(qf[5]),
                     FLASH_LOOP_D256_QF6(qf[6]), FLASH_LOOP_D256_QF7(qf[7]),
                     FLASH_LOOP_D256_QF8(qf[8]), FLASH_LOOP_D256_QF9(qf[9]),
                     FLASH_LOOP_D256_QF10(qf[10]), FLASH_LOOP_D256_QF11(qf[11]),
                     FLASH_LOOP_D256_QF12(qf[12]), FLASH_LOOP_D256_QF13(qf[13]),
                     FLASH_LOOP_D256_QF14(qf[14]), FLASH_LOOP_D256_QF15(qf[15]),
                     [iters] "+&s"(iterations), [flag] "+&s"(flag), [koff] "+&s"(k_offset),
                     [voff] "+&s"(v_offset), [tcount] "+&s"(steps_done), [bcount] "+&s"(block_count),
                     [idle] "+&s"(idle_256), [m0save] "=&s"(saved_m0), [t0] "=&s"(scalar_temp0),
                     [t1] "=&s"(scalar_temp1), [t2] "=&s"(scalar_temp2)
                   : FLASH_LOOP_D256_ONES(ones),
                     FLASH_LOOP_D256_KADDR0(k_read[0]), FLASH_LOOP_D256_KADDR1(k_read[1]),
                     FLASH_LOOP_D256_KADDR2(k_read[2]), FLASH_LOOP_D256_KADDR3(k_read[3]),
                     FLASH_LOOP_D256_VADDR0(v_read[0]), FLASH_LOOP_D256_VADDR1(v_read[1]),
                     FLASH_LOOP_D256_KFILL0(k_fill[0]), FLASH_LOOP_D256_KFILL1(k1),
                     FLASH_LOOP_D256_KFILL2(k2), FLASH_LOOP_D256_KFILL3(k3),
                     FLASH_LOOP_D256_VFILL0(v_fill[0]), FLASH_LOOP_D256_VFILL1(v1),
                     FLASH_LOOP_D256_VFILL2(v2), FLASH_LOOP_D256_VFILL3(v3),
                     FLASH_LOOP_D256_ROWLIM(row_limit_lane),
                     [krsrc] "s"(k_all), [vrsrc] "s"(v_all), [scale2] "s"(scale2_bits),
                     [kstep] "s"(k_block_step), [vstep] "s"(v_block_step), [ldsw] "s"(lds_wave),
                     [ldsbase] "s"(lds_base), [nblk] "s"(wave_blocks)
                   : FLASH_LOOP_D256_CLOBBERS);
    } else if constexpr (D == 128) {
      // the second load of a pair lands 1024 bytes further on in LDS through the
      // instruction's offset, which also moves its global address: taken out of
      // the lane's offset again
      const uint32_t k_second = k_fill[1] - 1024u, v_second = v_fill[1] - 1024u;
      const int k_read_high[KS] = {k_read[0] + 65536, k_read[1] + 65536, k_read[2] + 65536,
                                   k_read[3] + 65536, k_read[4] + 65536, k_read[5] + 65536,
                                   k_read[6] + 65536, k_read[7] + 65536};
      const int v_read_high[DB] = {v_read[0] + 65536, v_read[1] + 65536, v_read[2] + 65536,
                                   v_read[3] + 65536};
      asm volatile(FLASH_LOOP_D128_ASM
                   : FLASH_LOOP_D128_O0(o_acc[0]), FLASH_LOOP_D128_O1(o_acc[1]),
                     FLASH_LOOP_D128_O2(o_acc[2]), FLASH_LOOP_D128_O3(o_acc[3]),
                     FLASH_LOOP_D128_L(l_acc), FLASH_LOOP_D128_MUSED(m_used),
                     FLASH_LOOP_D128_MTRUE(m_true), FLASH_LOOP_D128_THR(threshold),
                     [iters] "+&s"(iterations), [flag] "+&s"(flag), [koff] "+&s"(k_offset),
                     [voff] "+&s"(v_offset), [tcount] "+&s"(steps_done), [vblk] "+&s"(v_block),
                     [idle] "+&s"(idle_steps), [m0save] "=&s"(saved_m0), [t0] "=&s"(scalar_temp0),
                     [t1] "=&s"(scalar_temp1)
                   : FLASH_LOOP_D128_QF0(qf[0]), FLASH_LOOP_D128_QF1(qf[1]),
                     FLASH_LOOP_D128_QF2(qf[2]), FLASH_LOOP_D128_QF3(qf[3]),
                     FLASH_LOOP_D128_QF4(qf[4]), FLASH_LOOP_D128_QF5(qf[5]),
                     FLASH_LOOP_D128_QF6(qf[6]), FLASH_LOOP_D128_QF7(qf[7]),
                     FLASH_LOOP_D128_ONES(ones),
                     FLASH_LOOP_D128_KADDR0_0(k_read[0]), FLASH_LOOP_D128_KADDR0_1(k_read[1]),
                     FLASH_LOOP_D128_KADDR0_2(k_read[2]), FLASH_LOOP_D128_KADDR0_3(k_read[3]),
                     FLASH_LOOP_D128_KADDR0_4(k_read[4]), FLASH_LOOP_D128_KADDR0_5(k_read[5]),
                     FLASH_LOOP_D128_KADDR0_6(k_read[6]), FLASH_LOOP_D128_KADDR0_7(k_read[7]),
                     FLASH_LOOP_D128_KADDR1_0(k_read_high[0]), FLASH_LOOP_D128_KADDR1_1(k_read_high[1]),
                     FLASH_LOOP_D128_KADDR1_2(k_read_high[2]), FLASH_LOOP_D128_KADDR1_3(k_read_high[3]),
                     FLASH_LOOP_D128_KADDR1_4(k_read_high[4]), FLASH_LOOP_D128_KADDR1_5(k_read_high[5]),
                     FLASH_LOOP_D128_KADDR1_6(k_read_high[6]), FLASH_LOOP_D128_KADDR1_7(k_read_high[7]),
                     FLASH_LOOP_D128_VADDR0_0(v_read[0]), FLASH_LOOP_D128_VADDR0_1(v_read[1]),
                     FLASH_LOOP_D128_VADDR0_2(v_read[2]), FLASH_LOOP_D128_VADDR0_3(v_read[3]),
                     FLASH_LOOP_D128_VADDR1_0(v_read_high[0]), FLASH_LOOP_D128_VADDR1_1(v_read_high[1]),
                     FLASH_LOOP_D128_VADDR1_2(v_read_high[2]), FLASH_LOOP_D128_VADDR1_3(v_read_high[3]),
                     FLASH_LOOP_D128_KFILL0(k_fill[0]), FLASH_LOOP_D128_KFILL1(k_second),
                     FLASH_LOOP_D128_VFILL0(v_fill[0]), FLASH_LOOP_D128_VFILL1(v_second),
                     FLASH_LOOP_D128_ROWLIM(row_limit_lane),
                     [krsrc] "s"(k_all), [vrsrc] "s"(v_all), [scale2] "s"(scale2_bits),
                     [kstep] "s"(k_tile_step), [vstep] "s"(v_tile_step), [ldsw] "s"(lds_wave),
                     [nblk] "s"(wave_blocks)
                   : FLASH_LOOP_D128_CLOBBERS);
    } else {
      // all four stages within reach of one base register per operand
      const uint32_t k_second = k_fill[1] - 1024u, v_second = v_fill[1] - 1024u;
      asm volatile(FLASH_LOOP_D64_ASM
                   : FLASH_LOOP_D64_O0(o_acc[0]), FLASH_LOOP_D64_O1(o_acc[1]),
                     FLASH_LOOP_D64_L(l_acc), FLASH_LOOP_D64_MUSED(m_used),
                     FLASH_LOOP_D64_MTRUE(m_true), FLASH_LOOP_D64_THR(threshold),
                     [iters] "+&s"(iterations), [flag] "+&s"(flag), [koff] "+&s"(k_offset),
                     [voff] "+&s"(v_offset), [tcount] "+&s"(steps_done), [vblk] "+&s"(v_block),
                     [idle] "+&s"(idle_steps), [m0save] "=&s"(saved_m0), [t0] "=&s"(scalar_temp0),
                     [t1] "=&s"(scalar_temp1)
                   : FLASH_LOOP_D64_QF0(qf[0]), FLASH_LOOP_D64_QF1(qf[1]),
                     FLASH_LOOP_D64_QF2(qf[2]), FLASH_LOOP_D64_QF3(qf[3]),
                     FLASH_LOOP_D64_ONES(ones),
                     FLASH_LOOP_D64_KADDR0_0(k_read[0]), FLASH_LOOP_D64_KADDR0_1(k_read[1]),
                     FLASH_LOOP_D64_KADDR0_2(k_read[2]), FLASH_LOOP_D64_KADDR0_3(k_read[3]),
                     FLASH_LOOP_D64_VADDR0_0(v_read[0]), FLASH_LOOP_D64_VADDR0_1(v_read[1]),
                     FLASH_LOOP_D64_KFILL0(k_fill[0]), FLASH_LOOP_D64_KFILL1(k_second),
                     FLASH_LOOP_D64_VFILL0(v_fill[0]), FLASH_LOOP_D64_VFILL1(v_second),
                     FLASH_LOOP_D64_ROWLIM(row_limit_lane),
                     [krsrc] "s"(k_all), [vrsrc] "s"(v_all), [scale2] "s"(scale2_bits),
                     [kstep] "s"(k_tile_step), [vstep] "s"(v_tile_step), [ldsw] "s"(lds_wave),
                     [nblk] "s"(wave_blocks)
                   : FLASH_LOOP_D64_CLOBBERS);
    }
  }
  // ---- epilogue ------------------------------------------------------------------
  // The arithmetic of flash_forward_kernel's epilogue.  Every access goes
  // through a bounds-checked buffer descriptor instead of a branch: rows past
  // the end (and, for the row statistics, the upper lane halves) get an
  // offset beyond the descriptor's range, which the hardware drops.  The
  // kernel thus never narrows exec, and nothing the register allocator spills
  // around the loop statement above can be saved under a partial mask.
  {
    constexpr uint32_t kDropped = 0x7fffffffu;  // beyond every descriptor below
    // The lane's LDS and row offsets below depend on the lane alone.  Computed
    // from an opaque copy of it they stay inside the loop over tiles: hoisted
    // out of it they would sit in spilled registers through the loop statement
    // and come back one dependent reload at a time.
    int lane_here = lane;
    asm volatile("" : "+v"(lane_here));
    const int h = lane_here / 32, n = lane_here % 32;
    const int q_row = wave_q0 + n;
    const bool in_range = q_row < a.q_rows;
    const long long row_bytes = static_cast<long long>(a.q_rows - 1) * a.o_row_stride * 2;
    uint16_t* o_base = a.out + seq * a.o_seq_stride + head * a.o_head_stride;
    const __amdgpu_buffer_rsrc_t o_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        o_base, 0, static_cast<int>(row_bytes + D * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t core_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        a.core ? a.core + (o_base - a.out) : o_base, 0, static_cast<int>(row_bytes + D * 2),
        0x00020000);
    const uint16_t* gate_base =
        a.gate ? a.gate + seq * a.gate_seq_stride + head * a.gate_head_stride : a.q;
    const __amdgpu_buffer_rsrc_t gate_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(gate_base), 0,
        static_cast<int>(static_cast<long long>(a.q_rows - 1) * a.gate_row_stride * 2 + D * 2),
        0x00020000);
    {
    const float l_used = l_acc[0] > 0.0f ? l_acc[0] : 1.0f;
    const float inverse = 1.0f / l_used;
    // A lane owns, for its query, channels 32db + 8j + 4h .. +3 of O^T: written
    // straight from there a store instruction would touch 32 rows, 16 bytes
    // each.  The wave's 32 x D block goes through LDS instead (its own 8 KiB of
    // the two stages the diagonal tiles above never use, so no barrier is
    // needed), and comes back as whole rows: sixteen lanes a row, 16 bytes a
    // lane, for the gate logits, the output and the optional ungated copy.
    // Chunk c of row r sits at slot c ^ (r & 15): both directions spread over
    // the banks.
    unsigned char* rows_out = lds + 2 * kStageBytes + wave * (32 * D * 2);
    constexpr int kRowChunks = D / 8, kRowsAtOnce = 64 / kRowChunks;  // 16-byte pieces a row
    const int part = lane_here / kRowChunks, chunk = lane_here % kRowChunks;
    // every gate load is requested before the first store: a load returns
    // behind the stores issued before it, and those take their time
    uint32x4 gate_words[32 / kRowsAtOnce];
    if (a.gate) {
#pragma unroll
      for (int i = 0; i < 32 / kRowsAtOnce; ++i) {
        const int row = wave_q0 + kRowsAtOnce * i + part;
        const uint32_t gate_at =
            row < a.q_rows
                ? static_cast<uint32_t>(static_cast<long long>(row) * a.gate_row_stride * 2) + chunk * 16
                : kDropped;
        gate_words[i] = __builtin_amdgcn_raw_buffer_load_b128(gate_rsrc, gate_at, 0, 0);
      }
    }
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int chunk = 4 * db + j;
        const uint2 plain = {pack_bf16(o_acc[db][4 * j + 0] * inverse, o_acc[db][4 * j + 1] * inverse),
                             pack_bf16(o_acc[db][4 * j + 2] * inverse, o_acc[db][4 * j + 3] * inverse)};
        *reinterpret_cast<uint2*>(rows_out + n * (D * 2) + ((chunk ^ (n & (kRowChunks - 1))) * 16) + 8 * h) = plain;
      }
    __builtin_amdgcn_s_waitcnt(0xC07F);
#pragma unroll
    for (int i = 0; i < 32 / kRowsAtOnce; ++i) {
      const int r = kRowsAtOnce * i + part;
      const uint4 core_bits =
          *reinterpret_cast<const uint4*>(rows_out + r * (D * 2) + ((chunk ^ (r & (kRowChunks - 1))) * 16));
      const int row = wave_q0 + r;
      const bool row_in_range = row < a.q_rows;
      const uint32_t at = row_in_range
                              ? static_cast<uint32_t>(static_cast<long long>(row) * a.o_row_stride * 2) + chunk * 16
                              : kDropped;
      const uint32x4 core_words = {core_bits.x, core_bits.y, core_bits.z, core_bits.w};
      if (a.core) __builtin_amdgcn_raw_buffer_store_b128(core_words, core_rsrc, at, 0, 0);
      uint32x4 out_words = core_words;
      if (a.gate) {
        // out = bf16(bf16(core) * bf16(sigmoid(gate))): qwen_attention.cc:103-108
        const uint32x4 gw = gate_words[i];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const float low = __uint_as_float(core_words[w] << 16) *
                            round_to_bf16(gate_sigmoid(__uint_as_float(gw[w] << 16)));
          const float high = __uint_as_float(core_words[w] & 0xffff0000u) *
                             round_to_bf16(gate_sigmoid(__uint_as_float(gw[w] & 0xffff0000u)));
          out_words[w] = pack_bf16(low, high);
        }
      }
      __builtin_amdgcn_raw_buffer_store_b128(out_words, o_rsrc, at, 0, 0);
    }
    // statistics relative to the true maximum (attention.cc:161-168), from the
    // lower lane half
    const float normalizer = l_used * __builtin_amdgcn_exp2f(m_used - m_true * scale2);
    const float maximum = m_true * a.scale;
    const uint32_t stat_at = in_range && h == 0 ? static_cast<uint32_t>(q_row) * 4u : kDropped;
    const long long stat = (static_cast<long long>(seq) * a.query_heads + head) * a.q_rows;
    if (a.maxima)
      __builtin_amdgcn_raw_buffer_store_b32(
          __float_as_uint(maximum),
          __builtin_amdgcn_make_buffer_rsrc(a.maxima + stat, 0, a.q_rows * 4, 0x00020000), stat_at,
          0, 0);
    if (a.normalizers)
      __builtin_amdgcn_raw_buffer_store_b32(
          __float_as_uint(normalizer),
          __builtin_amdgcn_make_buffer_rsrc(a.normalizers + stat, 0, a.q_rows * 4, 0x00020000),
          stat_at, 0, 0);
    if (a.lse) {
      float* lse_base = a.lse + static_cast<long long>(seq) * a.q_rows * a.query_heads + head;
      const long long lse_bytes = (static_cast<long long>(a.q_rows - 1) * a.query_heads + 1) * 4;
      const uint32_t lse_at =
          in_range && h == 0 ? static_cast<uint32_t>(static_cast<long long>(q_row) * a.query_heads * 4)
                             : kDropped;
      __builtin_amdgcn_raw_buffer_store_b32(
          __float_as_uint(maximum + __logf(normalizer)),
          __builtin_amdgcn_make_buffer_rsrc(lse_base, 0, static_cast<int>(lse_bytes), 0x00020000),
          lse_at, 0, 0);
    }
    }
  }
  // the next tile's fills must not overtake this tile's last LDS reads
  __syncthreads();
  }
}

}  // namespace

// ---- host side: packing tiles into per-workgroup lists ------------------------------------
namespace {

struct ScheduleKey {
  int q_rows = -1, kv_rows = 0, start_position = 0, query_heads = 0, group = 0, sequences = 0,
      workgroups = 0,  // resident at once: compute units x workgroups a compute unit
      tile_rows = 0;   // query rows of a tile
  bool operator==(const ScheduleKey& o) const {
    return q_rows == o.q_rows && kv_rows == o.kv_rows && start_position == o.start_position &&
           query_heads == o.query_heads && group == o.group && sequences == o.sequences &&
           workgroups == o.workgroups && tile_rows == o.tile_rows;
  }
};

// Cost of a query tile in key tiles: those it walks plus a fixed part (fills
// in flight before the first product, the epilogue, the end-of-tile barriers)
// that was measured at seven to eleven key tiles' time.
constexpr int kFixedCost = 8;

int tile_cost(const ScheduleKey& k, int q_tile) {
  const long long last_row = std::min<long long>((q_tile + 1LL) * k.tile_rows, k.q_rows) - 1;
  const long long visible = std::min<long long>(k.kv_rows, k.start_position + last_row + 1);
  return static_cast<int>((visible + BN - 1) / BN) + kFixedCost;
}

// Longest-first greedy packing, then sweeps over all pairs of lists: the swap
// or move between two lists that brings their loads closest is made, until a
// sweep changes nothing.  Items are indices into `cost`.  (8192 rows, 24 heads
// on 64 lists: greedy leaves the fullest list 8 % over the mean, the sweeps
// under 1 %.)
void pack(const std::vector<int>& cost, int lists, std::vector<std::vector<int>>& out) {
  std::vector<int> order(cost.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = static_cast<int>(i);
  std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return cost[x] > cost[y]; });
  out.assign(lists, {});
  std::vector<long long> load(lists, 0);
  for (int item : order) {
    int best = 0;
    for (int b = 1; b < lists; ++b)
      if (load[b] < load[best]) best = b;
    out[best].push_back(item);
    load[best] += cost[item];
  }
  for (int sweep = 0; sweep < 16; ++sweep) {
    bool changed = false;
    for (int p = 0; p < lists; ++p)
      for (int q = p + 1; q < lists; ++q) {
        const long long gap = load[p] - load[q];  // a transfer of `delta` from p to q leaves gap - 2 delta
        if (gap == 0) continue;
        long long best_gap = gap < 0 ? -gap : gap;
        int best_a = -2, best_b = -2;
        long long best_delta = 0;
        auto consider = [&](long long delta, int ia, int ib) {
          long long left = gap - 2 * delta;
          if (left < 0) left = -left;
          if (left < best_gap) best_gap = left, best_a = ia, best_b = ib, best_delta = delta;
        };
        for (size_t ia = 0; ia < out[p].size(); ++ia) {
          consider(cost[out[p][ia]], static_cast<int>(ia), -1);
          for (size_t ib = 0; ib < out[q].size(); ++ib)
            consider(cost[out[p][ia]] - cost[out[q][ib]], static_cast<int>(ia), static_cast<int>(ib));
        }
        for (size_t ib = 0; ib < out[q].size(); ++ib)
          consider(-static_cast<long long>(cost[out[q][ib]]), -1, static_cast<int>(ib));
        if (best_a == -2) continue;
        if (best_a >= 0 && best_b >= 0) {
          std::swap(out[p][best_a], out[q][best_b]);
        } else if (best_a >= 0) {
          out[q].push_back(out[p][best_a]);
          out[p].erase(out[p].begin() + best_a);
        } else {
          out[p].push_back(out[q][best_b]);
          out[q].erase(out[q].begin() + best_b);
        }
        load[p] -= best_delta;
        load[q] += best_delta;
        changed = true;
      }
    if (!changed) break;
  }
}

// Fills `schedule` and returns the number of workgroups, or 0 when the launch
// should number its tiles by workgroup index instead (more tiles than the table
// holds, fewer tiles than compute units, an unusual device).
int build_schedule(const ScheduleKey& k, Schedule& schedule) {
  schedule.slots = 0;
  const int q_tiles = (k.q_rows + k.tile_rows - 1) / k.tile_rows;
  const int kv_heads = k.query_heads / k.group;
  const int kv_units = k.sequences * kv_heads;
  const long long items = 1LL * q_tiles * k.sequences * k.query_heads;
  if (k.workgroups % 8 != 0 || k.workgroups <= 0 || items <= k.workgroups ||
      items >= kNoItem)
    return 0;
  // Workgroup i runs on XCD i mod 8 and every XCD has its own L2: the heads of
  // a kv head stay on as few XCDs as the unit count allows.  All partitions
  // hold the same multiset of tiles, so one packing serves them all.
  int partitions, xcds_each, units_each;
  if (kv_units % 8 == 0)
    partitions = 8, xcds_each = 1, units_each = kv_units / 8;
  else if (8 % kv_units == 0)
    partitions = kv_units, xcds_each = 8 / kv_units, units_each = 1;
  else
    partitions = 1, xcds_each = 8, units_each = kv_units;
  const int lists = k.workgroups / 8 * xcds_each;
  std::vector<int> cost;
  cost.reserve(static_cast<size_t>(units_each) * k.group * q_tiles);
  for (int local = 0; local < units_each * k.group; ++local)
    for (int t = 0; t < q_tiles; ++t) cost.push_back(tile_cost(k, t));
  std::vector<std::vector<int>> packed;
  pack(cost, lists, packed);
  size_t slots = 0;
  for (const auto& list : packed) slots = std::max(slots, list.size());
  if (slots == 0 || slots * k.workgroups > static_cast<size_t>(kScheduleEntries)) return 0;
  for (size_t i = 0; i < slots * k.workgroups; ++i) schedule.item[i] = kNoItem;
  for (int p = 0; p < partitions; ++p)
    for (int j = 0; j < lists; ++j) {
      // list j of partition p -> workgroup on XCD x: the partition's XCDs are
      // p, p + partitions, ...
      const int xcd = p + partitions * (j % xcds_each);
      const int workgroup = (j / xcds_each) * 8 + (partitions == 1 ? j % 8 : xcd);
      std::vector<int> list = packed[j];
      std::stable_sort(list.begin(), list.end(), [&](int x, int y) { return cost[x] > cost[y]; });
      for (size_t e = 0; e < list.size(); ++e) {
        const int local = list[e] / q_tiles, q_tile = list[e] % q_tiles;
        // local = (unit within the partition) * group + head within the group
        const int unit = partitions == 1 ? local / k.group
                                         : (kv_units % 8 == 0 ? p + 8 * (local / k.group) : p);
        const int sequence = unit / kv_heads, kv_head = unit % kv_heads;
        const int head = kv_head * k.group + local % k.group;
        schedule.item[workgroup * slots + e] =
            static_cast<uint16_t>((sequence * k.query_heads + head) * q_tiles + q_tile);
      }
    }
  schedule.slots = static_cast<int>(slots);
  return k.workgroups;
}

}  // namespace

int launch_flash_forward_pipelined(hipStream_t stream, const FlashForwardArgs& a, int head_dim,
                                   int sequences) {
  if (head_dim != 64 && head_dim != 128 && head_dim != 256) return PLUTO_HIP_EUNSUPPORTED;
  const int tile_rows =
      32 * (head_dim == 256 ? kWaves<256> : head_dim == 128 ? kWaves<128> : kWaves<64>);
  const int per_compute_unit = head_dim == 64 ? 2 : 1;  // resident workgroups
  const long long q_tiles = (a.q_rows + tile_rows - 1) / tile_rows;
  const long long units = q_tiles * sequences * (a.query_heads / a.group);
  long long blocks = (units + 7) / 8 * 8 * a.group;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  // The packing depends on the shape only; a thread keeps the last one it made.
  thread_local ScheduleKey known;
  thread_local Schedule schedule;
  thread_local int scheduled_blocks = 0;
  ScheduleKey key;
  key.q_rows = a.q_rows, key.kv_rows = a.kv_rows, key.start_position = a.start_position;
  key.query_heads = a.query_heads, key.group = a.group, key.sequences = sequences;
  key.tile_rows = tile_rows;
  int device = 0, compute_units = 0;
  if (hipGetDevice(&device) != hipSuccess ||
      hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device) !=
          hipSuccess)
    compute_units = 0;
  key.workgroups = compute_units * per_compute_unit;
  if (!(key == known)) {
    scheduled_blocks = build_schedule(key, schedule);
    known = key;
  }
  if (scheduled_blocks > 0) blocks = scheduled_blocks;
  if (head_dim == 256)
    flash_forward_pipelined_kernel<256>
        <<<dim3(static_cast<unsigned>(blocks)), 64 * kWaves<256>, 0, stream>>>(
            a, static_cast<int>(units), schedule);
  else if (head_dim == 128)
    flash_forward_pipelined_kernel<128>
        <<<dim3(static_cast<unsigned>(blocks)), 64 * kWaves<128>, 0, stream>>>(
            a, static_cast<int>(units), schedule);
  else
    flash_forward_pipelined_kernel<64>
        <<<dim3(static_cast<unsigned>(blocks)), 64 * kWaves<64>, 0, stream>>>(
            a, static_cast<int>(units), schedule);
  return launch_status();
}

}  // namespace pluto_hip

extern "C" int pluto_hip_test_forward_schedule(int head_dim, int q_rows, int kv_rows,
                                               int start_position, int query_heads, int group,
                                               int sequences, int workgroups_resident,
                                               uint16_t* items, int capacity, int* workgroups,
                                               int* slots) {
  using namespace pluto_hip;
  if ((head_dim != 64 && head_dim != 128 && head_dim != 256) || q_rows <= 0 || kv_rows <= 0 ||
      start_position < 0 || query_heads <= 0 || group <= 0 || query_heads % group != 0 ||
      sequences <= 0 || workgroups_resident < 0 || !items || capacity < 0 || !workgroups || !slots)
    return PLUTO_HIP_EINVAL;
  ScheduleKey key;
  key.q_rows = q_rows, key.kv_rows = kv_rows, key.start_position = start_position;
  key.query_heads = query_heads, key.group = group, key.sequences = sequences;
  key.tile_rows =
      32 * (head_dim == 256 ? kWaves<256> : head_dim == 128 ? kWaves<128> : kWaves<64>);
  key.workgroups = workgroups_resident;
  static thread_local Schedule schedule;
  *workgroups = build_schedule(key, schedule);
  *slots = schedule.slots;
  const long long entries = static_cast<long long>(*workgroups) * schedule.slots;
  if (entries > capacity) return PLUTO_HIP_ELIMIT;
  for (long long i = 0; i < entries; ++i) items[i] = schedule.item[i];
  return 0;
}
