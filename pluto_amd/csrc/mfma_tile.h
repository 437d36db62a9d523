// LDS tile layouts shared by the bf16 MFMA attention kernels.
//
// v_mfma_f32_32x32x16_bf16 register layout (wave64, lane l, h = l/32, n = l%32):
//   A operand: 8 bf16 = A[row n][contraction slots 8h..8h+7]
//   B operand: 8 bf16 = B[contraction slots 8h..8h+7][column n]
//   C/D:       16 fp32, register i = C[row 8*(i/4) + 4h + i%4][column n]
// The contraction index may be enumerated in any order provided A and B use
// the same one.  A product whose B operand is a previous accumulator (lane
// keeps column n, registers 8s..8s+7 of the accumulator become the 8 slots of
// step s) therefore contracts over accumulator rows in the order
//   slot (s, h, e) -> row 16s + 8*(e/4) + 4h + e%4,
// and the matching A operand must be stored in that "accumulator order".
#pragma once

#include "common.h"

namespace pluto_hip {

__device__ inline bf16x8 as_bf16x8(uint4 v) {
  return __builtin_bit_cast(bf16x8, v);
}

// 16-bit element e (0..7) of a 16-byte register group, e known at compile time.
__device__ inline uint32_t half_word(uint4 v, int e) {
  const uint32_t w = e < 2 ? v.x : e < 4 ? v.y : e < 6 ? v.z : v.w;
  return (e & 1) ? (w >> 16) : (w & 0xffffu);
}

// Row-major tile [rows][D] of bf16 kept as 16-byte chunks (KCH = D/8 per row).
// XOR-ing the chunk with the row spreads the 8 rows read by consecutive lanes
// over all LDS banks.
template <int KCH>
__device__ inline int row_major_index(int row, int chunk) {
  return row * KCH + (chunk ^ (row & 7));
}

__device__ inline int swizzle_d(int d) { return (d & 7) ^ ((d >> 3) & 7); }

// Transposed tile [D][ROWS]: row d holds ROWS source rows in accumulator order
// as ROWS/8 chunks of 8.  Chunk c = 2*step + h (step = 16-row contraction step).
template <int ROWS>
__device__ inline int transposed_index(int d, int chunk) {
  return d * (ROWS / 8) + (chunk ^ swizzle_d(d));
}

// Writes a 4-row x 8-channel block (rows 4*quad..4*quad+3 of the tile,
// channels 8g..8g+7, one 16-byte register group per row) into a transposed
// tile.  quad = 8*blk + 4*s2 + 2*u + hh addresses source rows
// 32*blk + 16*s2 + 8*u + 4*hh + r, which sit in chunk 4*blk + 2*s2 + hh at
// positions 4u + r.
template <int ROWS>
__device__ inline void transposed_store(uint4* tile, int quad, int g, uint4 r0,
                                        uint4 r1, uint4 r2, uint4 r3) {
  uint2* tile2 = reinterpret_cast<uint2*>(tile);
  const int blk = quad >> 3, s2 = (quad >> 2) & 1, u = (quad >> 1) & 1,
            hh = quad & 1;
  const int chunk = 4 * blk + 2 * s2 + hh;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int d = 8 * g + e;
    uint2 packed;
    packed.x = half_word(r0, e) | (half_word(r1, e) << 16);
    packed.y = half_word(r2, e) | (half_word(r3, e) << 16);
    tile2[2 * transposed_index<ROWS>(d, chunk) + u] = packed;
  }
}

// Two floats to packed bf16 (one v_cvt_pk_bf16_f32).
__device__ inline uint32_t pack_bf16(float lo, float hi) {
  floatx2 two = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(two, bf16x2));
}

// Accumulator registers 8*s2 .. 8*s2+7 as a bf16 B operand.
__device__ inline bf16x8 accumulator_to_operand(const floatx16& acc, int s2) {
  return __builtin_bit_cast(
      bf16x8, make_uint4(pack_bf16(acc[8 * s2 + 0], acc[8 * s2 + 1]),
                         pack_bf16(acc[8 * s2 + 2], acc[8 * s2 + 3]),
                         pack_bf16(acc[8 * s2 + 4], acc[8 * s2 + 5]),
                         pack_bf16(acc[8 * s2 + 6], acc[8 * s2 + 7])));
}

__device__ inline floatx16 mfma32(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// XCD-aware renumbering of a 1-D grid: hardware deals workgroups round-robin
// to the 8 XCDs (each with a private L2); this makes consecutive logical ids
// land on the same XCD.
__device__ inline int xcd_logical_block() {
  if (gridDim.x % 8 != 0) return blockIdx.x;
  return (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
}

}  // namespace pluto_hip
