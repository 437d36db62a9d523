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

typedef __attribute__((ext_vector_type(4))) short shortx4;
typedef __attribute__((address_space(3))) void lds_void;

// Buffer descriptor over [base, base + bytes) for direct-to-LDS loads: loads
// beyond `bytes` deliver 0.  base and bytes must be the same in every lane.
typedef int int32x4 __attribute__((ext_vector_type(4)));
__device__ inline int32x4 make_rsrc(const void* base, uint32_t bytes) {
  const uint64_t address = reinterpret_cast<uint64_t>(base);
  int32x4 d;
  d.x = __builtin_amdgcn_readfirstlane(static_cast<int>(address));
  d.y = __builtin_amdgcn_readfirstlane(static_cast<int>((address >> 32) & 0xffff));
  d.z = __builtin_amdgcn_readfirstlane(static_cast<int>(bytes));
  d.w = 0x00020000;
  return d;
}

// One direct-to-LDS load: lane l's BYTES (16 or 4) from byte `offset` of the
// descriptor land at `lds` + l * BYTES; `lds` is the same in every lane.
// Written as assembly on purpose: for the builtin the compiler makes every
// later LDS read wait for all outstanding fills (it cannot tell the stage that
// is being filled from the one that is being read), which serializes a
// double-buffered loop inside each wave.  Callers order fills and reads
// themselves: s_waitcnt vmcnt + a workgroup barrier before a stage is read,
// a barrier after its last read before it is refilled.  The instruction takes
// the LDS base from M0, which cannot be named as a clobber, so the statement
// saves M0 in a scalar temporary and restores it after the load has been
// issued (the base is read at issue): whatever the compiler keeps in M0
// survives.
template <int BYTES>
__device__ inline void lds_fill(int32x4 descriptor, const void* lds, uint32_t offset) {
  static_assert(BYTES == 16 || BYTES == 4);
  const uint32_t address = __builtin_amdgcn_readfirstlane(
      static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_void*)lds)));
  uint32_t saved_m0;
  if constexpr (BYTES == 16)
    asm volatile(
        "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
        "buffer_load_dwordx4 %2, %3, 0 offen lds\n\ts_mov_b32 m0, %0"
        : "=&s"(saved_m0)
        : "s"(address), "v"(offset), "s"(descriptor)
        : "memory");
  else
    asm volatile(
        "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
        "buffer_load_dword %2, %3, 0 offen lds\n\ts_mov_b32 m0, %0"
        : "=&s"(saved_m0)
        : "s"(address), "v"(offset), "s"(descriptor)
        : "memory");
}

// LDS transpose read (ds_read_b64_tr_b16).  Within every group of 16 lanes,
// source lane s = 4*kk + b supplies 8 bytes (four 16-bit elements) at its
// address, and destination lane L = 4*b + e receives element e of source lanes
// b, b+4, b+8, b+12.  When source lane (kk, b) points at row kk, columns
// 4b..4b+3 of a row-major tile, lane L ends up with column L of rows 0..3.
__device__ inline uint2 lds_transpose_read(const unsigned char* tile, int byte_offset) {
  const shortx4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) shortx4*)(tile + byte_offset));
  return __builtin_bit_cast(uint2, v);
}

// Values of a per-lane quantity in the lower and in the upper lane half,
// each broadcast to both halves.  v_permlane32_swap exchanges the upper half of
// its first register with the lower half of its second; starting from two
// copies of v the first ends up all-lower, the second all-upper.  Written as
// inline assembly because both registers are results; the wait states around
// it cover the instruction's hazards with neighbouring vector instructions,
// which the compiler cannot see into.
__device__ inline void half_swap(float v, float& lower, float& upper) {
  float first = v, second = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1"
               : "+v"(first), "+v"(second));
  lower = first;
  upper = second;
}
// Per-lane value combined over both lane halves (lanes l and l ^ 32).
__device__ inline float half_swap_max(float v) {
  float lower, upper;
  half_swap(v, lower, upper);
  return fmaxf(lower, upper);
}
__device__ inline float half_swap_sum(float v) {
  float lower, upper;
  half_swap(v, lower, upper);
  return lower + upper;
}

// Row-major bf16 tile [rows][D] in LDS whose 16-byte chunk c of row r sits at
// slot c ^ tile_swizzle(r) of the row.  The permutation serves both ways the
// matrix cores read such a tile without bank conflicts: 16-byte row reads
// (eight consecutive rows, same chunk -> eight different slots) and transpose
// reads (four consecutive rows x two adjacent chunks -> eight different slots).
__device__ inline int tile_swizzle(int row) { return 2 * (row & 3) + ((row >> 2) & 1); }

// Queues the fill of a ROWS x D tile by direct-to-LDS buffer loads.  Load i of
// a lane writes 16 bytes at chunk (wave*LOADS + i)*64 + lane of the tile;
// offsets[i] = byte offset, from the tile's first row, of the chunk that
// belongs there (see tile_fill_offset).  base points at row `row0`; rows at or
// beyond `rows` read as zero.
template <int D, int LOADS>
__device__ inline void tile_fill(unsigned char* tile, int wave, const uint16_t* base,
                                 long long row_stride, int row0, int rows,
                                 const uint32_t* offsets) {
  const long long rows_left = rows - 1 - row0;
  const int32x4 rsrc = make_rsrc(
      base, rows_left < 0 ? 0u : static_cast<uint32_t>((rows_left * row_stride + D) * 2));
#pragma unroll
  for (int i = 0; i < LOADS; ++i)
    lds_fill<16>(rsrc, tile + (wave * LOADS + i) * 1024, offsets[i]);
}

template <int D>
__device__ inline uint32_t tile_fill_offset(int position, long long row_stride) {
  constexpr int KCH = D / 8;
  const int row = position / KCH, slot = position % KCH;
  return static_cast<uint32_t>(row * row_stride * 2 + (slot ^ tile_swizzle(row)) * 16);
}

// Byte offset of this lane's 16-byte row read: row n, chunk c.
template <int D>
__device__ inline int tile_row_read(int n, int chunk) {
  return (n * (D / 8) + (chunk ^ tile_swizzle(n))) * 16;
}

// Byte offset of this lane's transpose read for channel block db (channels
// 32db .. 32db+31 land on lanes n = lane % 32): as a source the lane supplies
// row 4*(lane/32) + kk, channels 32db + 16*((lane/16)%2) + 4b .. +3, with
// kk = (lane%16)/4 and b = lane%4.  Add (16*s2 + 8*part) rows for the keys of
// contraction step s2, part 0 = slots 0..3, part 1 = slots 4..7.
template <int D>
__device__ inline int tile_transpose_read(int lane, int db) {
  const int gq = lane / 16, kk = (lane % 16) / 4, b = lane % 4;
  const int row = 4 * (gq / 2) + kk;
  const int chunk = 4 * db + 2 * (gq % 2) + b / 2;
  return (row * (D / 8) + (chunk ^ tile_swizzle(row))) * 16 + (b % 2) * 8;
}

// Transposed A operand (32 channels x 16 rows in accumulator order) from a
// row-major tile: rows 16*s2 + {0..3, 8..11} + 4*(lane/32) of `block`.
template <int D>
__device__ inline bf16x8 tile_transposed_operand(const unsigned char* block, int lane_offset,
                                                 int s2) {
  const int at = lane_offset + 16 * s2 * (D / 8) * 16;
  const uint2 lo = lds_transpose_read(block, at);
  const uint2 hi = lds_transpose_read(block, at + 8 * (D / 8) * 16);
  return __builtin_bit_cast(bf16x8, make_uint4(lo.x, lo.y, hi.x, hi.y));
}

// XCD-aware renumbering of a 1-D grid: hardware deals workgroups round-robin
// to the 8 XCDs (each with a private L2); this makes consecutive logical ids
// land on the same XCD.
__device__ inline int xcd_logical_block() {
  if (gridDim.x % 8 != 0) return blockIdx.x;
  return (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
}

}  // namespace pluto_hip
