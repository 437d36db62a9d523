// FullyConnectedLayer, imported path (src/llm/layers/fully_connected.cc):
//   ImportedMatVecKernel          :40-68   y = bf16(W x), W output-major
//   QuantizeImportedInputKernel   :70-88   FP8 storage: x -> fp8(x / s) * s in
//                                          groups of 128, s = max|x| / 448
//   ImportedForward               :295-341 bf16 token -> fp32 -> (quantize) ->
//                                          mat-vec -> bf16
// One frozen checkpoint matrix [output_dim, input_dim] in bf16, fp32 or OCP
// FP8 E4M3 with FP32 scales [ceil(out/128), ceil(in/128)] times one bf16
// token.  Byte-bound: every weight is read once.  A wave owns four output
// rows and reads them in 16-byte pieces (whenever rows start 16-byte aligned),
// the token comes from the FP32 copy the first kernel leaves in the workspace;
// all arithmetic is FP32, the 64 lane sums are added by a butterfly.
#include <algorithm>

#include "dense.h"

namespace pluto_hip {
namespace {

constexpr int kGroup = 128;  // quantization group and scale block edge

// Value of an OCP FP8 E4M3 code: 1-4-3 bits, bias 7, no infinities, S.1111.111
// is NaN, subnormals m * 2^-9.
__device__ inline float fp8_value(uint32_t bits) {
  const uint32_t exponent = (bits >> 3) & 15u, mantissa = bits & 7u;
  float magnitude;
  if (exponent == 0)
    magnitude = static_cast<float>(mantissa) * 0.001953125f;
  else if (exponent == 15 && mantissa == 7)
    magnitude = __builtin_nanf("");
  else
    magnitude = __uint_as_float(((exponent + 120u) << 23) | (mantissa << 20));
  return (bits & 0x80u) ? -magnitude : magnitude;
}

// The FP8 E4M3 value nearest to v (ties to even, saturating at +-448), as a
// float: what element_cast to FP8 and back gives (fully_connected.cc:86-87).
__device__ inline float fp8_round(float v) {
  const float a = fabsf(v);
  if (a >= 448.0f) return copysignf(448.0f, v);
  int exponent = static_cast<int>((__float_as_uint(a) >> 23) & 255u) - 127;  // floor(log2 a)
  if (exponent < -6) exponent = -6;                                          // subnormal grid
  const float step = __uint_as_float(static_cast<uint32_t>(exponent - 3 + 127) << 23);
  const float rounded = __builtin_rintf(a / step) * step;  // a / step is exact
  return copysignf(fminf(rounded, 448.0f), v);
}

// token[i] = float(x[i]), for FP8 storage quantized per group of 128.
template <bool FP8>
__global__ void __launch_bounds__(kGroup)
imported_token_kernel(const uint16_t* x, int n, float* token) {
  __shared__ float largest[2];
  x += static_cast<size_t>(blockIdx.y) * n;      // one token per grid row
  token += static_cast<size_t>(blockIdx.y) * n;
  const int i = blockIdx.x * kGroup + threadIdx.x;
  const float v = i < n ? bf16_bits_to_float(x[i]) : 0.0f;
  if constexpr (!FP8) {
    if (i < n) token[i] = v;
  } else {
    const float mine = wave_max(fabsf(v));
    if (threadIdx.x % 64 == 0) largest[threadIdx.x / 64] = mine;
    __syncthreads();
    const float scale = fmaxf(largest[0], largest[1]) / 448.0f;
    // only the divisor is floored: the result keeps the group's own scale
    if (i < n) token[i] = fp8_round(v / fmaxf(scale, 1e-12f)) * scale;
  }
}

struct MatVecArgs {
  const void* weights = nullptr;
  const float* scales = nullptr;  // FP8 only
  const float* token = nullptr;  // [tokens, cols]
  uint16_t* out = nullptr;       // [tokens, rows]
  int cols = 0, rows = 0;
};

typedef float floatx2 __attribute__((ext_vector_type(2)));

// Four FP8 E4M3 codes of a word as floats, by the hardware conversion.
__device__ inline void fp8_word(uint32_t word, float* out) {
  const floatx2 lo = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(word), false);
  const floatx2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(word), true);
  out[0] = lo.x, out[1] = lo.y, out[2] = hi.x, out[3] = hi.y;
}

constexpr int kRowsPerWave = 4;

// STORAGE: 0 bf16, 1 fp32, 2 FP8 E4M3.  A wave owns four consecutive output
// rows: a lane takes 16-byte pieces of them at the same columns, so the token
// values of a piece are loaded once for four rows and four weight loads are
// in flight per lane.  TOKENS tokens share one pass over the weights; each
// token's sum is formed exactly as in the one-token kernel.
template <int STORAGE, int TOKENS>
__global__ void __launch_bounds__(256) imported_matvec_kernel(MatVecArgs a) {
  constexpr int kElementBytes = STORAGE == 0 ? 2 : (STORAGE == 1 ? 4 : 1);
  constexpr int kPiece = 16 / kElementBytes;  // elements per 16-byte load
  constexpr int R = kRowsPerWave;
  const int lane = threadIdx.x % 64;
  const int row0 = (blockIdx.x * 4 + threadIdx.x / 64) * R;
  if (row0 >= a.rows) return;
  const int scale_cols = (a.cols + kGroup - 1) / kGroup;
  size_t row_start[R];
  const float* scale_row[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = min(row0 + r, a.rows - 1);  // rows past the end repeat the last one
    row_start[r] = static_cast<size_t>(row) * a.cols;
    scale_row[r] =
        STORAGE == 2 ? a.scales + static_cast<size_t>(row / kGroup) * scale_cols : nullptr;
  }
  float sum[TOKENS][R];
#pragma unroll
  for (int t = 0; t < TOKENS; ++t)
#pragma unroll
    for (int r = 0; r < R; ++r) sum[t][r] = 0.0f;
  auto element = [&](int r, int c) {
    const size_t i = row_start[r] + c;
    if constexpr (STORAGE == 0)
      return bf16_bits_to_float(static_cast<const uint16_t*>(a.weights)[i]);
    else if constexpr (STORAGE == 1)
      return static_cast<const float*>(a.weights)[i];
    else
      return fp8_value(static_cast<const uint8_t*>(a.weights)[i]) * scale_row[r][c / kGroup];
  };
  int done = 0;
  if ((static_cast<size_t>(a.cols) * kElementBytes) % 16 == 0) {
    // every row starts on a 16-byte boundary (the buffer itself is at least
    // 256-byte aligned): whole pieces, a piece never straddles a scale block
    const unsigned char* base = static_cast<const unsigned char*>(a.weights);
    const int pieces = a.cols / kPiece;
    for (int p = lane; p < pieces; p += 64) {
      const int c0 = p * kPiece;
      uint4 raw[R];
#pragma unroll
      for (int r = 0; r < R; ++r)
        raw[r] = *reinterpret_cast<const uint4*>(base + row_start[r] * kElementBytes +
                                                 static_cast<size_t>(p) * 16);
      // the rows' values of this piece, decoded once for all tokens
      float w[R][kPiece];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const uint32_t words[4] = {raw[r].x, raw[r].y, raw[r].z, raw[r].w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if constexpr (STORAGE == 0) {
            w[r][2 * k] = __uint_as_float(words[k] << 16);
            w[r][2 * k + 1] = __uint_as_float(words[k] & 0xffff0000u);
          } else if constexpr (STORAGE == 1) {
            w[r][k] = __uint_as_float(words[k]);
          } else {
            fp8_word(words[k], &w[r][4 * k]);
          }
        }
      }
#pragma unroll
      for (int t = 0; t < TOKENS; ++t) {
        float x[kPiece];
#pragma unroll
        for (int q = 0; q < kPiece / 4; ++q) {
          const float4 v = *reinterpret_cast<const float4*>(
              a.token + static_cast<size_t>(t) * a.cols + c0 + 4 * q);
          x[4 * q] = v.x, x[4 * q + 1] = v.y, x[4 * q + 2] = v.z, x[4 * q + 3] = v.w;
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if constexpr (STORAGE == 2) {
            float part = 0.0f;
#pragma unroll
            for (int e = 0; e < kPiece; ++e) part += w[r][e] * x[e];
            sum[t][r] += part * scale_row[r][c0 / kGroup];
          } else {
#pragma unroll
            for (int e = 0; e < kPiece; ++e) sum[t][r] += w[r][e] * x[e];
          }
        }
      }
    }
    done = pieces * kPiece;
  }
  for (int c = done + lane; c < a.cols; c += 64) {
    float value[R];
#pragma unroll
    for (int r = 0; r < R; ++r) value[r] = element(r, c);
#pragma unroll
    for (int t = 0; t < TOKENS; ++t) {
      const float x = a.token[static_cast<size_t>(t) * a.cols + c];
#pragma unroll
      for (int r = 0; r < R; ++r) sum[t][r] += value[r] * x;
    }
  }
#pragma unroll
  for (int t = 0; t < TOKENS; ++t)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float total = wave_sum(sum[t][r]);
      if (lane == 0 && row0 + r < a.rows)
        a.out[static_cast<size_t>(t) * a.rows + row0 + r] = float_to_bf16_bits(total);
    }
}

// ---- more than eight tokens: the matrix cores --------------------------------
// out[t, r] = sum_k w[r, k] x[t, k] as a 32-row x 32-token tile per wave on
// v_mfma_f32_32x32x16_bf16.  bf16 weights and tokens are exact operands.  FP8
// codes are exact in bf16 too, so FP8 weights are multiplied unscaled with the
// FP8 values of the quantized tokens, and each block of 128 contraction
// elements is scaled once by (weight block scale) x (token group scale):
// the same products as (w s_w)(x s_x), summed in FP32 in a different order.
// Lane (n, h) covers elements [64 h, 64 h + 64) of a 128-element block, for
// weight row n (A operand) and for token n (B operand).  The eight waves of a
// workgroup share a tile and take every eighth block; their partial tiles are
// added in wave order through LDS.

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;

// Tokens as FP8 values in bf16 and their group scales [tokens, n / 128].  The
// values are written in the order the matrix-core kernel reads them, so that
// each of its loads is one contiguous KiB: [pass of 32 tokens][block of 128
// columns][step j][lane = token % 32 + 32 h][8], the lane's elements being
// columns 128 block + 64 h + 8 j .. + 7.
__global__ void __launch_bounds__(kGroup)
imported_token_fp8_kernel(const uint16_t* x, int n, uint16_t* values, float* scales) {
  __shared__ float largest[2];
  const int token = blockIdx.y, block = blockIdx.x, c = threadIdx.x;
  x += static_cast<size_t>(token) * n;
  const int i = block * kGroup + c;
  const float v = i < n ? bf16_bits_to_float(x[i]) : 0.0f;
  const float mine = wave_max(fabsf(v));
  if (threadIdx.x % 64 == 0) largest[threadIdx.x / 64] = mine;
  __syncthreads();
  const float scale = fmaxf(largest[0], largest[1]) / 448.0f;
  const size_t pass = token / 32;
  const int lane = token % 32 + 32 * (c / 64), step = (c % 64) / 8;
  if (i < n)
    values[(((pass * gridDim.x + block) * 8 + step) * 64 + lane) * 8 + c % 8] =
        float_to_bf16_bits(fp8_round(v / fmaxf(scale, 1e-12f)));
  if (threadIdx.x == 0) scales[static_cast<size_t>(token) * gridDim.x + block] = scale;
}

struct TileArgs {
  const void* weights = nullptr;
  const float* weight_scales = nullptr;  // FP8 only
  const uint16_t* tokens = nullptr;      // bf16 [count, cols]; FP8: one pass in operand order
  const float* token_scales = nullptr;   // FP8 only: [count, cols / 128]
  uint16_t* out = nullptr;               // [count, rows]
  int cols = 0, rows = 0, count = 0;     // count <= 32
};

template <bool HIGH>
__device__ inline uint32_t fp8_pair_to_bf16(uint32_t word) {
  const floatx2 v = __builtin_amdgcn_cvt_pk_f32_fp8(static_cast<int>(word), HIGH);
  return (__float_as_uint(v.y) & 0xffff0000u) | (__float_as_uint(v.x) >> 16);
}

constexpr int kTileWaves = 8;  // waves that split a tile's contraction

// Several matrices applied to the same tokens in one launch: workgroup b works
// on matrix i with first_block[i] <= b < first_block[i + 1], tile b - first_block[i].
constexpr int kManyMax = 8;
struct TileManyArgs {
  const void* weights[kManyMax];
  const float* weight_scales[kManyMax];
  uint16_t* out[kManyMax];
  int rows[kManyMax];
  int first_block[kManyMax + 1];
  int matrices = 0;
  const uint16_t* tokens = nullptr;
  const float* token_scales = nullptr;
  int cols = 0, count = 0;
};

// One tile: 32 rows of the matrix times up to 32 tokens, the contraction split
// over the workgroup's waves.  AHEAD (FP8 only): blocks of a wave whose weight
// loads are issued together.
template <bool FP8, int AHEAD>
__device__ __forceinline__ void imported_tile(const TileArgs& a, int tile,
                                              float (*partial)[16][64]) {
  const int lane = threadIdx.x % 64, n = lane % 32, h = lane / 32;
  const int wave = threadIdx.x / 64;
  const int row_base = tile * 32;
  const int row = min(row_base + n, a.rows - 1);   // rows and tokens past the end repeat
  const int token = min(n, a.count - 1);           // the last one and are not stored
  const int groups = a.cols / kGroup;
  const unsigned char* w = static_cast<const unsigned char*>(a.weights) +
                           (static_cast<size_t>(row) * a.cols + 64 * h) * (FP8 ? 1 : 2);
  // FP8: operand order, 1 KiB a step; otherwise the token's own row
  const uint16_t* x = FP8 ? a.tokens + lane * 8 : a.tokens + static_cast<size_t>(token) * a.cols + 64 * h;
  const float* block_scale =
      FP8 ? a.weight_scales + static_cast<size_t>(row_base / kGroup) * groups : nullptr;
  const float* group_scale = FP8 ? a.token_scales + static_cast<size_t>(token) * groups : nullptr;
  floatx16 total;
#pragma unroll
  for (int i = 0; i < 16; ++i) total[i] = 0.0f;
  if constexpr (FP8) {
    // A wave's weight rows are few bytes (64 a lane and block): the loads of
    // AHEAD of its blocks (all of them for widths up to 8192) are issued before
    // anything is waited for, so that the latency of HBM is paid once a batch
    // and not once a block; the tokens (L2 hits) follow one block ahead of the
    // products.  Blocks past the end repeat the last one (loads without
    // branches) and are not added.
    constexpr int kAhead = AHEAD;
    for (int g0 = wave; g0 < groups; g0 += kTileWaves * kAhead) {
      uint4 raw[kAhead][4];
#pragma unroll
      for (int b = 0; b < kAhead; ++b) {
        const int g = min(g0 + b * kTileWaves, groups - 1);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          raw[b][j] = *reinterpret_cast<const uint4*>(w + static_cast<size_t>(g) * kGroup + 16 * j);
      }
      uint4 xs[2][8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        xs[0][j] = *reinterpret_cast<const uint4*>(x + (static_cast<size_t>(g0) * 8 + j) * 512);
#pragma unroll
      for (int b = 0; b < kAhead; ++b) {
        const int g = g0 + b * kTileWaves;
        if (b + 1 < kAhead) {
          const int next = min(g + kTileWaves, groups - 1);
#pragma unroll
          for (int j = 0; j < 8; ++j)
            xs[(b + 1) % 2][j] =
                *reinterpret_cast<const uint4*>(x + (static_cast<size_t>(next) * 8 + j) * 512);
        }
        floatx16 acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t lo = j % 2 == 0 ? raw[b][j / 2].x : raw[b][j / 2].z;
          const uint32_t hi = j % 2 == 0 ? raw[b][j / 2].y : raw[b][j / 2].w;
          const uint4 bits = make_uint4(fp8_pair_to_bf16<false>(lo), fp8_pair_to_bf16<true>(lo),
                                        fp8_pair_to_bf16<false>(hi), fp8_pair_to_bf16<true>(hi));
          acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, bits),
                                                        __builtin_bit_cast(bf16x8, xs[b % 2][j]),
                                                        acc, 0, 0, 0);
        }
        // a block past the end contributes nothing (its scale is read in range)
        const int in_range = min(g, groups - 1);
        const float scale = g < groups ? block_scale[in_range] * group_scale[in_range] : 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) total[i] += acc[i] * scale;
      }
    }
  } else {
    for (int g = wave; g < groups; g += kTileWaves) {
      uint4 xs[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) xs[j] = *reinterpret_cast<const uint4*>(x + g * kGroup + 8 * j);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint4 bits =
            *reinterpret_cast<const uint4*>(w + (static_cast<size_t>(g) * kGroup + 8 * j) * 2);
        total = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, bits),
                                                        __builtin_bit_cast(bf16x8, xs[j]), total,
                                                        0, 0, 0);
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < 16; ++i) partial[wave - 1][i][lane] = total[i];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int w = 0; w < kTileWaves - 1; ++w) total[i] += partial[w][i][lane];
  // accumulator element 4 q + i = (row 8 q + 4 h + i, token n)
  if (n >= a.count) return;
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = row_base + 8 * q + 4 * h + i;
      if (r < a.rows)
        a.out[static_cast<size_t>(n) * a.rows + r] = float_to_bf16_bits(total[4 * q + i]);
    }
}

template <bool FP8, int AHEAD = 1>
__global__ void __launch_bounds__(64 * kTileWaves) imported_tile_kernel(TileArgs a) {
  __shared__ float partial[kTileWaves - 1][16][64];
  imported_tile<FP8, AHEAD>(a, blockIdx.x, partial);
}

template <bool FP8, int AHEAD = 1>
__global__ void __launch_bounds__(64 * kTileWaves) imported_tile_many_kernel(TileManyArgs m) {
  __shared__ float partial[kTileWaves - 1][16][64];
  int which = 0;
  while (which + 1 < m.matrices && static_cast<int>(blockIdx.x) >= m.first_block[which + 1])
    ++which;
  TileArgs a;
  a.weights = m.weights[which];
  a.weight_scales = m.weight_scales[which];
  a.tokens = m.tokens;
  a.token_scales = m.token_scales;
  a.out = m.out[which];
  a.cols = m.cols;
  a.rows = m.rows[which];
  a.count = m.count;
  imported_tile<FP8, AHEAD>(a, blockIdx.x - m.first_block[which], partial);
}

template <int AHEAD>
void launch_fp8_tiles_ahead(hipStream_t s, const TileArgs& t, int blocks) {
  imported_tile_kernel<true, AHEAD><<<blocks, 64 * kTileWaves, 0, s>>>(t);
}

// Picks AHEAD = blocks a wave owns, up to eight.
void launch_fp8_tiles(hipStream_t s, const TileArgs& t, int blocks) {
  const int groups = t.cols / kGroup;
  switch (std::min(8, (groups + kTileWaves - 1) / kTileWaves)) {
    case 1: return launch_fp8_tiles_ahead<1>(s, t, blocks);
    case 2: return launch_fp8_tiles_ahead<2>(s, t, blocks);
    case 3: return launch_fp8_tiles_ahead<3>(s, t, blocks);
    case 4: return launch_fp8_tiles_ahead<4>(s, t, blocks);
    case 5: return launch_fp8_tiles_ahead<5>(s, t, blocks);
    case 6: return launch_fp8_tiles_ahead<6>(s, t, blocks);
    case 7: return launch_fp8_tiles_ahead<7>(s, t, blocks);
    default: return launch_fp8_tiles_ahead<8>(s, t, blocks);
  }
}

template <int AHEAD>
void launch_fp8_tiles_many_ahead(hipStream_t s, const TileManyArgs& t, int blocks) {
  imported_tile_many_kernel<true, AHEAD><<<blocks, 64 * kTileWaves, 0, s>>>(t);
}

void launch_fp8_tiles_many(hipStream_t s, const TileManyArgs& t, int blocks) {
  const int groups = t.cols / kGroup;
  switch (std::min(8, (groups + kTileWaves - 1) / kTileWaves)) {
    case 1: return launch_fp8_tiles_many_ahead<1>(s, t, blocks);
    case 2: return launch_fp8_tiles_many_ahead<2>(s, t, blocks);
    case 3: return launch_fp8_tiles_many_ahead<3>(s, t, blocks);
    case 4: return launch_fp8_tiles_many_ahead<4>(s, t, blocks);
    case 5: return launch_fp8_tiles_many_ahead<5>(s, t, blocks);
    case 6: return launch_fp8_tiles_many_ahead<6>(s, t, blocks);
    case 7: return launch_fp8_tiles_many_ahead<7>(s, t, blocks);
    default: return launch_fp8_tiles_many_ahead<8>(s, t, blocks);
  }
}

// The matrix-core path takes bf16 and FP8 weights whose rows are whole
// 128-element blocks; fewer than nine tokens are cheaper on the vector path.
bool tile_path(int storage, int tokens, int input_dim) {
  return storage != PLUTO_HIP_MATRIX_F32 && tokens > 8 && input_dim % kGroup == 0;
}

template <int STORAGE>
void launch_matvec(hipStream_t s, MatVecArgs a, int tokens) {
  const unsigned blocks =
      static_cast<unsigned>((a.rows + 4 * kRowsPerWave - 1) / (4 * kRowsPerWave));
  // up to eight tokens share a pass over the weights
  while (tokens > 0) {
    const int now = tokens >= 8 ? 8 : (tokens >= 4 ? 4 : (tokens >= 2 ? 2 : 1));
    if (now == 8)
      imported_matvec_kernel<STORAGE, 8><<<blocks, 256, 0, s>>>(a);
    else if (now == 4)
      imported_matvec_kernel<STORAGE, 4><<<blocks, 256, 0, s>>>(a);
    else if (now == 2)
      imported_matvec_kernel<STORAGE, 2><<<blocks, 256, 0, s>>>(a);
    else
      imported_matvec_kernel<STORAGE, 1><<<blocks, 256, 0, s>>>(a);
    a.token += static_cast<size_t>(now) * a.cols;
    a.out += static_cast<size_t>(now) * a.rows;
    tokens -= now;
  }
}

}  // namespace

namespace {
size_t tile_values_bytes(int tokens, int input_dim) {
  const size_t padded = (static_cast<size_t>(tokens) + 31) / 32 * 32;
  return align_up(padded * input_dim * 2, 256);
}
}  // namespace

size_t dense_imported_workspace_bytes(int tokens, int input_dim) {
  // FP32 tokens (vector path), or their FP8 values in bf16, in whole passes of
  // 32 tokens, and the group scales (matrix-core path)
  const size_t vector_path = align_up(static_cast<size_t>(tokens) * input_dim * sizeof(float), 256);
  const size_t groups = (static_cast<size_t>(input_dim) + kGroup - 1) / kGroup;
  const size_t tile_path = tile_values_bytes(tokens, input_dim) + align_up(tokens * groups * 4, 256);
  return std::max(vector_path, tile_path) + 256;
}

int launch_dense_imported_forward(hipStream_t s, int storage, const void* weights,
                                  const float* scales, const void* input, int tokens,
                                  int input_dim, int output_dim, void* output, void* workspace) {
  const dim3 groups(static_cast<unsigned>((input_dim + kGroup - 1) / kGroup),
                    static_cast<unsigned>(tokens));
  if (tile_path(storage, tokens, input_dim)) {
    const bool fp8 = storage == PLUTO_HIP_MATRIX_FP8_E4M3;
    TileArgs t;
    t.weights = weights;
    t.weight_scales = scales;
    t.tokens = static_cast<const uint16_t*>(input);
    t.cols = input_dim;
    t.rows = output_dim;
    if (fp8) {
      uint16_t* values = static_cast<uint16_t*>(workspace);
      float* token_scales = reinterpret_cast<float*>(static_cast<char*>(workspace) +
                                                     tile_values_bytes(tokens, input_dim));
      imported_token_fp8_kernel<<<groups, kGroup, 0, s>>>(static_cast<const uint16_t*>(input),
                                                          input_dim, values, token_scales);
      t.tokens = values;
      t.token_scales = token_scales;
    }
    t.out = static_cast<uint16_t*>(output);
    const unsigned blocks = static_cast<unsigned>((output_dim + 31) / 32);
    for (int done = 0; done < tokens; done += 32) {
      t.count = tokens - done < 32 ? tokens - done : 32;
      if (fp8)
        launch_fp8_tiles(s, t, blocks);
      else
        imported_tile_kernel<false><<<blocks, 64 * kTileWaves, 0, s>>>(t);
      t.tokens += static_cast<size_t>(32) * input_dim;
      if (fp8) t.token_scales += static_cast<size_t>(32) * (input_dim / kGroup);
      t.out += static_cast<size_t>(32) * output_dim;
    }
    return launch_status();
  }
  float* token = static_cast<float*>(workspace);
  if (storage == PLUTO_HIP_MATRIX_FP8_E4M3)
    imported_token_kernel<true><<<groups, kGroup, 0, s>>>(static_cast<const uint16_t*>(input),
                                                          input_dim, token);
  else
    imported_token_kernel<false><<<groups, kGroup, 0, s>>>(static_cast<const uint16_t*>(input),
                                                           input_dim, token);
  MatVecArgs a;
  a.weights = weights;
  a.scales = scales;
  a.token = token;
  a.out = static_cast<uint16_t*>(output);
  a.cols = input_dim;
  a.rows = output_dim;
  if (storage == PLUTO_HIP_MATRIX_BF16)
    launch_matvec<0>(s, a, tokens);
  else if (storage == PLUTO_HIP_MATRIX_F32)
    launch_matvec<1>(s, a, tokens);
  else
    launch_matvec<2>(s, a, tokens);
  return launch_status();
}

// Several matrices of one storage kind and input width applied to the same
// tokens: the tokens are prepared once and every pass of 32 tokens is one
// launch over the tiles of all matrices.  Takes the matrix-core path only
// (tile_path()); the caller falls back to one call a matrix otherwise.
int launch_dense_imported_forward_many(hipStream_t s, int storage, int matrices,
                                       const void* const* weights, const float* const* scales,
                                       const int* output_dims, const void* input, int tokens,
                                       int input_dim, void* const* outputs, void* workspace) {
  const bool fp8 = storage == PLUTO_HIP_MATRIX_FP8_E4M3;
  TileManyArgs t;
  t.matrices = matrices;
  t.cols = input_dim;
  t.tokens = static_cast<const uint16_t*>(input);
  t.first_block[0] = 0;
  for (int i = 0; i < kManyMax; ++i) {
    const bool used = i < matrices;
    t.weights[i] = used ? weights[i] : nullptr;
    t.weight_scales[i] = used && fp8 ? scales[i] : nullptr;
    t.out[i] = used ? static_cast<uint16_t*>(outputs[i]) : nullptr;
    t.rows[i] = used ? output_dims[i] : 0;
    t.first_block[i + 1] = t.first_block[i] + (used ? (output_dims[i] + 31) / 32 : 0);
  }
  if (fp8) {
    const dim3 groups(static_cast<unsigned>((input_dim + kGroup - 1) / kGroup),
                      static_cast<unsigned>(tokens));
    uint16_t* values = static_cast<uint16_t*>(workspace);
    float* token_scales = reinterpret_cast<float*>(static_cast<char*>(workspace) +
                                                   tile_values_bytes(tokens, input_dim));
    imported_token_fp8_kernel<<<groups, kGroup, 0, s>>>(static_cast<const uint16_t*>(input),
                                                        input_dim, values, token_scales);
    t.tokens = values;
    t.token_scales = token_scales;
  }
  const int blocks = t.first_block[matrices];
  for (int done = 0; done < tokens; done += 32) {
    t.count = tokens - done < 32 ? tokens - done : 32;
    if (fp8)
      launch_fp8_tiles_many(s, t, blocks);
    else
      imported_tile_many_kernel<false><<<blocks, 64 * kTileWaves, 0, s>>>(t);
    t.tokens += static_cast<size_t>(32) * input_dim;
    if (fp8) t.token_scales += static_cast<size_t>(32) * (input_dim / kGroup);
    for (int i = 0; i < matrices; ++i) t.out[i] += static_cast<size_t>(32) * output_dims[i];
  }
  return launch_status();
}

}  // namespace pluto_hip

using namespace pluto_hip;

extern "C" {

static int validate_imported(int storage, const float* scales, int tokens, int input_dim,
                             int output_dim) {
  if (storage != PLUTO_HIP_MATRIX_BF16 && storage != PLUTO_HIP_MATRIX_F32 &&
      storage != PLUTO_HIP_MATRIX_FP8_E4M3)
    return PLUTO_HIP_EINVAL;
  // fully_connected.cc:271-275: dimensions in [1, 1048576]
  if (input_dim <= 0 || input_dim > PLUTO_HIP_IMPORTED_MAX_DIM || output_dim <= 0 ||
      output_dim > PLUTO_HIP_IMPORTED_MAX_DIM)
    return PLUTO_HIP_EINVAL;
  if (tokens <= 0 || tokens > PLUTO_HIP_IMPORTED_MAX_TOKENS) return PLUTO_HIP_EINVAL;
  // :279-281: only FP8 weights have block scales
  if ((storage == PLUTO_HIP_MATRIX_FP8_E4M3) != (scales != nullptr)) return PLUTO_HIP_EINVAL;
  return 0;
}

size_t pluto_hip_dense_imported_workspace_bytes(int input_dim) {
  return pluto_hip_dense_imported_batch_workspace_bytes(1, input_dim);
}

size_t pluto_hip_dense_imported_batch_workspace_bytes(int tokens, int input_dim) {
  if (input_dim <= 0 || input_dim > PLUTO_HIP_IMPORTED_MAX_DIM || tokens <= 0 ||
      tokens > PLUTO_HIP_IMPORTED_MAX_TOKENS)
    return 0;
  return dense_imported_workspace_bytes(tokens, input_dim);
}

int pluto_hip_dense_imported_forward(void* stream, int storage, const void* weights,
                                     const float* scales, const void* input, int input_dim,
                                     int output_dim, void* output, void* workspace,
                                     size_t workspace_bytes) {
  return pluto_hip_dense_imported_forward_batch(stream, storage, weights, scales, input, 1,
                                                input_dim, output_dim, output, workspace,
                                                workspace_bytes);
}

int pluto_hip_dense_imported_forward_batch(void* stream, int storage, const void* weights,
                                           const float* scales, const void* input, int tokens,
                                           int input_dim, int output_dim, void* output,
                                           void* workspace, size_t workspace_bytes) {
  const int status = validate_imported(storage, scales, tokens, input_dim, output_dim);
  if (status != 0) return status;
  if (!weights || !input || !output) return PLUTO_HIP_EINVAL;
  if (!workspace || workspace_bytes < dense_imported_workspace_bytes(tokens, input_dim))
    return PLUTO_HIP_EWORKSPACE;
  return launch_dense_imported_forward(static_cast<hipStream_t>(stream), storage, weights, scales,
                                       input, tokens, input_dim, output_dim, output, workspace);
}

int pluto_hip_dense_imported_forward_many(void* stream, int storage, int matrices,
                                          const void* const* weights,
                                          const float* const* scales, const int* output_dims,
                                          const void* input, int tokens, int input_dim,
                                          void* const* outputs, void* workspace,
                                          size_t workspace_bytes) {
  if (matrices <= 0 || matrices > PLUTO_HIP_IMPORTED_MAX_MATRICES || !weights || !output_dims ||
      !outputs || !input)
    return PLUTO_HIP_EINVAL;
  const bool fp8 = storage == PLUTO_HIP_MATRIX_FP8_E4M3;
  if (fp8 && !scales) return PLUTO_HIP_EINVAL;
  long long tiles = 0;
  for (int i = 0; i < matrices; ++i) {
    const int status = validate_imported(storage, fp8 ? scales[i] : nullptr, tokens, input_dim,
                                         output_dims[i]);
    if (status != 0) return status;
    if (!fp8 && scales && scales[i]) return PLUTO_HIP_EINVAL;
    if (!weights[i] || !outputs[i]) return PLUTO_HIP_EINVAL;
    tiles += (output_dims[i] + 31) / 32;
  }
  if (tiles > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  if (!workspace || workspace_bytes < dense_imported_workspace_bytes(tokens, input_dim))
    return PLUTO_HIP_EWORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (tile_path(storage, tokens, input_dim))
    return launch_dense_imported_forward_many(s, storage, matrices, weights, scales, output_dims,
                                              input, tokens, input_dim, outputs, workspace);
  // few tokens, FP32 matrices or a ragged width: one call a matrix, same results
  for (int i = 0; i < matrices; ++i) {
    const int status = launch_dense_imported_forward(s, storage, weights[i],
                                                     fp8 ? scales[i] : nullptr, input, tokens,
                                                     input_dim, output_dims[i], outputs[i],
                                                     workspace);
    if (status != 0) return status;
  }
  return 0;
}

}  // extern "C"
