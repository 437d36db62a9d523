// FullyConnectedLayer, trainable path (src/llm/layers/fully_connected.cc):
//   DenseForwardKernel         :97-131   y = bias + x w        (FP32 accumulate)
//   DenseInputGradientKernel   :134-164  dx = dy w^T
//   DenseWeightGradientKernel  :167-196  dw = x^T dy
//   DenseBias*GradientKernel   :198-247  db = column sums of dy, fixed order
// Operands are multiplied as 16-bit values (bf16 for bf16 activations, IEEE
// half for FP32 activations: MmaType, :31-33) and summed in FP32.  The FP32
// master matrix [input_dim, output_dim] and the FP32 gradient are converted
// to 16 bits once per call; the products then run on v_mfma_f32_32x32x16_*
// from LDS tiles filled by direct-to-LDS loads:
//   y and dx:      rows of both operands are contiguous along the contraction
//                  (x and w^T; dy and w) -> 16-byte row reads
//   dw:            the contraction runs over tokens, both operands (x, dy) are
//                  read through the LDS transpose read; the token range is
//                  split over workgroups and the slices are added in a fixed
//                  order
// Widths that are not multiples of 64 take a one-thread-per-element kernel
// with the same operand rounding.
#include "dense.h"

#include "mfma_tile.h"

namespace pluto_hip {
namespace {

typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int kDepth = 64;        // contraction elements per LDS tile
constexpr int kBiasRows = 256;    // fully_connected.cc:38

template <bool HALF>
__device__ inline floatx16 mma(uint4 a, uint4 b, floatx16 c) {
  if constexpr (HALF)
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a),
                                                  __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <bool HALF>
__device__ inline uint16_t to_operand(float value) {
  if constexpr (HALF) {
    const _Float16 h = static_cast<_Float16>(value);
    return __builtin_bit_cast(uint16_t, h);
  } else {
    return float_to_bf16_bits(value);
  }
}

template <bool HALF>
__device__ inline float operand_value(float value) {
  if constexpr (HALF)
    return static_cast<float>(static_cast<_Float16>(value));
  else
    return round_to_bf16(value);
}

// out[r, c] = operand(in[r, c]) or, transposed, out[c, r] = operand(in[r, c]).
template <bool HALF, bool TRANSPOSE>
__global__ void __launch_bounds__(256)
convert_kernel(const float* in, long long rows, int cols, uint16_t* out) {
  if constexpr (!TRANSPOSE) {
    const long long total = rows * cols;
    for (long long i = blockIdx.x * 256LL + threadIdx.x; i < total; i += 256LL * gridDim.x)
      out[i] = to_operand<HALF>(in[i]);
  } else {
    __shared__ uint16_t tile[32][33];
    const int c0 = blockIdx.x * 32;
    const long long r0 = blockIdx.y * 32LL;
    const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;
    for (int j = ty; j < 32; j += 8) {
      const long long r = r0 + j;
      const int c = c0 + tx;
      tile[j][tx] = (r < rows && c < cols) ? to_operand<HALF>(in[r * cols + c]) : 0;
    }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) {
      const int c = c0 + j;
      const long long r = r0 + tx;
      if (c < cols && r < rows) out[c * rows + r] = tile[tx][j];
    }
  }
}

struct ProductArgs {
  const uint16_t* left = nullptr;    // [m_rows, depth]   -> output rows
  const uint16_t* right = nullptr;   // [n_rows, depth]   -> output columns
  const float* bias = nullptr;       // optional [n_rows]
  void* out = nullptr;               // [m_rows, n_rows], bf16 or fp32
  int m_rows = 0, n_rows = 0, depth = 0;
  bool out_bf16 = false;
};

// Workgroup barrier that leaves queued global loads in flight (the library
// barrier waits for them too).
__device__ inline void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int COUNT>
__device__ inline void wait_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(COUNT) : "memory");
}

// out[m, n] = bias[n] + sum_k left[m, k] right[n, k]; depth % 64 == 0.  A
// workgroup of NWAVES waves, arranged 2 x (NWAVES / 2), owns a
// (64 JM) x (16 NWAVES JN) tile and each wave a (32 JM) x (32 JN) part of it.
// STAGES LDS stages of 64 contraction elements are filled STAGES - 1 steps
// ahead.
template <bool HALF, int JM, int JN, int STAGES, int NWAVES>
__global__ void __launch_bounds__(64 * NWAVES)
product_rows_kernel(ProductArgs a) {
  constexpr int THREADS = 64 * NWAVES;
  constexpr int KS = kDepth / 16;  // matrix instructions along the contraction per stage
  constexpr int TM = 64 * JM, TN = 32 * (NWAVES / 2) * JN;
  constexpr int kLeftBytes = TM * kDepth * 2, kRightBytes = TN * kDepth * 2;
  constexpr int kStageBytes = kLeftBytes + kRightBytes;
  constexpr int LEFT_LOADS = TM * (kDepth / 8) / THREADS;
  constexpr int RIGHT_LOADS = TN * (kDepth / 8) / THREADS;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[STAGES * kStageBytes];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int n_tiles = (a.n_rows + TN - 1) / TN;
  const int logical = xcd_logical_block();
  const int m0 = (logical / n_tiles) * TM, n0 = (logical % n_tiles) * TN;
  const int wm = 32 * JM * (wave / (NWAVES / 2)), wn = 32 * JN * (wave % (NWAVES / 2));
  uint32_t left_fill[LEFT_LOADS], right_fill[RIGHT_LOADS];
#pragma unroll
  for (int i = 0; i < LEFT_LOADS; ++i)
    left_fill[i] = tile_fill_offset<kDepth>((wave * LEFT_LOADS + i) * 64 + lane, a.depth);
#pragma unroll
  for (int i = 0; i < RIGHT_LOADS; ++i)
    right_fill[i] = tile_fill_offset<kDepth>((wave * RIGHT_LOADS + i) * 64 + lane, a.depth);
  // Rows 32 apart share the swizzle: block j of a quarter is 32 j rows further.
  constexpr int kBlockStep = 32 * (kDepth / 8) * 16;
  int left_read[KS], right_read[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    left_read[ks] = tile_row_read<kDepth>(wm + n, 2 * ks + h);
    right_read[ks] = tile_row_read<kDepth>(wn + n, 2 * ks + h);
  }
  // acc[jm][jn]: a lane holds output column n0 + wn + 32 jn + n of rows
  // m0 + wm + 32 jm + 8 q + 4 h + i (element 4 q + i)
  floatx16 acc[JM][JN];
#pragma unroll
  for (int jn = 0; jn < JN; ++jn) {
    const int column = n0 + wn + 32 * jn + n;
    const float start = (a.bias && column < a.n_rows) ? a.bias[column] : 0.0f;
#pragma unroll
    for (int jm = 0; jm < JM; ++jm)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[jm][jn][i] = start;
  }
  const uint16_t* left = a.left + static_cast<long long>(m0) * a.depth;
  const uint16_t* right = a.right + static_cast<long long>(n0) * a.depth;
  const int steps = a.depth / kDepth;
  auto fill_stage = [&](int step) {
    unsigned char* stage = lds + (step % STAGES) * kStageBytes;
    tile_fill<kDepth, LEFT_LOADS>(stage, wave, left + step * kDepth, a.depth, m0, a.m_rows,
                                  left_fill);
    tile_fill<kDepth, RIGHT_LOADS>(stage + kLeftBytes, wave, right + step * kDepth, a.depth, n0,
                                   a.n_rows, right_fill);
  };
  for (int step = 0; step < STAGES - 1 && step < steps; ++step) fill_stage(step);
  for (int step = 0; step < steps; ++step) {
    // stage `step` has landed once at most the STAGES - 2 later fills remain
    if (step + STAGES - 2 < steps)
      wait_loads<(STAGES - 2) * (LEFT_LOADS + RIGHT_LOADS)>();
    else
      wait_loads<0>();
    lds_barrier();
    if (step + STAGES - 1 < steps) fill_stage(step + STAGES - 1);
    const unsigned char* left_tile = lds + (step % STAGES) * kStageBytes;
    const unsigned char* right_tile = left_tile + kLeftBytes;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 l[JM], r[JN];
#pragma unroll
      for (int j = 0; j < JM; ++j)
        l[j] = *reinterpret_cast<const uint4*>(left_tile + left_read[ks] + j * kBlockStep);
#pragma unroll
      for (int j = 0; j < JN; ++j)
        r[j] = *reinterpret_cast<const uint4*>(right_tile + right_read[ks] + j * kBlockStep);
#pragma unroll
      for (int jm = 0; jm < JM; ++jm)
#pragma unroll
        for (int jn = 0; jn < JN; ++jn) acc[jm][jn] = mma<HALF>(l[jm], r[jn], acc[jm][jn]);
    }
  }
  // 32 lanes store 32 consecutive columns of a row: 64 or 128 contiguous bytes
#pragma unroll
  for (int jm = 0; jm < JM; ++jm)
#pragma unroll
    for (int jn = 0; jn < JN; ++jn) {
      const int column = n0 + wn + 32 * jn + n;
      if (column >= a.n_rows) continue;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = m0 + wm + 32 * jm + 8 * (i / 4) + 4 * h + i % 4;
        if (row >= a.m_rows) continue;
        const long long at = static_cast<long long>(row) * a.n_rows + column;
        if (a.out_bf16)
          static_cast<uint16_t*>(a.out)[at] = float_to_bf16_bits(acc[jm][jn][i]);
        else
          static_cast<float*>(a.out)[at] = acc[jm][jn][i];
      }
    }
}

// Short contractions take 128 x 128 tiles (more workgroups to overlap the
// start-up and the stores); from 1536 elements on, 256 x 256 tiles of eight
// waves, which halve the operand traffic from L2, are faster.
template <bool HALF>
void launch_product_rows(hipStream_t s, const ProductArgs& p) {
  auto blocks = [&](int tm, int tn) {
    return static_cast<unsigned>((p.m_rows + tm - 1) / tm) *
           static_cast<unsigned>((p.n_rows + tn - 1) / tn);
  };
  if (p.depth >= 1536)
    product_rows_kernel<HALF, 4, 2, 2, 8><<<blocks(256, 256), 512, 0, s>>>(p);
  else
    product_rows_kernel<HALF, 2, 2, 2, 4><<<blocks(128, 128), 256, 0, s>>>(p);
}

struct GramArgs {
  const uint16_t* left = nullptr;   // [rows, m_cols]
  const uint16_t* right = nullptr;  // [rows, n_cols]
  float* out = nullptr;             // [slices, m_cols, n_cols] partial sums
  int rows = 0, m_cols = 0, n_cols = 0, slices = 1;
};

// out[slice][m, n] = sum over the slice's rows r of left[r, m] right[r, n];
// m_cols and n_cols are multiples of 64.  A workgroup owns a 128 x 128 tile
// and one slice of the rows; both operands come from row-major [64 rows, 128]
// LDS tiles through the transpose read, 16 rows a contraction step.
template <bool HALF>
__global__ void __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(2, 2)))
product_columns_kernel(GramArgs a) {
  constexpr int kRows = 64;   // rows per LDS tile
  constexpr int kWidth = 128;
  constexpr int kBytes = kRows * kWidth * 2;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * kBytes];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int h = lane / 32, n = lane % 32;
  const int n_tiles = (a.n_cols + kWidth - 1) / kWidth, m_tiles = (a.m_cols + kWidth - 1) / kWidth;
  const int tile = blockIdx.x % (n_tiles * m_tiles), slice = blockIdx.x / (n_tiles * m_tiles);
  const int m0 = (tile / n_tiles) * kWidth, n0 = (tile % n_tiles) * kWidth;
  const int wm = 64 * (wave / 2), wn = 64 * (wave % 2);
  const int per_slice = ((a.rows + a.slices - 1) / a.slices + kRows - 1) / kRows * kRows;
  const int first = slice * per_slice, last = min(first + per_slice, a.rows);
  constexpr int LOADS = kRows * (kWidth / 8) / kThreads;  // 4
  uint32_t left_fill[LOADS], right_fill[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    left_fill[i] = tile_fill_offset<kWidth>((wave * LOADS + i) * 64 + lane, a.m_cols);
    right_fill[i] = tile_fill_offset<kWidth>((wave * LOADS + i) * 64 + lane, a.n_cols);
  }
  int left_read[2], right_read[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    left_read[j] = tile_transpose_read<kWidth>(lane, (wm + 32 * j) / 32);
    right_read[j] = tile_transpose_read<kWidth>(lane, (wn + 32 * j) / 32);
  }
  floatx16 acc[2][2];
#pragma unroll
  for (int jm = 0; jm < 2; ++jm)
#pragma unroll
    for (int jn = 0; jn < 2; ++jn)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[jm][jn][i] = 0.0f;
  // A tile may be wider than what is left of a row (widths are multiples of
  // 64, tiles 128 wide): those columns then hold the start of the next row,
  // which only reaches output elements that are not stored.  The descriptor
  // ends with row `last - 1`, so nothing is read beyond the slice.
  auto fill_tile = [&](unsigned char* tile, const uint16_t* matrix, int stride, int col0, int r0,
                       const uint32_t* offsets) {
    const long long begin = static_cast<long long>(r0) * stride + col0;
    const long long left_elements = static_cast<long long>(last) * stride - begin;
    const int32x4 rsrc = make_rsrc(
        matrix + begin, left_elements <= 0 ? 0u : static_cast<uint32_t>(left_elements * 2));
#pragma unroll
    for (int i = 0; i < LOADS; ++i)
      lds_fill<16>(rsrc, tile + (wave * LOADS + i) * 1024, offsets[i]);
  };
  auto fill_stage = [&](int step) {
    unsigned char* stage = lds + (step & 1) * 2 * kBytes;
    const int r0 = first + step * kRows;
    fill_tile(stage, a.left, a.m_cols, m0, r0, left_fill);
    fill_tile(stage + kBytes, a.right, a.n_cols, n0, r0, right_fill);
  };
  const int steps = first < last ? (last - first + kRows - 1) / kRows : 0;
  if (steps > 0) fill_stage(0);
  for (int step = 0; step < steps; ++step) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (step + 1 < steps) fill_stage(step + 1);
    const unsigned char* left_tile = lds + (step & 1) * 2 * kBytes;
    const unsigned char* right_tile = left_tile + kBytes;
#pragma unroll
    for (int s2 = 0; s2 < kRows / 16; ++s2) {
      uint4 l[2], r[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        l[j] = __builtin_bit_cast(uint4, tile_transposed_operand<kWidth>(left_tile, left_read[j], s2));
        r[j] = __builtin_bit_cast(uint4, tile_transposed_operand<kWidth>(right_tile, right_read[j], s2));
      }
#pragma unroll
      for (int jm = 0; jm < 2; ++jm)
#pragma unroll
        for (int jn = 0; jn < 2; ++jn) acc[jm][jn] = mma<HALF>(l[jm], r[jn], acc[jm][jn]);
    }
  }
  float* out = a.out + static_cast<long long>(slice) * a.m_cols * a.n_cols;
#pragma unroll
  for (int jm = 0; jm < 2; ++jm)
#pragma unroll
    for (int jn = 0; jn < 2; ++jn) {
      const int column = n0 + wn + 32 * jn + n;
      if (column >= a.n_cols) continue;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = m0 + wm + 32 * jm + 8 * (i / 4) + 4 * h + i % 4;
        if (row < a.m_cols) out[static_cast<long long>(row) * a.n_cols + column] = acc[jm][jn][i];
      }
    }
}

// out[i] = sum over slices of partial[slice][i], ascending.
__global__ void __launch_bounds__(256)
sum_slices_kernel(const float* partial, long long elements, int slices, float* out) {
  const long long i = blockIdx.x * 256LL + threadIdx.x;
  if (i >= elements) return;
  float sum = 0.0f;
  for (int s = 0; s < slices; ++s) sum += partial[s * elements + i];
  out[i] = sum;
}

// Column sums of [rows, width] in two levels with a fixed order
// (fully_connected.cc:198-247: 256-row partitions, then the partitions), and
// optionally the 16-bit copy of the same values: the gradient is read once
// for both.  A workgroup takes 64 columns of a 256-row partition; thread
// (lane, quad) = (tid / 16, tid % 16) adds rows lane, lane + 16, ... of four
// adjacent columns, and the sixteen lanes' sums are added in ascending order.
template <bool HALF>
__global__ void __launch_bounds__(256)
column_partial_kernel(const float* in, int rows, int width, float* partial, uint16_t* copy) {
  __shared__ float lanes[16][64];
  const int quad = threadIdx.x % 16, lane = threadIdx.x / 16;
  const int c = blockIdx.x * 64 + quad * 4;
  const int r0 = blockIdx.y * kBiasRows, r1 = min(r0 + kBiasRows, rows);
  float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (width % 4 == 0 && c < width) {
#pragma unroll 4
    for (int r = r0 + lane; r < r1; r += 16) {
      const long long at = static_cast<long long>(r) * width + c;
      const float4 value = *reinterpret_cast<const float4*>(in + at);
      sum[0] += value.x, sum[1] += value.y, sum[2] += value.z, sum[3] += value.w;
      if (copy) {
        ushort4 out;
        out.x = to_operand<HALF>(value.x), out.y = to_operand<HALF>(value.y);
        out.z = to_operand<HALF>(value.z), out.w = to_operand<HALF>(value.w);
        *reinterpret_cast<ushort4*>(copy + at) = out;
      }
    }
  } else {
    for (int r = r0 + lane; r < r1; r += 16)
      for (int e = 0; e < 4; ++e)
        if (c + e < width) {
          const float value = in[static_cast<long long>(r) * width + c + e];
          sum[e] += value;
          if (copy) copy[static_cast<long long>(r) * width + c + e] = to_operand<HALF>(value);
        }
  }
  for (int e = 0; e < 4; ++e) lanes[lane][quad * 4 + e] = sum[e];
  __syncthreads();
  const int column = blockIdx.x * 64 + threadIdx.x;
  if (threadIdx.x < 64 && column < width) {
    float total = lanes[0][threadIdx.x];
    for (int l = 1; l < 16; ++l) total += lanes[l][threadIdx.x];
    partial[static_cast<long long>(blockIdx.y) * width + column] = total;
  }
}

__global__ void __launch_bounds__(256)
column_final_kernel(const float* partial, int parts, int width, float* out) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= width) return;
  float sum = 0.0f;
#pragma unroll 16
  for (int p = 0; p < parts; ++p) sum += partial[static_cast<long long>(p) * width + c];
  out[c] = sum;
}

// Any shape: one thread per output element, operands rounded like the matrix
// cores' and summed in FP32 in ascending order.
//   mode 0: out[r, o] = bias[o] + sum_i x[r, i] w[i, o]   (x in `dtype`)
//   mode 1: out[r, i] = sum_o g[r, o] w[i, o]
//   mode 2: out[i, o] = sum_r x[r, i] g[r, o]
template <bool HALF>
__global__ void __launch_bounds__(256)
generic_dense_kernel(int mode, int dtype, const void* x, const float* w, const float* g,
                     const float* bias, int rows, int input_dim, int output_dim, void* out) {
  const long long i = blockIdx.x * 256LL + threadIdx.x;
  const long long total = mode == 0   ? 1LL * rows * output_dim
                          : mode == 1 ? 1LL * rows * input_dim
                                      : 1LL * input_dim * output_dim;
  if (i >= total) return;
  auto activation = [&](long long at) {
    return operand_value<HALF>(load_element(x, at, dtype));
  };
  float sum = 0.0f;
  if (mode == 0) {
    const int r = static_cast<int>(i / output_dim), o = static_cast<int>(i % output_dim);
    sum = bias[o];
    for (int k = 0; k < input_dim; ++k)
      sum += activation(1LL * r * input_dim + k) * operand_value<HALF>(w[1LL * k * output_dim + o]);
    store_element(out, i, dtype, sum);
    return;
  }
  if (mode == 1) {
    const int r = static_cast<int>(i / input_dim), k = static_cast<int>(i % input_dim);
    for (int o = 0; o < output_dim; ++o)
      sum += operand_value<HALF>(g[1LL * r * output_dim + o]) *
             operand_value<HALF>(w[1LL * k * output_dim + o]);
  } else {
    const int k = static_cast<int>(i / output_dim), o = static_cast<int>(i % output_dim);
    for (int r = 0; r < rows; ++r)
      sum += activation(1LL * r * input_dim + k) * operand_value<HALF>(g[1LL * r * output_dim + o]);
  }
  static_cast<float*>(out)[i] = sum;
}

unsigned blocks_for(long long elements, long long cap = 1LL << 20) {
  const long long blocks = (elements + 255) / 256;
  return static_cast<unsigned>(blocks < cap ? blocks : cap);
}

bool matrix_cores(int input_dim, int output_dim) {
  return input_dim % 64 == 0 && output_dim % 64 == 0;
}

int weight_slices(int rows, int input_dim, int output_dim) {
  const long long tiles = ((input_dim + 127) / 128) * static_cast<long long>((output_dim + 127) / 128);
  // two workgroups a compute unit: as many slices as still run in one round
  long long slices = 512 / tiles;
  const long long most = (rows + 255) / 256;     // at least 256 rows a slice
  if (slices > most) slices = most;
  return static_cast<int>(slices < 1 ? 1 : slices);
}

struct Layout {
  size_t matrix16, input16, gradient16, partial, bias_partial, total;
};

Layout layout(int dtype, int rows, int input_dim, int output_dim) {
  Layout l{};
  size_t at = 0;
  auto take = [&](size_t bytes) {
    const size_t offset = at;
    at += align_up(bytes, 256);
    return offset;
  };
  const size_t r = rows, in = input_dim, out = output_dim;
  l.matrix16 = take(in * out * 2);
  l.input16 = take(dtype == PLUTO_HIP_F32 ? r * in * 2 : 0);
  l.gradient16 = take(r * out * 2);
  l.partial = take(static_cast<size_t>(weight_slices(rows, input_dim, output_dim)) * in * out * 4);
  l.bias_partial = take(static_cast<size_t>((rows + kBiasRows - 1) / kBiasRows) * out * 4);
  l.total = at;
  return l;
}

template <bool HALF, bool TRANSPOSE>
void convert(hipStream_t s, const float* in, long long rows, int cols, uint16_t* out) {
  if constexpr (TRANSPOSE)
    convert_kernel<HALF, true><<<dim3((cols + 31) / 32, static_cast<unsigned>((rows + 31) / 32)),
                                 256, 0, s>>>(in, rows, cols, out);
  else
    convert_kernel<HALF, false><<<blocks_for(rows * cols, 8192), 256, 0, s>>>(in, rows, cols, out);
}

template <bool HALF>
int forward(hipStream_t s, int dtype, const void* input, const float* matrix, const float* bias,
            int rows, int input_dim, int output_dim, void* output, char* scratch) {
  if (!matrix_cores(input_dim, output_dim)) {
    generic_dense_kernel<HALF><<<blocks_for(1LL * rows * output_dim), 256, 0, s>>>(
        0, dtype, input, matrix, nullptr, bias, rows, input_dim, output_dim, output);
    return launch_status();
  }
  const Layout l = layout(dtype, rows, input_dim, output_dim);
  uint16_t* matrix16 = reinterpret_cast<uint16_t*>(scratch + l.matrix16);  // w^T [out, in]
  convert<HALF, true>(s, matrix, input_dim, output_dim, matrix16);
  const uint16_t* input16 = static_cast<const uint16_t*>(input);
  if (dtype == PLUTO_HIP_F32) {
    uint16_t* copy = reinterpret_cast<uint16_t*>(scratch + l.input16);
    convert<HALF, false>(s, static_cast<const float*>(input), rows, input_dim, copy);
    input16 = copy;
  }
  ProductArgs p;
  p.left = input16;
  p.right = matrix16;
  p.bias = bias;
  p.out = output;
  p.m_rows = rows;
  p.n_rows = output_dim;
  p.depth = input_dim;
  p.out_bf16 = dtype == PLUTO_HIP_BF16;
  launch_product_rows<HALF>(s, p);
  return launch_status();
}

template <bool HALF>
int backward(hipStream_t s, int dtype, const void* input, const float* matrix,
             const float* d_output, int rows, int input_dim, int output_dim, float* d_input,
             float* d_matrix, float* d_bias, char* scratch) {
  const Layout l = layout(dtype, rows, input_dim, output_dim);
  // bias gradient: 256-row partitions, then the partitions in order
  float* bias_partial = reinterpret_cast<float*>(scratch + l.bias_partial);
  const int parts = (rows + kBiasRows - 1) / kBiasRows;
  const bool cores = matrix_cores(input_dim, output_dim);
  uint16_t* gradient16 = reinterpret_cast<uint16_t*>(scratch + l.gradient16);  // dy [rows, out]
  column_partial_kernel<HALF><<<dim3((output_dim + 63) / 64, parts), 256, 0, s>>>(
      d_output, rows, output_dim, bias_partial, cores ? gradient16 : nullptr);
  column_final_kernel<<<(output_dim + 63) / 64, 64, 0, s>>>(bias_partial, parts, output_dim,
                                                            d_bias);
  if (!cores) {
    generic_dense_kernel<HALF><<<blocks_for(1LL * rows * input_dim), 256, 0, s>>>(
        1, dtype, input, matrix, d_output, nullptr, rows, input_dim, output_dim, d_input);
    generic_dense_kernel<HALF><<<blocks_for(1LL * input_dim * output_dim), 256, 0, s>>>(
        2, dtype, input, matrix, d_output, nullptr, rows, input_dim, output_dim, d_matrix);
    return launch_status();
  }
  uint16_t* matrix16 = reinterpret_cast<uint16_t*>(scratch + l.matrix16);      // w [in, out]
  convert<HALF, false>(s, matrix, input_dim, output_dim, matrix16);
  const uint16_t* input16 = static_cast<const uint16_t*>(input);
  if (dtype == PLUTO_HIP_F32) {
    uint16_t* copy = reinterpret_cast<uint16_t*>(scratch + l.input16);
    convert<HALF, false>(s, static_cast<const float*>(input), rows, input_dim, copy);
    input16 = copy;
  }
  // dx[r, i] = sum_o dy[r, o] w[i, o]
  ProductArgs p;
  p.left = gradient16;
  p.right = matrix16;
  p.out = d_input;
  p.m_rows = rows;
  p.n_rows = input_dim;
  p.depth = output_dim;
  launch_product_rows<HALF>(s, p);
  int status = launch_status();
  if (status != 0) return status;
  // dw[i, o] = sum_r x[r, i] dy[r, o], the rows in slices
  GramArgs g;
  g.left = input16;
  g.right = gradient16;
  g.rows = rows;
  g.m_cols = input_dim;
  g.n_cols = output_dim;
  g.slices = weight_slices(rows, input_dim, output_dim);
  g.out = g.slices == 1 ? d_matrix : reinterpret_cast<float*>(scratch + l.partial);
  const unsigned tiles = static_cast<unsigned>((input_dim + 127) / 128) *
                         static_cast<unsigned>((output_dim + 127) / 128);
  product_columns_kernel<HALF><<<tiles * g.slices, kThreads, 0, s>>>(g);
  status = launch_status();
  if (status != 0 || g.slices == 1) return status;
  const long long elements = 1LL * input_dim * output_dim;
  sum_slices_kernel<<<blocks_for(elements), 256, 0, s>>>(g.out, elements, g.slices, d_matrix);
  return launch_status();
}

}  // namespace

size_t dense_workspace_bytes(int dtype, int rows, int input_dim, int output_dim) {
  return layout(dtype, rows, input_dim, output_dim).total;
}

int launch_dense_forward(hipStream_t stream, int dtype, const void* input, const float* matrix,
                         const float* bias, int rows, int input_dim, int output_dim, void* output,
                         void* workspace) {
  char* scratch = static_cast<char*>(workspace);
  return dtype == PLUTO_HIP_BF16
             ? forward<false>(stream, dtype, input, matrix, bias, rows, input_dim, output_dim,
                              output, scratch)
             : forward<true>(stream, dtype, input, matrix, bias, rows, input_dim, output_dim,
                             output, scratch);
}

int launch_dense_backward(hipStream_t stream, int dtype, const void* input, const float* matrix,
                          const float* d_output, int rows, int input_dim, int output_dim,
                          float* d_input, float* d_matrix, float* d_bias, void* workspace) {
  char* scratch = static_cast<char*>(workspace);
  return dtype == PLUTO_HIP_BF16
             ? backward<false>(stream, dtype, input, matrix, d_output, rows, input_dim,
                               output_dim, d_input, d_matrix, d_bias, scratch)
             : backward<true>(stream, dtype, input, matrix, d_output, rows, input_dim, output_dim,
                              d_input, d_matrix, d_bias, scratch);
}

}  // namespace pluto_hip

using namespace pluto_hip;

extern "C" {

static int validate_dense(int dtype, int rows, int input_dim, int output_dim) {
  // fully_connected.cc:318-338: BF16 and FP32 activations are the trainable types
  if (dtype != PLUTO_HIP_F32 && dtype != PLUTO_HIP_BF16) return PLUTO_HIP_EUNSUPPORTED;
  if (rows <= 0 || input_dim <= 0 || output_dim <= 0) return PLUTO_HIP_EINVAL;
  if (static_cast<long long>(rows) * input_dim > 0x7fffffffLL ||
      static_cast<long long>(rows) * output_dim > 0x7fffffffLL ||
      static_cast<long long>(input_dim) * output_dim > 0x7fffffffLL)
    return PLUTO_HIP_ERANGE;
  return 0;
}

size_t pluto_hip_dense_workspace_bytes(int dtype, int rows, int input_dim, int output_dim) {
  if (validate_dense(dtype, rows, input_dim, output_dim) != 0) return 0;
  return dense_workspace_bytes(dtype, rows, input_dim, output_dim);
}

int pluto_hip_dense_forward(void* stream, int dtype, const void* input, const float* matrix,
                            const float* bias, int rows, int input_dim, int output_dim,
                            void* output, void* workspace, size_t workspace_bytes) {
  const int status = validate_dense(dtype, rows, input_dim, output_dim);
  if (status != 0) return status;
  if (!input || !matrix || !bias || !output) return PLUTO_HIP_EINVAL;
  if (!workspace || workspace_bytes < dense_workspace_bytes(dtype, rows, input_dim, output_dim))
    return PLUTO_HIP_EWORKSPACE;
  return launch_dense_forward(static_cast<hipStream_t>(stream), dtype, input, matrix, bias, rows,
                              input_dim, output_dim, output, workspace);
}

int pluto_hip_dense_backward(void* stream, int dtype, const void* input, const float* matrix,
                             const float* d_output, int rows, int input_dim, int output_dim,
                             float* d_input, float* d_matrix, float* d_bias, void* workspace,
                             size_t workspace_bytes) {
  const int status = validate_dense(dtype, rows, input_dim, output_dim);
  if (status != 0) return status;
  if (!input || !matrix || !d_output || !d_input || !d_matrix || !d_bias) return PLUTO_HIP_EINVAL;
  if (!workspace || workspace_bytes < dense_workspace_bytes(dtype, rows, input_dim, output_dim))
    return PLUTO_HIP_EWORKSPACE;
  return launch_dense_backward(static_cast<hipStream_t>(stream), dtype, input, matrix, d_output,
                               rows, input_dim, output_dim, d_input, d_matrix, d_bias, workspace);
}

}  // extern "C"
