// Batched single-token GQA decode against a bf16 KV cache: split-K over blocks
// of the sequence, tuned as an HBM streaming kernel.
//
// Semantics: FullAttentionKernel (src/llm/layers/util/cached_attention_ops.cc:
// 83-126) for every sequence of the batch.  One workgroup owns one
// (sequence, kv head, block of `split_tokens` cache rows) and serves ALL query
// heads of the group, so every K and V byte is read from HBM exactly once (the
// reference launches one program per query head and streams the cache once per
// head of the group).
//
//   scores  S^T[token, head] = K[token, :] . q[head, :] with
//           v_mfma_f32_16x16x32_bf16: the A operand (16 tokens x 32 channels) is
//           loaded straight from global memory, 16 bytes per lane, the four
//           lanes of a token together one 64-byte sector per load;
//           the group's heads are the (zero padded) 16 columns.
//   values  O[head, :] += p[head, token] * V[token, :] on the vector ALU: 16
//           bytes of V per lane, probabilities broadcast from LDS.  The kernel
//           is bound by HBM, not by this arithmetic.
// Partial (o, m, l) triples are written per block; a second kernel combines a
// sequence's blocks in ascending order (fixed order: bitwise repeatable) and
// applies bf16(bf16(core) * bf16(sigmoid(gate))).
#include "gqa.h"

namespace pluto_hip {
namespace {

constexpr int kMaxSplit = 512;
constexpr int kThreads = 256;

__device__ inline bf16x8 load_bf16x8(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

__device__ inline int find_sequence(const DecodeBatch& batch, int block) {
  int lo = 0, hi = batch.count - 1;
  while (lo < hi) {  // last b with block_start[b] <= block
    const int mid = (lo + hi + 1) / 2;
    if (batch.block_start[mid] <= block) lo = mid; else hi = mid - 1;
  }
  return lo;
}

template <int D, int GROUP>
__global__ void __launch_bounds__(kThreads)
decode_split_kernel(DecodeArgs a, DecodeBatch batch) {
  constexpr int KSTEPS = D / 32;
  constexpr int LANES_PER_ROW = D / 8;     // phase 2: 16-byte pieces per V row
  constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
  // The probabilities (phases 1-2) and the per-wave partial outputs (after
  // phase 2) share one LDS area, so that eight workgroups fit a compute unit.
  constexpr int kProbFloats = kMaxSplit * 8, kOutFloats = 4 * GROUP * D;
  __shared__ __attribute__((aligned(16))) float shared_area[kProbFloats > kOutFloats ? kProbFloats : kOutFloats];
  float (*p_lds)[8] = reinterpret_cast<float (*)[8]>(shared_area);
  float (*o_lds)[GROUP][D] = reinterpret_cast<float (*)[GROUP][D]>(shared_area);
  __shared__ float wave_max[4][16];
  __shared__ float wave_sum_lds[4][16];

  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int kh = a.key_value_heads;
  const int g = blockIdx.x % kh;
  const int block = blockIdx.x / kh;
  const int b = find_sequence(batch, block);
  const int seq = batch.first + b;
  const int length = batch.positions[b] + 1;
  const int split = a.split_tokens;
  const int t0 = (block - batch.block_start[b]) * split;
  const int per_wave = split / 4;
  const uint16_t* keys = static_cast<const uint16_t*>(batch.keys[b]) + g * a.head_stride;
  const uint16_t* values = static_cast<const uint16_t*>(batch.values[b]) + g * a.head_stride;
  const float scale2 = a.scale * kLog2e;

  // ---- phase 1: scores -------------------------------------------------
  const int hq = lane / 16, n = lane % 16;
  bf16x8 qf[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    uint4 bits = make_uint4(0, 0, 0, 0);
    if (n < GROUP)
      bits = *reinterpret_cast<const uint4*>(
          a.q + (static_cast<long long>(seq) * a.query_heads + g * GROUP + n) * D +
          32 * ks + 8 * hq);
    qf[ks] = __builtin_bit_cast(bf16x8, bits);
  }
  // first batch of V rows for phase 2, requested now so that it travels while
  // phase 1 computes (per_wave is a multiple of 16 rows, kBatch passes cover
  // at most that)
  constexpr int kBatch = 2;  // measured: 2 beats 1, 4, 8 and 16
  const int sub = lane / LANES_PER_ROW, piece = lane % LANES_PER_ROW;
  auto load_v = [&](int pass) {
    const int token_local = wave * per_wave + pass * ROWS_PER_PASS + sub;
    const int token = min(t0 + token_local, length - 1);
    return *reinterpret_cast<const uint4*>(values + static_cast<long long>(token) * a.token_stride +
                                           8 * piece);
  };
  uint4 v_next[kBatch];
#pragma unroll
  for (int i = 0; i < kBatch; ++i) v_next[i] = load_v(i);
  const int groups = per_wave / 16;  // 16-token groups per wave (<= 8)
  floatx4 s[kMaxSplit / 64];
  float local_max = kMasked;
#pragma unroll
  for (int grp = 0; grp < kMaxSplit / 64; ++grp) {
    if (grp < groups) {
      const int token_local = wave * per_wave + 16 * grp;
      int token = t0 + token_local + n;  // A operand row = lane % 16
      token = min(token, length - 1);    // stay inside the valid prefix
      // contraction step ks covers channels 32 ks .. 32 ks + 31: the four lanes
      // of a token read one 64-byte sector per load
      const uint16_t* row = keys + static_cast<long long>(token) * a.token_stride + 8 * hq;
      floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(load_bf16x8(row + 32 * ks), qf[ks], acc,
                                                      0, 0, 0);
      // accumulator register r = (token 4*hq + r of the group, head n)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int t = t0 + token_local + 4 * hq + r;
        const float v = t < length ? acc[r] * scale2 : kMasked;
        acc[r] = v;
        local_max = fmaxf(local_max, v);
      }
      s[grp] = acc;
    }
  }
  local_max = fmaxf(local_max, __shfl_xor(local_max, 16, 64));
  local_max = fmaxf(local_max, __shfl_xor(local_max, 32, 64));
  if (hq == 0) wave_max[wave][n] = local_max;
  __syncthreads();
  const float block_max = fmaxf(fmaxf(wave_max[0][n], wave_max[1][n]),
                                fmaxf(wave_max[2][n], wave_max[3][n]));
  float local_sum = 0.0f;
#pragma unroll
  for (int grp = 0; grp < kMaxSplit / 64; ++grp) {
    if (grp < groups) {
      const int token_local = wave * per_wave + 16 * grp + 4 * hq;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float p = __builtin_amdgcn_exp2f(s[grp][r] - block_max);
        local_sum += p;
        if (n < 8) p_lds[token_local + r][n] = p;
      }
    }
  }
  local_sum += __shfl_xor(local_sum, 16, 64);
  local_sum += __shfl_xor(local_sum, 32, 64);
  if (hq == 0) wave_sum_lds[wave][n] = local_sum;
  __syncthreads();

  // ---- phase 2: O += p V ------------------------------------------------
  float acc[GROUP][8];
#pragma unroll
  for (int hh = 0; hh < GROUP; ++hh)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[hh][e] = 0.0f;
  const int passes = per_wave / ROWS_PER_PASS;
  // V rows travel in batches of kBatch loads per lane; a batch is requested
  // while the previous one is consumed (the first one before phase 1's
  // barriers, see above).
  for (int first = 0; first < passes; first += kBatch) {
    uint4 now[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) now[i] = v_next[i];
    if (first + kBatch < passes) {
#pragma unroll
      for (int i = 0; i < kBatch; ++i) v_next[i] = load_v(first + kBatch + i);
    }
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
      if (first + i >= passes) break;  // narrow heads with the smallest split
      const int token_local = wave * per_wave + (first + i) * ROWS_PER_PASS + sub;
      const uint4 bits = now[i];
      const float4 p0 = *reinterpret_cast<const float4*>(&p_lds[token_local][0]);
      const float4 p1 = *reinterpret_cast<const float4*>(&p_lds[token_local][4]);
      const float p[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
      const uint32_t w[4] = {bits.x, bits.y, bits.z, bits.w};
      float v[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = __uint_as_float(w[j] << 16);
        v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
#pragma unroll
      for (int hh = 0; hh < GROUP; ++hh)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[hh][e] += p[hh] * v[e];
    }
  }
  // exchange stages outermost: the exchanges of a stage are in flight together
#pragma unroll
  for (int offset = LANES_PER_ROW; offset < 64; offset <<= 1) {
    float other[GROUP][8];
#pragma unroll
    for (int hh = 0; hh < GROUP; ++hh)
#pragma unroll
      for (int e = 0; e < 8; ++e) other[hh][e] = __shfl_xor(acc[hh][e], offset, 64);
#pragma unroll
    for (int hh = 0; hh < GROUP; ++hh)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[hh][e] += other[hh][e];
  }
  __syncthreads();  // every wave is done with the probabilities
  if (sub == 0) {
#pragma unroll
    for (int hh = 0; hh < GROUP; ++hh) {
      float4 lo = make_float4(acc[hh][0], acc[hh][1], acc[hh][2], acc[hh][3]);
      float4 hi = make_float4(acc[hh][4], acc[hh][5], acc[hh][6], acc[hh][7]);
      *reinterpret_cast<float4*>(&o_lds[wave][hh][8 * piece]) = lo;
      *reinterpret_cast<float4*>(&o_lds[wave][hh][8 * piece + 4]) = hi;
    }
  }
  __syncthreads();
  const long long slot = (a.block_base + block) * kh + g;
  for (int i = tid; i < GROUP * D; i += kThreads) {
    const int hh = i / D, c = i % D;
    a.part_o[(slot * GROUP + hh) * D + c] =
        (o_lds[0][hh][c] + o_lds[1][hh][c]) + (o_lds[2][hh][c] + o_lds[3][hh][c]);
  }
  if (tid < GROUP) {
    a.part_m[slot * GROUP + tid] =
        fmaxf(fmaxf(wave_max[0][tid], wave_max[1][tid]), fmaxf(wave_max[2][tid], wave_max[3][tid]));
    a.part_l[slot * GROUP + tid] = (wave_sum_lds[0][tid] + wave_sum_lds[1][tid]) +
                                   (wave_sum_lds[2][tid] + wave_sum_lds[3][tid]);
  }
}

// One workgroup (4 waves) per (sequence, query head).  Wave w folds the blocks
// w, w+4, w+8, ... in ascending order, then the four partial results are added
// in wave order: a fixed summation tree, hence bitwise repeatable.  Ends with
// the sigmoid gate (cached_attention_ops.cc:119-125).
__global__ void __launch_bounds__(256)
decode_combine_kernel(DecodeCombineArgs a, DecodeBatch batch) {
  __shared__ float wave_max_lds[4];
  __shared__ float partial_o[4][256];
  __shared__ float partial_l[4];
  const int b = blockIdx.x / a.query_heads, head = blockIdx.x % a.query_heads;
  const int seq = batch.first + b;
  const int group = a.query_heads / a.key_value_heads;
  const int g = head / group, hh = head % group;
  const int D = a.head_dim;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int first = batch.block_start[b], blocks = batch.block_start[b + 1] - first;
  // partial results of block j live at slot0 + j * slot_step
  const long long slot0 = ((a.block_base + first) * a.key_value_heads + g) * group + hh;
  const long long slot_step = static_cast<long long>(a.key_value_heads) * group;
  float maximum = kMasked;
  for (int j = threadIdx.x; j < blocks; j += 256)
    maximum = fmaxf(maximum, a.part_m[slot0 + j * slot_step]);
  maximum = wave_max(maximum);
  if (lane == 0) wave_max_lds[wave] = maximum;
  __syncthreads();
  maximum = fmaxf(fmaxf(wave_max_lds[0], wave_max_lds[1]), fmaxf(wave_max_lds[2], wave_max_lds[3]));
  float normalizer = 0.0f;
  float o[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // head_dim <= 256 = 4 channels per lane
  // four blocks per step: all loads of a step are issued before their use
  for (int j0 = wave; j0 < blocks; j0 += 16) {
    float bm[4], bl[4], bo[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + 4 * u;
      const bool valid = j < blocks;
      const long long slot = slot0 + (valid ? j : j0) * slot_step;
      bm[u] = valid ? a.part_m[slot] : kMasked;
      bl[u] = a.part_l[slot];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        bo[u][i] = c < D ? a.part_o[slot * D + c] : 0.0f;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float w = j0 + 4 * u < blocks ? __builtin_amdgcn_exp2f(bm[u] - maximum) : 0.0f;
      normalizer += bl[u] * w;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] += bo[u][i] * w;
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) partial_o[wave][lane + 64 * i] = o[i];
  if (lane == 0) partial_l[wave] = normalizer;
  __syncthreads();
  const int c = threadIdx.x;
  if (c >= D) return;
  const float total = ((partial_l[0] + partial_l[1]) + partial_l[2]) + partial_l[3];
  const float sum = ((partial_o[0][c] + partial_o[1][c]) + partial_o[2][c]) + partial_o[3][c];
  const float core = sum / total;
  const long long at = static_cast<long long>(seq) * a.query_heads + head;
  const float logit = load_element(a.q_gate, (at * 2 + 1) * D + c, a.io_dtype);
  const float sigmoid = 1.0f / (1.0f + expf(-logit));
  const float value = a.round ? round_to_bf16(round_to_bf16(core) * round_to_bf16(sigmoid))
                              : core * sigmoid;
  store_element(a.out, at * D + c, a.io_dtype, value);
}

// Two-pass probability rows for inspection: one workgroup per (query head,
// query row).  Row r sees the first `first_visible + r` cache rows and is
// stored at probabilities[(head * rows + r) * row_width ..], zero beyond the
// visible prefix.
__global__ void __launch_bounds__(256)
attention_probabilities_kernel(const void* q, int q_dtype, CacheView cache, int query_heads,
                               int key_value_heads, int head_dim, int rows, int first_visible,
                               int row_width, float scale, float* probabilities) {
  __shared__ float query[256];
  __shared__ float reduce[4];
  const int head = blockIdx.x;
  const int r = blockIdx.y;
  const int length = first_visible + r;
  const int kv = head / (query_heads / key_value_heads);
  float* row = probabilities + (static_cast<long long>(head) * rows + r) * row_width;
  for (int c = threadIdx.x; c < head_dim; c += 256)
    query[c] = load_element(
        q, (static_cast<long long>(r) * query_heads + head) * head_dim + c, q_dtype);
  __syncthreads();
  float maximum = kMasked;
  for (int t = threadIdx.x; t < length; t += 256) {
    const long long base = t * cache.token_stride + kv * cache.head_stride;
    float score = 0.0f;
    for (int c = 0; c < head_dim; ++c)
      score += load_element(cache.keys, base + c, cache.dtype) * query[c];
    score *= scale;
    row[t] = score;
    maximum = fmaxf(maximum, score);
  }
  maximum = wave_max(maximum);
  if (threadIdx.x % 64 == 0) reduce[threadIdx.x / 64] = maximum;
  __syncthreads();
  maximum = fmaxf(fmaxf(reduce[0], reduce[1]), fmaxf(reduce[2], reduce[3]));
  __syncthreads();
  float sum = 0.0f;
  for (int t = threadIdx.x; t < length; t += 256) {
    const float p = expf(row[t] - maximum);
    row[t] = p;
    sum += p;
  }
  sum = wave_sum(sum);
  if (threadIdx.x % 64 == 0) reduce[threadIdx.x / 64] = sum;
  __syncthreads();
  sum = (reduce[0] + reduce[1]) + (reduce[2] + reduce[3]);
  for (int t = threadIdx.x; t < length; t += 256) row[t] = row[t] / sum;
  for (int t = length + threadIdx.x; t < row_width; t += 256) row[t] = 0.0f;
}

template <int D>
int launch_for_group(hipStream_t stream, const DecodeArgs& a, const DecodeBatch& batch,
                     int group, unsigned blocks) {
  switch (group) {
    case 1: decode_split_kernel<D, 1><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    case 2: decode_split_kernel<D, 2><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    case 4: decode_split_kernel<D, 4><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    case 6: decode_split_kernel<D, 6><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    case 8: decode_split_kernel<D, 8><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    default: return PLUTO_HIP_EUNSUPPORTED;
  }
  return launch_status();
}

}  // namespace

bool decode_fast_supported(int head_dim, int group) {
  const bool dim_ok = head_dim == 64 || head_dim == 128 || head_dim == 256;
  const bool group_ok = group == 1 || group == 2 || group == 4 || group == 6 || group == 8;
  return dim_ok && group_ok;
}

int launch_decode_fast(hipStream_t stream, const DecodeArgs& a, const DecodeBatch& batch) {
  const int group = a.query_heads / a.key_value_heads;
  const long long blocks =
      static_cast<long long>(batch.block_start[batch.count]) * a.key_value_heads;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  if (a.split_tokens < 64 || a.split_tokens > kMaxSplit || a.split_tokens % 64 != 0)
    return PLUTO_HIP_EINVAL;
  if (!kernel_enabled(kMainKernel)) return 0;
  switch (a.head_dim) {
    case 64: return launch_for_group<64>(stream, a, batch, group, static_cast<unsigned>(blocks));
    case 128: return launch_for_group<128>(stream, a, batch, group, static_cast<unsigned>(blocks));
    case 256: return launch_for_group<256>(stream, a, batch, group, static_cast<unsigned>(blocks));
    default: return PLUTO_HIP_EUNSUPPORTED;
  }
}

int launch_decode_combine(hipStream_t stream, const DecodeCombineArgs& a,
                          const DecodeBatch& batch) {
  if (!kernel_enabled(kAuxiliaryKernel)) return 0;
  decode_combine_kernel<<<batch.count * a.query_heads, 256, 0, stream>>>(a, batch);
  return launch_status();
}

int launch_attention_probabilities(hipStream_t stream, const void* q, int q_dtype,
                                   const CacheView& cache, int query_heads,
                                   int key_value_heads, int head_dim, int rows,
                                   int first_visible, int row_width, float scale,
                                   float* probabilities) {
  if (rows <= 0 || rows > 65535 || first_visible <= 0 ||
      static_cast<long long>(first_visible) + rows - 1 > row_width)
    return PLUTO_HIP_EINVAL;
  attention_probabilities_kernel<<<dim3(query_heads, rows), 256, 0, stream>>>(
      q, q_dtype, cache, query_heads, key_value_heads, head_dim, rows, first_visible, row_width,
      scale, probabilities);
  return launch_status();
}

}  // namespace pluto_hip
