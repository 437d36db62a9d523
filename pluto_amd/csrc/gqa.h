// Argument blocks and launchers of the Qwen grouped-query attention kernels.
#pragma once

#include "common.h"

namespace pluto_hip {

constexpr int kDecodeBatchMax = 64;  // sequences per decode launch

struct CacheView {
  void* keys = nullptr;
  void* values = nullptr;
  int dtype = PLUTO_HIP_BF16;
  long long token_stride = 0;
  long long head_stride = 0;
};

struct PrefillPrepareArgs {
  const void* qg = nullptr;  // bf16 [T, qh, 2, d]
  const void* k = nullptr;   // bf16 [T, kh, d]
  const void* v = nullptr;   // bf16 [T, kh, d]
  const float* q_norm = nullptr;
  const float* k_norm = nullptr;
  const float* cosines = nullptr;  // [T, rotary/2]
  const float* sines = nullptr;
  void* q_out = nullptr;  // [T, qh, d], bf16 when rounding, else fp32
  int q_out_dtype = PLUTO_HIP_BF16;
  CacheView cache;
  int length = 0, start_position = 0;
  int query_heads = 0, key_value_heads = 0, head_dim = 0, rotary_dim = 0;
  float epsilon = 1e-6f;
  bool round = true;
};

// Per-launch slice of a decode batch, passed by value as a kernel argument.
struct DecodeBatch {
  int count = 0;
  int sequence[kDecodeBatchMax];  // index of entry i in the full batch
  int positions[kDecodeBatchMax];
  void* keys[kDecodeBatchMax];
  void* values[kDecodeBatchMax];
  int block_start[kDecodeBatchMax + 1];  // prefix sum of split-K blocks
};

struct DecodePrepareArgs {
  const void* q_gate = nullptr;  // [batch, qh, 2, d]
  const void* k = nullptr;       // [batch, kh, d]
  const void* v = nullptr;
  int io_dtype = PLUTO_HIP_F32;
  const float* q_norm = nullptr;
  const float* k_norm = nullptr;
  void* q_out = nullptr;  // [batch, qh, d]
  int q_out_dtype = PLUTO_HIP_BF16;
  int cache_dtype = PLUTO_HIP_BF16;
  long long token_stride = 0, head_stride = 0;
  int query_heads = 0, key_value_heads = 0, head_dim = 0, rotary_dim = 0;
  float epsilon = 1e-6f, theta = 1e7f;
  bool round = true;
};

// Split-K block sizes of the decode step: a multiple of 64 up to 512 cache
// rows, or the size the fused kernel is specialised for at this head width.
// At head width 256 one workgroup occupies a compute unit alone, so nothing
// covers the time it spends starting up and handing over its partial results;
// blocks of 1024 rows halve that share (0.435 -> 0.412 ms at 32 sequences of
// 1024..32768 tokens, 24 / 4 heads).  At the narrower widths three workgroups
// share a compute unit and 512 rows measure best.
constexpr int decode_split_default(int head_dim) { return head_dim == 256 ? 1024 : 512; }
constexpr bool decode_split_valid(int head_dim, int split) {
  return split >= 64 && split % 64 == 0 &&
         (split <= 512 || split == decode_split_default(head_dim));
}

// The fused decode step (preparation of the new token, split-K attention over
// the cache, combine and gate in the workgroup that finishes a (sequence, kv
// head) last).
struct DecodeArgs {
  const void* q_gate = nullptr;  // [batch, qh, 2, d]
  const void* k = nullptr;       // [batch, kh, d]
  const void* v = nullptr;
  int io_dtype = PLUTO_HIP_F32;  // storage of q_gate, k, v and out
  const float* q_norm = nullptr;
  const float* k_norm = nullptr;
  void* out = nullptr;  // [batch, qh, d]
  long long token_stride = 0, head_stride = 0;  // of the bf16 caches
  int query_heads = 0, key_value_heads = 0, head_dim = 0, rotary_dim = 0;
  float epsilon = 1e-6f;
  int split_tokens = 512;
  float scale = 1.0f;
  // partial results of split-K block i (global index block_start[b] + j,
  // kv head g): o [block, kh, group, d], m and l [block, kh, group]
  float* part_o = nullptr;
  float* part_m = nullptr;
  float* part_l = nullptr;
  // one counter per (sequence, kv head) of the whole batch: zero when the
  // kernel starts, and zero again when it ends
  unsigned* arrivals = nullptr;
  long long block_base = 0;  // global index of this launch's first block
  // theta^(-2 f / rotary) for f < rotary / 2, evaluated on the host in FP64
  double inverse_frequency[128];
};

int launch_rope_table(hipStream_t stream, int start_position, int length,
                      int rotary_dim, float theta, bool round, float* cosines,
                      float* sines);
int launch_prefill_prepare(hipStream_t stream, const PrefillPrepareArgs& args);
int launch_decode_prepare(hipStream_t stream, const DecodePrepareArgs& args,
                          const DecodeBatch& batch);
bool decode_fast_supported(int head_dim, int group);
int launch_decode_fast(hipStream_t stream, const DecodeArgs& args,
                       const DecodeBatch& batch);
// Zeroes `count` arrival counters (a launch of its own: the fused kernel needs
// them zero, and leaves them zero).
// `always`: also when the test-support kernel mask has switched auxiliary kernels off
int launch_decode_clear(hipStream_t stream, unsigned* arrivals, int count, bool always = false);
// Two-pass probability rows (any dtype, any shape): row r of `rows` sees the
// first `first_visible + r` cache rows; output fp32 [query_heads, rows,
// row_width], zero beyond the visible prefix
// (AttentionProbabilitiesKernel, cached_attention_ops.cc:131-178; the probs
// tensor of ForwardKernel, qwen_attention.cc:68-119).
int launch_attention_probabilities(hipStream_t stream, const void* q, int q_dtype,
                                   const CacheView& cache, int query_heads,
                                   int key_value_heads, int head_dim, int rows,
                                   int first_visible, int row_width, float scale,
                                   float* probabilities);

// Pieces of the whole-sequence backward (gqa_backward.hip).
int launch_pack_heads(hipStream_t stream, const void* q, const void* k, const void* v, int dtype,
                      int length, int query_heads, int key_value_heads, int head_dim,
                      void* packed);
int launch_gate_backward(hipStream_t stream, const void* qg, const void* core, int core_dtype,
                         const float* dy, int length, int query_heads, int head_dim, bool round,
                         float* dc, float* dqg);
int launch_norm_rope_backward(hipStream_t stream, const void* input, const float* weight,
                              const float* packed_grad, const float* cosines, const float* sines,
                              int length, int heads, int query_heads, int head_dim, int rotary_dim,
                              int input_stride, float epsilon, bool key_mode, float* dx,
                              float* dv, float* parts);
int launch_reduce_norm(hipStream_t stream, const float* parts, long long rows, int head_dim,
                       float* partial, int chunks, float* dw);

}  // namespace pluto_hip
