// C ABI of Qwen grouped-query attention: validation, workspace carving and
// kernel selection for whole-sequence prefill and batched single-token decode.
#include <atomic>
#include <cmath>
#include <limits>
#include <mutex>

#include "attn_generic.h"
#include "flash_fwd_mfma.h"
#include "gqa.h"

// Fixed scratch of pluto_hip_gqa_decode_static: split-K partial results and
// the prepared queries of one decode call.  Every GPU the library runs on
// holds its own copy of the array until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress: kernels and copies
// take the per-device address kept in static_scratch_address.
constexpr size_t kStaticScratchBytes = PLUTO_HIP_GQA_DECODE_STATIC_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace pluto_hip {
bool force_generic();  // mha_capi.hip
namespace {

constexpr int kMaxDevices = 64;
std::atomic<void*> static_scratch_address[kMaxDevices];
std::mutex static_scratch_mutex;
// Set when a call on the fixed scratch returned an error after it had queued
// work: its kernels may leave arrival counters behind that are not zero, so
// the next call on that device clears them first.
std::atomic<bool> static_scratch_dirty[kMaxDevices];

// Device address of `scratch` on the calling thread's current device, looked
// up once per device.
int static_scratch(void** address, int* device_out = nullptr) {
  int device = 0;
  hipError_t error = hipGetDevice(&device);
  if (error != hipSuccess) return static_cast<int>(error);
  if (device < 0 || device >= kMaxDevices) return PLUTO_HIP_EUNSUPPORTED;
  void* known = static_scratch_address[device].load(std::memory_order_acquire);
  if (!known) {
    std::lock_guard<std::mutex> lock(static_scratch_mutex);
    known = static_scratch_address[device].load(std::memory_order_relaxed);
    if (!known) {
      error = hipGetSymbolAddress(&known, HIP_SYMBOL(scratch));
      if (error != hipSuccess) return static_cast<int>(error);
      if (!known) return static_cast<int>(hipErrorInvalidSymbol);
      static_scratch_address[device].store(known, std::memory_order_release);
    }
  }
  *address = known;
  if (device_out) *device_out = device;
  return 0;
}

// ValidateCachedAttention, parameter part (cached_attention_ops.cc:286-297).
int validate_params(const pluto_hip_attention_params* p) {
  if (!p) return PLUTO_HIP_EINVAL;
  const int int_max = std::numeric_limits<int>::max();
  if (p->query_heads <= 0 || p->key_value_heads <= 0 ||
      p->query_heads % p->key_value_heads != 0 || p->head_dim <= 0 ||
      p->head_dim > 256 || p->rotary_dim <= 0 || p->rotary_dim > p->head_dim ||
      p->rotary_dim % 2 != 0 || p->capacity <= 0 || p->capacity > int_max - 32 ||
      !std::isfinite(p->rope_theta) || p->rope_theta <= 0.0f ||
      !std::isfinite(p->rms_norm_epsilon) || p->rms_norm_epsilon <= 0.0f ||
      p->query_heads > int_max / (2 * p->head_dim) ||
      p->query_heads > int_max - p->key_value_heads)
    return PLUTO_HIP_EINVAL;
  return 0;
}

int validate_cache(const pluto_hip_kv_cache_view* c, const pluto_hip_attention_params* p) {
  if (!c || !c->keys || !c->values) return PLUTO_HIP_EINVAL;
  if (c->dtype != PLUTO_HIP_F32 && c->dtype != PLUTO_HIP_BF16) return PLUTO_HIP_EINVAL;
  if (c->token_stride < p->head_dim && c->head_stride < p->head_dim) return PLUTO_HIP_EINVAL;
  if (c->token_stride <= 0 || c->head_stride <= 0) return PLUTO_HIP_EINVAL;
  return 0;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

size_t element_bytes(int dtype) { return dtype == PLUTO_HIP_BF16 ? 2 : 4; }

struct PrefillLayout {
  size_t cosines, sines, queries, total;
};

PrefillLayout prefill_layout(const pluto_hip_attention_params* p, int length) {
  PrefillLayout l{};
  const size_t table = align_up(static_cast<size_t>(length) * (p->rotary_dim / 2) * 4, 256);
  l.cosines = 0;
  l.sines = table;
  l.queries = 2 * table;
  l.total = l.queries + align_up(static_cast<size_t>(length) * p->query_heads * p->head_dim *
                                     (p->round_to_bfloat16 ? 2 : 4),
                                 256);
  return l;
}

// Scratch of the whole-sequence backward.
struct PrefillBackwardLayout {
  size_t cosines, sines, queries, keys, values, packed, core, maxima, normalizers, dc, d_packed,
      q_parts, k_parts, partial, attention, total;
  size_t attention_bytes;
  int dtype;  // storage of the packed view and of the recomputed core
};
constexpr int kNormReduceChunks = 128;

PrefillBackwardLayout prefill_backward_layout(const pluto_hip_attention_params* p, int length,
                                              bool q_weight_grad, bool k_weight_grad) {
  PrefillBackwardLayout l{};
  const size_t T = static_cast<size_t>(length);
  const size_t qh = p->query_heads, kh = p->key_value_heads, d = p->head_dim;
  // bf16 storage (matrix-core kernels, bf16 tolerance) where those kernels
  // exist; everything else runs the FP32 kernels on FP32 storage.
  const bool flash = p->round_to_bfloat16 && (d == 64 || d == 128) && !force_generic();
  l.dtype = flash ? PLUTO_HIP_BF16 : PLUTO_HIP_F32;
  const size_t element = flash ? 2 : 4;
  size_t at = 0;
  auto take = [&](size_t bytes) {
    const size_t offset = at;
    at += align_up(bytes, 256);
    return offset;
  };
  l.cosines = take(T * (p->rotary_dim / 2) * 4);
  l.sines = take(T * (p->rotary_dim / 2) * 4);
  l.queries = take(T * qh * d * element);
  l.keys = take(T * kh * d * element);
  l.values = take(T * kh * d * element);
  l.packed = take(3 * T * qh * d * element);
  l.core = take(T * qh * d * element);
  l.maxima = take(T * qh * 4);
  l.normalizers = take(T * qh * 4);
  l.dc = take(T * qh * d * 4);
  l.d_packed = take(3 * T * qh * d * 4);
  l.q_parts = take(q_weight_grad ? T * qh * d * 4 : 0);
  l.k_parts = take(k_weight_grad ? T * kh * d * 4 : 0);
  l.partial = take((q_weight_grad || k_weight_grad) ? kNormReduceChunks * d * 4 : 0);
  l.attention_bytes = pluto_hip_mha_backward_workspace_bytes(
      l.dtype, length, length, p->query_heads, p->query_heads * p->head_dim);
  l.attention = take(l.attention_bytes);
  l.total = at;
  return l;
}

int split_or_default(int split_tokens, int head_dim) {
  return split_tokens == 0 ? decode_split_default(head_dim) : split_tokens;
}

long long decode_blocks(int batch, const int* positions, int split) {
  long long blocks = 0;
  for (int b = 0; b < batch; ++b) blocks += (static_cast<long long>(positions[b]) + split) / split;
  return blocks;
}

// What the forward pass can leave for the backward pass: the attention output
// before the gate (bf16 [length, qh * d]) and the two row statistics (fp32
// [qh, length] each), as the matrix-core backward kernels read them.
struct SavedLayout {
  size_t core, maxima, normalizers, total;
};
SavedLayout saved_layout(const pluto_hip_attention_params* p, int length) {
  SavedLayout l{};
  const size_t rows = static_cast<size_t>(length) * p->query_heads;
  l.core = 0;
  l.maxima = align_up(rows * p->head_dim * 2, 256);
  l.normalizers = l.maxima + align_up(rows * 4, 256);
  l.total = l.normalizers + align_up(rows * 4, 256);
  return l;
}
bool saved_supported(const pluto_hip_attention_params* p, int cache_dtype) {
  return p->round_to_bfloat16 && cache_dtype == PLUTO_HIP_BF16 &&
         (p->head_dim == 64 || p->head_dim == 128) && !force_generic();
}

}  // namespace
}  // namespace pluto_hip

using namespace pluto_hip;

extern "C" {

int pluto_hip_attention_params_validate(const pluto_hip_attention_params* p) {
  return validate_params(p);
}

size_t pluto_hip_gqa_prefill_workspace_bytes(const pluto_hip_attention_params* p, int length) {
  if (validate_params(p) != 0 || length <= 0) return 0;
  return prefill_layout(p, length).total;
}

size_t pluto_hip_gqa_prefill_saved_bytes(const pluto_hip_attention_params* p, int length,
                                         int cache_dtype) {
  if (validate_params(p) != 0 || length <= 0 || !saved_supported(p, cache_dtype)) return 0;
  return saved_layout(p, length).total;
}

int pluto_hip_gqa_prefill(void* stream, const pluto_hip_attention_params* p, int length,
                          int start_position, const void* qg, const void* k, const void* v,
                          const float* q_norm, const float* k_norm,
                          const pluto_hip_kv_cache_view* cache, void* out, float* lse,
                          void* saved, void* workspace, size_t workspace_bytes) {
  int status = validate_params(p);
  if (status != 0) return status;
  if (length <= 0 || start_position < 0) return PLUTO_HIP_EINVAL;
  if (!qg || !k || !v || !q_norm || !k_norm || !out) return PLUTO_HIP_EINVAL;
  status = validate_cache(cache, p);
  if (status != 0) return status;
  // cached_attention_ops.cc:318-320: appending beyond capacity fails first.
  if (static_cast<long long>(start_position) + length > p->capacity) return PLUTO_HIP_ERANGE;
  // the saved state describes a whole sequence attended from position 0
  if (saved && (start_position != 0 || !saved_supported(p, cache->dtype)))
    return PLUTO_HIP_EUNSUPPORTED;
  const PrefillLayout layout = prefill_layout(p, length);
  if (!workspace || workspace_bytes < layout.total) return PLUTO_HIP_EWORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  char* scratch = static_cast<char*>(workspace);
  float* cosines = reinterpret_cast<float*>(scratch + layout.cosines);
  float* sines = reinterpret_cast<float*>(scratch + layout.sines);
  void* queries = scratch + layout.queries;
  const bool round = p->round_to_bfloat16 != 0;
  const int qh = p->query_heads, kh = p->key_value_heads, d = p->head_dim;

  status = launch_rope_table(s, start_position, length, p->rotary_dim, p->rope_theta, round,
                             cosines, sines);
  if (status != 0) return status;
  PrefillPrepareArgs prep;
  prep.qg = qg;
  prep.k = k;
  prep.v = v;
  prep.q_norm = q_norm;
  prep.k_norm = k_norm;
  prep.cosines = cosines;
  prep.sines = sines;
  prep.q_out = queries;
  prep.q_out_dtype = round ? PLUTO_HIP_BF16 : PLUTO_HIP_F32;
  prep.cache = {cache->keys, cache->values, cache->dtype, cache->token_stride,
                cache->head_stride};
  prep.length = length;
  prep.start_position = start_position;
  prep.query_heads = qh;
  prep.key_value_heads = kh;
  prep.head_dim = d;
  prep.rotary_dim = p->rotary_dim;
  prep.epsilon = p->rms_norm_epsilon;
  prep.round = round;
  status = launch_prefill_prepare(s, prep);
  if (status != 0) return status;

  const float scale = 1.0f / std::sqrt(static_cast<float>(d));
  const uint16_t* gate = static_cast<const uint16_t*>(qg) + d;
  if (round && cache->dtype == PLUTO_HIP_BF16 && !force_generic()) {
    FlashForwardArgs f;
    f.q = static_cast<const uint16_t*>(queries);
    f.q_row_stride = 1LL * qh * d;
    f.q_head_stride = d;
    f.k = static_cast<const uint16_t*>(cache->keys);
    f.v = static_cast<const uint16_t*>(cache->values);
    f.k_row_stride = f.v_row_stride = cache->token_stride;
    f.k_head_stride = f.v_head_stride = cache->head_stride;
    f.out = static_cast<uint16_t*>(out);
    f.o_row_stride = 1LL * qh * d;
    f.o_head_stride = d;
    f.gate = gate;
    f.gate_row_stride = 2LL * qh * d;
    f.gate_head_stride = 2LL * d;
    f.lse = lse;
    if (saved) {
      const SavedLayout sl = saved_layout(p, length);
      f.core = reinterpret_cast<uint16_t*>(static_cast<char*>(saved) + sl.core);
      f.maxima = reinterpret_cast<float*>(static_cast<char*>(saved) + sl.maxima);
      f.normalizers = reinterpret_cast<float*>(static_cast<char*>(saved) + sl.normalizers);
    }
    f.q_rows = length;
    f.kv_rows = start_position + length;
    f.start_position = start_position;
    f.query_heads = qh;
    f.group = qh / kh;
    f.scale = scale;
    if (flash_forward_supported(f, d)) {
      note_path(PLUTO_HIP_PATH_FLASH);
      return launch_flash_forward(s, f, d, 1);
    }
    if (saved) return PLUTO_HIP_EUNSUPPORTED;
  }
  GenericForwardArgs a;
  a.q = {queries, 0, 1LL * qh * d, d, prep.q_out_dtype};
  a.k = {cache->keys, 0, cache->token_stride, cache->head_stride, cache->dtype};
  a.v = {cache->values, 0, cache->token_stride, cache->head_stride, cache->dtype};
  a.gate = {gate, 0, 2LL * qh * d, 2LL * d, PLUTO_HIP_BF16};
  a.out = out;
  a.o_row_stride = 1LL * qh * d;
  a.o_head_stride = d;
  a.o_dtype = PLUTO_HIP_BF16;
  a.lse = lse;
  a.q_rows = length;
  a.kv_rows = start_position + length;
  a.start_position = start_position;
  a.query_heads = qh;
  a.group = qh / kh;
  a.head_dim = d;
  a.scale = scale;
  a.round_to_bf16 = round;
  note_path(PLUTO_HIP_PATH_GENERIC);
  return launch_generic_forward(s, a, 1);
}

size_t pluto_hip_gqa_prefill_backward_workspace_bytes(const pluto_hip_attention_params* p,
                                                      int length, int q_weight_grad,
                                                      int k_weight_grad) {
  if (validate_params(p) != 0 || length <= 0) return 0;
  return prefill_backward_layout(p, length, q_weight_grad != 0, k_weight_grad != 0).total;
}

int pluto_hip_gqa_prefill_backward(void* stream, const pluto_hip_attention_params* p, int length,
                                   const void* qg, const void* k, const void* v,
                                   const float* q_norm, const float* k_norm, const float* dy,
                                   const void* saved, float* dqg, float* dk, float* dv,
                                   float* dq_norm, float* dk_norm, void* workspace,
                                   size_t workspace_bytes) {
  int status = validate_params(p);
  if (status != 0) return status;
  if (length <= 0) return PLUTO_HIP_EINVAL;
  if (!qg || !k || !v || !q_norm || !k_norm || !dy || !dqg || !dk || !dv) return PLUTO_HIP_EINVAL;
  const PrefillBackwardLayout l = prefill_backward_layout(p, length, dq_norm != nullptr,
                                                          dk_norm != nullptr);
  if (l.attention_bytes == 0) return PLUTO_HIP_EINVAL;
  if (!workspace || workspace_bytes < l.total) return PLUTO_HIP_EWORKSPACE;
  if (saved && l.dtype != PLUTO_HIP_BF16) return PLUTO_HIP_EUNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  char* scratch = static_cast<char*>(workspace);
  float* cosines = reinterpret_cast<float*>(scratch + l.cosines);
  float* sines = reinterpret_cast<float*>(scratch + l.sines);
  const bool round = p->round_to_bfloat16 != 0;
  const int qh = p->query_heads, kh = p->key_value_heads, d = p->head_dim;
  const int E = qh * d;

  // Recompute what the forward pass derived from the inputs: normalised,
  // rotated q and k (PrepareKernel, qwen_attention.cc:30-63), then -- unless
  // the forward pass saved them -- the attention core with its row statistics.
  status = launch_rope_table(s, 0, length, p->rotary_dim, p->rope_theta, round, cosines, sines);
  if (status != 0) return status;
  PrefillPrepareArgs prep;
  prep.qg = qg;
  prep.k = k;
  prep.v = v;
  prep.q_norm = q_norm;
  prep.k_norm = k_norm;
  prep.cosines = cosines;
  prep.sines = sines;
  prep.q_out = scratch + l.queries;
  prep.q_out_dtype = l.dtype;
  prep.cache = {scratch + l.keys, scratch + l.values, l.dtype, 1LL * kh * d, d};
  prep.length = length;
  prep.start_position = 0;
  prep.query_heads = qh;
  prep.key_value_heads = kh;
  prep.head_dim = d;
  prep.rotary_dim = p->rotary_dim;
  prep.epsilon = p->rms_norm_epsilon;
  prep.round = round;
  status = launch_prefill_prepare(s, prep);
  if (status != 0) return status;
  status = launch_pack_heads(s, scratch + l.queries, scratch + l.keys, scratch + l.values, l.dtype,
                             length, qh, kh, d, scratch + l.packed);
  if (status != 0) return status;
  const void* core = scratch + l.core;
  const float* maxima = reinterpret_cast<const float*>(scratch + l.maxima);
  const float* normalizers = reinterpret_cast<const float*>(scratch + l.normalizers);
  if (saved) {
    const SavedLayout sl = saved_layout(p, length);
    const char* base = static_cast<const char*>(saved);
    core = base + sl.core;
    maxima = reinterpret_cast<const float*>(base + sl.maxima);
    normalizers = reinterpret_cast<const float*>(base + sl.normalizers);
  } else {
    status = pluto_hip_mha_forward(stream, l.dtype, scratch + l.packed, length, length, qh, E,
                                   scratch + l.core,
                                   reinterpret_cast<float*>(scratch + l.maxima),
                                   reinterpret_cast<float*>(scratch + l.normalizers));
    if (status != 0) return status;
  }

  float* dc = reinterpret_cast<float*>(scratch + l.dc);
  status = launch_gate_backward(s, qg, core, l.dtype, dy, length, qh, d, round, dc, dqg);
  if (status != 0) return status;
  float* d_packed = reinterpret_cast<float*>(scratch + l.d_packed);
  status = pluto_hip_mha_backward(stream, l.dtype, scratch + l.packed, core, dc, maxima,
                                  normalizers, length, length, qh, E, d_packed,
                                  scratch + l.attention, l.attention_bytes);
  if (status != 0) return status;

  float* q_parts = dq_norm ? reinterpret_cast<float*>(scratch + l.q_parts) : nullptr;
  float* k_parts = dk_norm ? reinterpret_cast<float*>(scratch + l.k_parts) : nullptr;
  status = launch_norm_rope_backward(s, qg, q_norm, d_packed, cosines, sines, length, qh, qh, d,
                                     p->rotary_dim, 2 * d, p->rms_norm_epsilon, false, dqg, nullptr,
                                     q_parts);
  if (status != 0) return status;
  status = launch_norm_rope_backward(s, k, k_norm, d_packed, cosines, sines, length, kh, qh, d,
                                     p->rotary_dim, d, p->rms_norm_epsilon, true, dk, dv, k_parts);
  if (status != 0) return status;
  float* partial = reinterpret_cast<float*>(scratch + l.partial);
  if (dq_norm) {
    status = launch_reduce_norm(s, q_parts, 1LL * length * qh, d, partial, kNormReduceChunks,
                                dq_norm);
    if (status != 0) return status;
  }
  if (dk_norm) {
    status = launch_reduce_norm(s, k_parts, 1LL * length * kh, d, partial, kNormReduceChunks,
                                dk_norm);
    if (status != 0) return status;
  }
  return 0;
}

int pluto_hip_gqa_prefill_probabilities(void* stream, const pluto_hip_attention_params* p,
                                        int length, int start_position,
                                        const pluto_hip_kv_cache_view* cache,
                                        const void* workspace, size_t workspace_bytes,
                                        float* probabilities) {
  int status = validate_params(p);
  if (status != 0) return status;
  if (length <= 0 || start_position < 0 || !probabilities) return PLUTO_HIP_EINVAL;
  status = validate_cache(cache, p);
  if (status != 0) return status;
  if (static_cast<long long>(start_position) + length > p->capacity) return PLUTO_HIP_ERANGE;
  const PrefillLayout layout = prefill_layout(p, length);
  if (!workspace || workspace_bytes < layout.total) return PLUTO_HIP_EWORKSPACE;
  const CacheView view{cache->keys, cache->values, cache->dtype, cache->token_stride,
                       cache->head_stride};
  const float scale = 1.0f / std::sqrt(static_cast<float>(p->head_dim));
  const char* queries = static_cast<const char*>(workspace) + layout.queries;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // The grid's second dimension holds at most 65535 rows per launch.
  const int width = start_position + length;
  if (length > 65535) return PLUTO_HIP_EUNSUPPORTED;
  return launch_attention_probabilities(
      s, queries, p->round_to_bfloat16 ? PLUTO_HIP_BF16 : PLUTO_HIP_F32, view, p->query_heads,
      p->key_value_heads, p->head_dim, length, start_position + 1, width, scale, probabilities);
}

// Scratch of a decode call: arrival counters (one per sequence and kv head),
// prepared queries (read by the any-shape kernels and the probabilities pass),
// split-K partial results.
struct DecodeLayout {
  size_t arrivals, queries, part_o, part_m, part_l, total;
};
static DecodeLayout decode_layout(const pluto_hip_attention_params* p, int batch, long long blocks,
                                  size_t arrivals_bytes) {
  DecodeLayout l{};
  const size_t heads = static_cast<size_t>(p->query_heads);
  size_t at = 0;
  auto take = [&](size_t bytes) {
    const size_t offset = at;
    at += align_up(bytes, 256);
    return offset;
  };
  l.arrivals = take(arrivals_bytes);
  l.queries = take(static_cast<size_t>(batch) * heads * p->head_dim * 4);
  l.part_o = take(static_cast<size_t>(blocks) * heads * p->head_dim * 4);
  l.part_m = take(static_cast<size_t>(blocks) * heads * 4);
  l.part_l = take(static_cast<size_t>(blocks) * heads * 4);
  l.total = at;
  return l;
}

size_t pluto_hip_gqa_decode_workspace_bytes(const pluto_hip_attention_params* p, int batch,
                                            const int* positions, int split_tokens) {
  if (validate_params(p) != 0 || batch <= 0 || !positions) return 0;
  const int split = split_or_default(split_tokens, p ? p->head_dim : 0);
  if (!decode_split_valid(p->head_dim, split)) return 0;
  for (int b = 0; b < batch; ++b)
    if (positions[b] < 0) return 0;
  const long long blocks = decode_blocks(batch, positions, split);
  return decode_layout(p, batch, blocks,
                       static_cast<size_t>(batch) * p->key_value_heads * sizeof(unsigned))
      .total;
}

// Argument checks of the decode entry points; everything is rejected before
// any work is queued.
static int decode_check(const pluto_hip_attention_params* p, int batch, int io_dtype,
                        const void* q_gate, const void* k, const void* v, const float* q_norm,
                        const float* k_norm, const int* positions,
                        const pluto_hip_kv_cache_view* caches, const void* out, int split) {
  int status = validate_params(p);
  if (status != 0) return status;
  if (batch <= 0 || (io_dtype != PLUTO_HIP_F32 && io_dtype != PLUTO_HIP_BF16))
    return PLUTO_HIP_EINVAL;
  // cached_attention_ops.cc:314-317: null pointers are rejected before any work.
  if (!q_gate || !k || !v || !q_norm || !k_norm || !out || !positions || !caches)
    return PLUTO_HIP_EINVAL;
  if (!decode_split_valid(p->head_dim, split)) return PLUTO_HIP_EINVAL;
  for (int b = 0; b < batch; ++b) {
    status = validate_cache(&caches[b], p);
    if (status != 0) return status;
    if (caches[b].dtype != caches[0].dtype || caches[b].token_stride != caches[0].token_stride ||
        caches[b].head_stride != caches[0].head_stride)
      return PLUTO_HIP_EINVAL;
    if (positions[b] < 0) return PLUTO_HIP_EINVAL;
  }
  for (int b = 0; b < batch; ++b)  // cached_attention_ops.cc:318-320
    if (positions[b] >= p->capacity) return PLUTO_HIP_ERANGE;
  return 0;
}

// The fixed scratch starts with room for this many arrival counters; they are
// zero when the library is loaded and every call that runs to its end leaves
// them zero.  pluto_hip_gqa_decode_static_reset re-zeroes them.
constexpr size_t kStaticArrivalBytes = 16384;

static int decode_run(void* stream, const pluto_hip_attention_params* p, int batch, int io_dtype,
                      const void* q_gate, const void* k, const void* v, const float* q_norm,
                      const float* k_norm, const int* positions,
                      const pluto_hip_kv_cache_view* caches, void* out,
                      float* const* probabilities, int split, void* workspace,
                      const DecodeLayout& layout, bool clear_arrivals);

int pluto_hip_gqa_decode(void* stream, const pluto_hip_attention_params* p, int batch,
                         int io_dtype, const void* q_gate, const void* k, const void* v,
                         const float* q_norm, const float* k_norm, const int* positions,
                         const pluto_hip_kv_cache_view* caches, void* out,
                         float* const* probabilities, int split_tokens, void* workspace,
                         size_t workspace_bytes) {
  const int split = split_or_default(split_tokens, p ? p->head_dim : 0);
  const int status =
      decode_check(p, batch, io_dtype, q_gate, k, v, q_norm, k_norm, positions, caches, out, split);
  if (status != 0) return status;
  const DecodeLayout layout =
      decode_layout(p, batch, decode_blocks(batch, positions, split),
                    static_cast<size_t>(batch) * p->key_value_heads * sizeof(unsigned));
  if (!workspace || workspace_bytes < layout.total) return PLUTO_HIP_EWORKSPACE;
  // whatever the workspace held: the counters are cleared by a launch of their own
  return decode_run(stream, p, batch, io_dtype, q_gate, k, v, q_norm, k_norm, positions, caches,
                    out, probabilities, split, workspace, layout, true);
}

size_t pluto_hip_gqa_decode_static_bytes(void) { return kStaticScratchBytes; }

int pluto_hip_gqa_decode_static_prepare(void) {
  void* address = nullptr;
  return static_scratch(&address);
}

int pluto_hip_gqa_decode_static(void* stream, const pluto_hip_attention_params* p, int batch,
                                int io_dtype, const void* q_gate, const void* k, const void* v,
                                const float* q_norm, const float* k_norm, const int* positions,
                                const pluto_hip_kv_cache_view* caches, void* out,
                                float* const* probabilities, int split_tokens) {
  const int split = split_or_default(split_tokens, p ? p->head_dim : 0);
  int status =
      decode_check(p, batch, io_dtype, q_gate, k, v, q_norm, k_norm, positions, caches, out, split);
  if (status != 0) return status;
  if (static_cast<size_t>(batch) * p->key_value_heads * sizeof(unsigned) > kStaticArrivalBytes)
    return PLUTO_HIP_ELIMIT;
  const DecodeLayout layout =
      decode_layout(p, batch, decode_blocks(batch, positions, split), kStaticArrivalBytes);
  if (layout.total > kStaticScratchBytes) return PLUTO_HIP_ELIMIT;
  void* address = nullptr;
  int device = 0;
  status = static_scratch(&address, &device);
  if (status != 0) return status;
  // The counters at the head of the array are zero since the library was
  // loaded and every call that ran to its end left them zero: nothing to
  // clear, one launch.  A call that failed after it had queued work may have
  // left some behind; the first call after it clears them all.
  if (static_scratch_dirty[device].exchange(false, std::memory_order_acq_rel)) {
    status = launch_decode_clear(static_cast<hipStream_t>(stream),
                                 static_cast<unsigned*>(address),
                                 static_cast<int>(kStaticArrivalBytes / sizeof(unsigned)), true);
    if (status != 0) {
      static_scratch_dirty[device].store(true, std::memory_order_release);
      return status;
    }
  }
  status = decode_run(stream, p, batch, io_dtype, q_gate, k, v, q_norm, k_norm, positions, caches,
                      out, probabilities, split, address, layout, false);
  if (status != 0) static_scratch_dirty[device].store(true, std::memory_order_release);
  return status;
}

int pluto_hip_gqa_decode_static_reset(void* stream) {
  void* address = nullptr;
  int device = 0;
  const int status = static_scratch(&address, &device);
  if (status != 0) return status;
  // a fill kernel, not a memset: callers may record this into a graph
  const int cleared = launch_decode_clear(
      static_cast<hipStream_t>(stream), static_cast<unsigned*>(address),
      static_cast<int>(kStaticArrivalBytes / sizeof(unsigned)), true);
  if (cleared == 0) static_scratch_dirty[device].store(false, std::memory_order_release);
  return cleared;
}

static int decode_run(void* stream, const pluto_hip_attention_params* p, int batch, int io_dtype,
                      const void* q_gate, const void* k, const void* v, const float* q_norm,
                      const float* k_norm, const int* positions,
                      const pluto_hip_kv_cache_view* caches, void* out,
                      float* const* probabilities, int split, void* workspace,
                      const DecodeLayout& layout, bool clear_arrivals) {
  int status = 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int qh = p->query_heads, kh = p->key_value_heads, d = p->head_dim;
  const int group = qh / kh;
  const bool round = p->round_to_bfloat16 != 0;
  char* area = static_cast<char*>(workspace);
  void* queries = area + layout.queries;

  const pluto_hip_kv_cache_view& c0 = caches[0];
  bool fast = round && c0.dtype == PLUTO_HIP_BF16 && decode_fast_supported(d, group) &&
              p->rotary_dim / 2 <= 128 && !force_generic() && c0.token_stride % 8 == 0 &&
              c0.head_stride % 8 == 0;
  for (int b = 0; b < batch && fast; ++b)
    fast = aligned16(caches[b].keys) && aligned16(caches[b].values);
  const int q_dtype = round ? PLUTO_HIP_BF16 : PLUTO_HIP_F32;
  const float scale = 1.0f / std::sqrt(static_cast<float>(d));
  const size_t io_bytes = element_bytes(io_dtype);
  note_path(fast ? PLUTO_HIP_PATH_SPLIT_K : PLUTO_HIP_PATH_GENERIC);

  if (fast && clear_arrivals) {
    status = launch_decode_clear(s, reinterpret_cast<unsigned*>(area + layout.arrivals),
                                 batch * kh);
    if (status != 0) return status;
  }
  long long block_base = 0;
  for (int first = 0; first < batch; first += kDecodeBatchMax) {
    DecodeBatch slice;
    slice.count = batch - first < kDecodeBatchMax ? batch - first : kDecodeBatchMax;
    slice.block_start[0] = 0;
    // Long sequences first: the workgroups that combine a sequence's blocks then
    // run while shorter sequences are still streaming, not after everything
    // else (insertion sort of at most kDecodeBatchMax entries, on the stack).
    int order[kDecodeBatchMax];
    for (int i = 0; i < slice.count; ++i) {
      int at = i;
      while (at > 0 && positions[order[at - 1]] < positions[first + i]) {
        order[at] = order[at - 1];
        --at;
      }
      order[at] = first + i;
    }
    for (int i = 0; i < slice.count; ++i) {
      const int b = order[i];
      slice.sequence[i] = b;
      slice.positions[i] = positions[b];
      slice.keys[i] = caches[b].keys;
      slice.values[i] = caches[b].values;
      slice.block_start[i + 1] = slice.block_start[i] + (positions[b] + split) / split;
    }
    if (!fast || probabilities) {
      // the any-shape kernels and the probabilities pass read prepared queries
      // (and the appended row) from memory
      DecodePrepareArgs prep;
      prep.q_gate = q_gate;
      prep.k = k;
      prep.v = v;
      prep.io_dtype = io_dtype;
      prep.q_norm = q_norm;
      prep.k_norm = k_norm;
      prep.q_out = queries;
      prep.q_out_dtype = q_dtype;
      prep.cache_dtype = c0.dtype;
      prep.token_stride = c0.token_stride;
      prep.head_stride = c0.head_stride;
      prep.query_heads = qh;
      prep.key_value_heads = kh;
      prep.head_dim = d;
      prep.rotary_dim = p->rotary_dim;
      prep.epsilon = p->rms_norm_epsilon;
      prep.theta = p->rope_theta;
      prep.round = round;
      status = launch_decode_prepare(s, prep, slice);
      if (status != 0) return status;
    }
    if (fast) {
      DecodeArgs a;
      a.q_gate = q_gate;
      a.k = k;
      a.v = v;
      a.io_dtype = io_dtype;
      a.q_norm = q_norm;
      a.k_norm = k_norm;
      a.out = out;
      a.token_stride = c0.token_stride;
      a.head_stride = c0.head_stride;
      a.query_heads = qh;
      a.key_value_heads = kh;
      a.head_dim = d;
      a.rotary_dim = p->rotary_dim;
      a.epsilon = p->rms_norm_epsilon;
      a.split_tokens = split;
      a.scale = scale;
      a.part_o = reinterpret_cast<float*>(area + layout.part_o);
      a.part_m = reinterpret_cast<float*>(area + layout.part_m);
      a.part_l = reinterpret_cast<float*>(area + layout.part_l);
      a.arrivals = reinterpret_cast<unsigned*>(area + layout.arrivals);
      a.block_base = block_base;
      // the scalar specification's frequency, in FP64
      // (cached_attention_ops_test.cc:66-67)
      for (int f = 0; f < p->rotary_dim / 2; ++f)
        a.inverse_frequency[f] =
            std::pow(static_cast<double>(p->rope_theta), -2.0 * f / p->rotary_dim);
      status = launch_decode_fast(s, a, slice);
      if (status != 0) return status;
    } else {
      for (int i = 0; i < slice.count; ++i) {
        const int b = slice.sequence[i];
        GenericForwardArgs a;
        const char* qbase = static_cast<const char*>(queries) +
                            static_cast<size_t>(b) * qh * d * element_bytes(q_dtype);
        a.q = {qbase, 0, 1LL * qh * d, d, q_dtype};
        a.k = {caches[b].keys, 0, c0.token_stride, c0.head_stride, c0.dtype};
        a.v = {caches[b].values, 0, c0.token_stride, c0.head_stride, c0.dtype};
        const char* gbase = static_cast<const char*>(q_gate) +
                            (static_cast<size_t>(b) * qh * 2 * d + d) * io_bytes;
        a.gate = {gbase, 0, 2LL * qh * d, 2LL * d, io_dtype};
        a.out = static_cast<char*>(out) + static_cast<size_t>(b) * qh * d * io_bytes;
        a.o_row_stride = 1LL * qh * d;
        a.o_head_stride = d;
        a.o_dtype = io_dtype;
        a.q_rows = 1;
        a.kv_rows = positions[b] + 1;
        a.start_position = positions[b];
        a.query_heads = qh;
        a.group = group;
        a.head_dim = d;
        a.scale = scale;
        a.round_to_bf16 = round;
        status = launch_generic_forward(s, a, 1);
        if (status != 0) return status;
      }
    }
    if (probabilities) {
      for (int i = 0; i < slice.count; ++i) {
        const int b = slice.sequence[i];
        if (!probabilities[b]) continue;
        const char* qbase = static_cast<const char*>(queries) +
                            static_cast<size_t>(b) * qh * d * element_bytes(q_dtype);
        const CacheView view{caches[b].keys, caches[b].values, c0.dtype, c0.token_stride,
                             c0.head_stride};
        status = launch_attention_probabilities(s, qbase, q_dtype, view, qh, kh, d, 1,
                                                positions[b] + 1, positions[b] + 1, scale,
                                                probabilities[b]);
        if (status != 0) return status;
      }
    }
    block_base += slice.block_start[slice.count];
  }
  return 0;
}

}  // extern "C"
