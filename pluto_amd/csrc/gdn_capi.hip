// C ABI of the gated delta-net scan.
#include <cmath>

#include "gdn.h"

namespace pluto_hip {
bool force_generic();  // mha_capi.hip
namespace {

// DeltaNetState::Create (cached_attention_ops.cc:376-383) /
// SequenceDeltaNetLayer::Create (sequence_delta_net.cc:404-411) limits.
int validate_delta(const pluto_hip_delta_params* p) {
  if (!p) return PLUTO_HIP_EINVAL;
  if (p->key_heads <= 0 || p->value_heads <= 0 || p->value_heads % p->key_heads != 0 ||
      p->key_head_dim <= 0 || p->key_head_dim > 128 || p->value_head_dim <= 0 ||
      p->value_head_dim > 256 || p->conv_kernel_dim <= 0 || p->conv_kernel_dim > 32 ||
      !std::isfinite(p->rms_norm_epsilon) || p->rms_norm_epsilon <= 0.0f)
    return PLUTO_HIP_EINVAL;
  return 0;
}

GdnArgs make_args(const pluto_hip_delta_params* p, int batch, int length, const void* q,
                  const void* k, const void* v, const float* log_decay, const float* beta,
                  int normalize_qk, float q_scale, float* state) {
  GdnArgs a;
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k);
  a.v = static_cast<const uint16_t*>(v);
  a.q_token_stride = a.k_token_stride = 1LL * p->key_heads * p->key_head_dim;
  a.v_token_stride = 1LL * p->value_heads * p->value_head_dim;
  a.log_decay = log_decay;
  a.beta = beta;
  a.state = state;
  a.batch = batch;
  a.length = length;
  a.key_heads = p->key_heads;
  a.value_heads = p->value_heads;
  a.key_dim = p->key_head_dim;
  a.value_dim = p->value_head_dim;
  a.normalize_qk = normalize_qk;
  a.round_output = p->round_to_bfloat16;
  a.q_scale = q_scale;
  return a;
}

struct LayerLayout {
  size_t post, log_decay, beta, core, scan, total;
};

size_t chunk_scratch_bytes(const pluto_hip_delta_params* p, int batch, int length) {
  if (p->key_head_dim != 128 || p->value_head_dim != 128) return 0;
  const size_t chunks = (static_cast<size_t>(length) + 63) / 64;
  return static_cast<size_t>(batch) * p->value_heads * chunks * kGdnChunkBytes;
}

LayerLayout layer_layout(const pluto_hip_delta_params* p, int batch, int length) {
  const size_t tokens = static_cast<size_t>(batch) * length;
  const size_t channels = 2 * static_cast<size_t>(p->key_heads) * p->key_head_dim +
                          static_cast<size_t>(p->value_heads) * p->value_head_dim;
  const size_t element = p->round_to_bfloat16 ? 2 : 4;
  LayerLayout l{};
  l.post = 0;
  l.log_decay = align_up(tokens * channels * element, 256);
  l.beta = l.log_decay + align_up(tokens * p->value_heads * 4, 256);
  l.core = l.beta + align_up(tokens * p->value_heads * 4, 256);
  l.scan = l.core + align_up(tokens * p->value_heads * p->value_head_dim * element, 256);
  l.total = l.scan + (p->round_to_bfloat16 ? chunk_scratch_bytes(p, batch, length) : 0) + 256;
  return l;
}

}  // namespace
}  // namespace pluto_hip

using namespace pluto_hip;

extern "C" {

size_t pluto_hip_gdn_scan_workspace_bytes(const pluto_hip_delta_params* p, int batch,
                                          int length, int chunk) {
  if (validate_delta(p) != 0 || batch <= 0 || length <= 0) return 0;
  if (chunk != 0 && chunk != 64) return 0;
  if (p->key_head_dim != 128 || p->value_head_dim != 128) return 0;
  const size_t chunks = (static_cast<size_t>(length) + 63) / 64;
  return static_cast<size_t>(batch) * p->value_heads * chunks * kGdnChunkBytes;
}

int pluto_hip_gdn_scan(void* stream, const pluto_hip_delta_params* p, int batch, int length,
                       int chunk, const void* q, const void* k, const void* v,
                       const float* log_decay, const float* beta, int normalize_qk,
                       float q_scale, float* state, void* out, void* workspace,
                       size_t workspace_bytes) {
  int status = validate_delta(p);
  if (status != 0) return status;
  if (batch <= 0 || length <= 0) return PLUTO_HIP_EINVAL;
  if (chunk != 0 && chunk != 64) return PLUTO_HIP_EUNSUPPORTED;
  if (!q || !k || !v || !log_decay || !beta || !state || !out) return PLUTO_HIP_EINVAL;
  GdnArgs a = make_args(p, batch, length, q, k, v, log_decay, beta, normalize_qk, q_scale, state);
  a.out = static_cast<uint16_t*>(out);
  a.out_any = out;
  a.workspace = static_cast<char*>(workspace);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!force_generic() && workspace != nullptr && gdn_chunked_supported(a, 64)) {
    const size_t needed = pluto_hip_gdn_scan_workspace_bytes(p, batch, length, 64);
    if (workspace_bytes < needed) return PLUTO_HIP_EWORKSPACE;
    note_path(PLUTO_HIP_PATH_CHUNKED);
    return launch_gdn_chunked(s, a);
  }
  note_path(PLUTO_HIP_PATH_RECURRENCE);
  return launch_gdn_recurrence(s, a, PLUTO_HIP_BF16);
}

int pluto_hip_gdn_recurrence(void* stream, const pluto_hip_delta_params* p, int batch,
                             int length, const void* q, const void* k, const void* v,
                             const float* log_decay, const float* beta, int normalize_qk,
                             float q_scale, float* state, void* out, int out_dtype) {
  int status = validate_delta(p);
  if (status != 0) return status;
  if (batch <= 0 || length <= 0) return PLUTO_HIP_EINVAL;
  if (out_dtype != PLUTO_HIP_F32 && out_dtype != PLUTO_HIP_BF16) return PLUTO_HIP_EINVAL;
  if (!q || !k || !v || !log_decay || !beta || !state || !out) return PLUTO_HIP_EINVAL;
  GdnArgs a = make_args(p, batch, length, q, k, v, log_decay, beta, normalize_qk, q_scale, state);
  a.out_any = out;
  return launch_gdn_recurrence(static_cast<hipStream_t>(stream), a, out_dtype);
}

size_t pluto_hip_gdn_layer_workspace_bytes(const pluto_hip_delta_params* p, int batch,
                                           int length) {
  if (validate_delta(p) != 0 || batch <= 0 || length <= 0) return 0;
  return layer_layout(p, batch, length).total;
}

int pluto_hip_gdn_layer_forward(void* stream, const pluto_hip_delta_params* p, int batch,
                                int length, const void* qkv, const void* z, const void* a,
                                const void* b, const float* conv_weight, const float* a_log,
                                const float* dt_bias, const float* norm, float* state,
                                void* out, void* workspace, size_t workspace_bytes) {
  int status = validate_delta(p);
  if (status != 0) return status;
  if (batch <= 0 || length <= 0) return PLUTO_HIP_EINVAL;
  if (!qkv || !z || !a || !b || !conv_weight || !a_log || !dt_bias || !norm || !state || !out)
    return PLUTO_HIP_EINVAL;
  const LayerLayout layout = layer_layout(p, batch, length);
  if (!workspace || workspace_bytes < layout.total) return PLUTO_HIP_EWORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  char* scratch = static_cast<char*>(workspace);
  const bool round = p->round_to_bfloat16 != 0;
  const int mid_dtype = round ? PLUTO_HIP_BF16 : PLUTO_HIP_F32;
  const int kh = p->key_heads, vh = p->value_heads, kd = p->key_head_dim, vd = p->value_head_dim;
  const int channels = 2 * kh * kd + vh * vd;
  const long long tokens = static_cast<long long>(batch) * length;
  void* post = scratch + layout.post;
  float* log_decay = reinterpret_cast<float*>(scratch + layout.log_decay);
  float* beta = reinterpret_cast<float*>(scratch + layout.beta);
  void* core = scratch + layout.core;
  status = launch_gdn_conv_sequence(s, qkv, PLUTO_HIP_BF16, conv_weight, batch, length, channels,
                                    p->conv_kernel_dim, round, post, mid_dtype);
  if (status != 0) return status;
  status = launch_gdn_gates(s, a, b, PLUTO_HIP_BF16, a_log, dt_bias, tokens, vh, round,
                            log_decay, beta);
  if (status != 0) return status;
  const size_t element = round ? 2 : 4;
  GdnArgs g;
  g.q = static_cast<const uint16_t*>(post);
  g.k = reinterpret_cast<const uint16_t*>(static_cast<char*>(post) + element * kh * kd);
  g.v = reinterpret_cast<const uint16_t*>(static_cast<char*>(post) + element * 2 * kh * kd);
  g.q_token_stride = g.k_token_stride = g.v_token_stride = channels;
  g.in_dtype = mid_dtype;
  g.log_decay = log_decay;
  g.beta = beta;
  g.state = state;
  g.out = static_cast<uint16_t*>(core);
  g.out_any = core;
  g.workspace = scratch + layout.scan;
  g.batch = batch;
  g.length = length;
  g.key_heads = kh;
  g.value_heads = vh;
  g.key_dim = kd;
  g.value_dim = vd;
  g.normalize_qk = 1;  // sequence_delta_net.cc:84-85
  g.round_output = round;
  g.q_scale = 1.0f / std::sqrt(static_cast<float>(kd));
  const bool chunked = round && !force_generic() && gdn_chunked_supported(g, 64);
  note_path(chunked ? PLUTO_HIP_PATH_CHUNKED : PLUTO_HIP_PATH_RECURRENCE);
  if (chunked)
    status = launch_gdn_chunked(s, g);
  else
    status = launch_gdn_recurrence(s, g, mid_dtype);
  if (status != 0) return status;
  return launch_gdn_output(s, core, mid_dtype, z, PLUTO_HIP_BF16, norm, tokens * vh, vd,
                           p->rms_norm_epsilon, round, out, PLUTO_HIP_BF16);
}

size_t pluto_hip_gdn_layer_backward_workspace_bytes(const pluto_hip_delta_params* p, int length,
                                                    int norm_grad) {
  if (validate_delta(p) != 0 || length <= 0 || length > 65535) return 0;
  return gdn_backward_workspace_bytes(p, length, norm_grad != 0);
}

int pluto_hip_gdn_layer_backward(void* stream, const pluto_hip_delta_params* p, int batch,
                                 int length, const void* qkv, const void* z, const void* a,
                                 const void* b, const float* conv_weight, const float* a_log,
                                 const float* dt_bias, const float* norm, const float* dy,
                                 float* dqkv, float* dz, float* da, float* db,
                                 float* d_conv_weight, float* d_a_log, float* d_dt_bias,
                                 float* d_norm, void* workspace, size_t workspace_bytes) {
  int status = validate_delta(p);
  if (status != 0) return status;
  // the q/k gather runs one grid row per token
  if (batch <= 0 || length <= 0 || length > 65535) return PLUTO_HIP_EINVAL;
  if (!qkv || !z || !a || !b || !conv_weight || !a_log || !dt_bias || !norm || !dy || !dqkv ||
      !dz || !da || !db)
    return PLUTO_HIP_EINVAL;
  const size_t needed = gdn_backward_workspace_bytes(p, length, d_norm != nullptr);
  if (!workspace || workspace_bytes < needed) return PLUTO_HIP_EWORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t channels =
      2ull * p->key_heads * p->key_head_dim + 1ull * p->value_heads * p->value_head_dim;
  const size_t width = 1ull * p->value_heads * p->value_head_dim, heads = p->value_heads;
  const size_t T = static_cast<size_t>(length);
  // Sequences are independent and share the scratch: they run one after the
  // other on the stream; parameter gradients accumulate over all of them.
  for (int sequence = 0; sequence < batch; ++sequence) {
    const size_t at = static_cast<size_t>(sequence) * T;
    status = launch_gdn_backward(
        s, p, length, static_cast<const uint16_t*>(qkv) + at * channels,
        static_cast<const uint16_t*>(z) + at * width, static_cast<const uint16_t*>(a) + at * heads,
        static_cast<const uint16_t*>(b) + at * heads, conv_weight, a_log, dt_bias, norm,
        dy + at * width, dqkv + at * channels, dz + at * width, da + at * heads, db + at * heads,
        d_conv_weight, d_a_log, d_dt_bias, d_norm, workspace);
    if (status != 0) return status;
  }
  return 0;
}

size_t pluto_hip_gdn_step_batch_workspace_bytes(const pluto_hip_delta_params* p, int batch) {
  if (validate_delta(p) != 0 || batch <= 0) return 0;
  const size_t n = static_cast<size_t>(batch);
  const size_t channels = 2 * static_cast<size_t>(p->key_heads) * p->key_head_dim +
                          static_cast<size_t>(p->value_heads) * p->value_head_dim;
  return align_up(n * channels * 4, 256) + 2 * align_up(n * p->value_heads * 4, 256) +
         align_up(n * p->value_heads * p->value_head_dim * 4, 256);
}

size_t pluto_hip_gdn_step_workspace_bytes(const pluto_hip_delta_params* p) {
  return pluto_hip_gdn_step_batch_workspace_bytes(p, 1);
}

int pluto_hip_gdn_step_batch(void* stream, const pluto_hip_delta_params* p, int batch,
                             int io_dtype, float* conv_states, float* recurrent_states,
                             const void* qkv, const void* z, const void* a, const void* b,
                             const float* conv_weight, const float* a_log, const float* dt_bias,
                             const float* norm, void* output, void* workspace,
                             size_t workspace_bytes) {
  int status = validate_delta(p);
  if (status != 0) return status;
  if (batch <= 0) return PLUTO_HIP_EINVAL;
  if (io_dtype != PLUTO_HIP_F32 && io_dtype != PLUTO_HIP_BF16) return PLUTO_HIP_EUNSUPPORTED;
  // cached_attention_ops.cc:405-408
  if (!conv_states || !recurrent_states || !qkv || !z || !a || !b || !conv_weight || !a_log ||
      !dt_bias || !norm || !output)
    return PLUTO_HIP_EINVAL;
  if (!workspace || workspace_bytes < pluto_hip_gdn_step_batch_workspace_bytes(p, batch))
    return PLUTO_HIP_EWORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool round = p->round_to_bfloat16 != 0;
  const int kh = p->key_heads, vh = p->value_heads, kd = p->key_head_dim, vd = p->value_head_dim;
  const int channels = 2 * kh * kd + vh * vd;
  const size_t n = static_cast<size_t>(batch);
  char* scratch = static_cast<char*>(workspace);
  float* convolved = reinterpret_cast<float*>(scratch);
  size_t offset = align_up(n * channels * 4, 256);
  float* log_decay = reinterpret_cast<float*>(scratch + offset);
  offset += align_up(n * vh * 4, 256);
  float* beta = reinterpret_cast<float*>(scratch + offset);
  offset += align_up(n * vh * 4, 256);
  float* core = reinterpret_cast<float*>(scratch + offset);
  status = launch_gdn_conv_step(s, qkv, io_dtype, conv_weight, batch, channels,
                                p->conv_kernel_dim, round, conv_states, convolved);
  if (status != 0) return status;
  if (!force_generic() && gdn_step_fused_supported(kd, vd))
    return launch_gdn_step_fused(s, convolved, z, a, b, io_dtype, a_log, dt_bias, norm, batch, kh,
                                 vh, kd, vd, p->rms_norm_epsilon, round, recurrent_states, output);
  status = launch_gdn_gates(s, a, b, io_dtype, a_log, dt_bias, batch, vh, round, log_decay, beta);
  if (status != 0) return status;
  GdnArgs g;
  g.q = reinterpret_cast<const uint16_t*>(convolved);
  g.k = reinterpret_cast<const uint16_t*>(convolved + kh * kd);
  g.v = reinterpret_cast<const uint16_t*>(convolved + 2 * kh * kd);
  g.q_token_stride = g.k_token_stride = g.v_token_stride = channels;
  g.in_dtype = PLUTO_HIP_F32;
  g.log_decay = log_decay;
  g.beta = beta;
  g.state = recurrent_states;
  g.out_any = core;
  g.batch = batch;
  g.length = 1;
  g.key_heads = kh;
  g.value_heads = vh;
  g.key_dim = kd;
  g.value_dim = vd;
  g.normalize_qk = 1;  // cached_attention_ops.cc:224-228
  g.round_output = round;
  g.q_scale = 1.0f / std::sqrt(static_cast<float>(kd));
  status = launch_gdn_recurrence(s, g, PLUTO_HIP_F32);
  if (status != 0) return status;
  return launch_gdn_output(s, core, PLUTO_HIP_F32, z, io_dtype, norm,
                           static_cast<long long>(batch) * vh, vd, p->rms_norm_epsilon, round,
                           output, io_dtype);
}

int pluto_hip_gdn_step(void* stream, const pluto_hip_delta_params* p, float* conv_state,
                       float* recurrent_state, const float* qkv, const float* z,
                       const float* a, const float* b, const float* conv_weight,
                       const float* a_log, const float* dt_bias, const float* norm,
                       float* output, void* workspace, size_t workspace_bytes) {
  return pluto_hip_gdn_step_batch(stream, p, 1, PLUTO_HIP_F32, conv_state, recurrent_state, qkv, z, a, b,
                                  conv_weight, a_log, dt_bias, norm, output, workspace,
                                  workspace_bytes);
}

}  // extern "C"
