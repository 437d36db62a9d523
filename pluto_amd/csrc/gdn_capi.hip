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
    return launch_gdn_chunked(s, a);
  }
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

}  // extern "C"
