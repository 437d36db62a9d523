// C ABI of GPT-2 style causal multi-head attention: validation and kernel
// selection.  The layer-level contract is that of AttentionLayer
// (src/llm/layers/attention.cc:400-596).
#include <cmath>

#include "attn_generic.h"
#include "flash_bwd_mfma.h"
#include "flash_fwd_mfma.h"

namespace pluto_hip {

// Test hooks.  pluto_hip_test_force_generic routes the calling thread's later
// calls through the any-shape FP32-arithmetic kernels so that the two
// implementations can be checked against each other on the device;
// pluto_hip_test_kernel_classes masks kernel classes for measurements.  Both
// are per thread: a thread that never calls them (every product caller) always
// gets normal kernel selection, whatever a test thread of the same process has
// set.  The library has no process-wide switches.
namespace {
thread_local int force_generic_flag = 0;
thread_local unsigned kernel_class_mask = ~0u;
thread_local int last_path = PLUTO_HIP_PATH_NONE;
}  // namespace
bool force_generic() { return force_generic_flag != 0; }
void note_path(int path) { last_path = path; }
bool kernel_enabled(KernelClass which) { return (kernel_class_mask & which) != 0; }

namespace {

int validate_mha(int dtype, int rows, int context_length, int num_heads,
                 int embedding_dim) {
  if (dtype != PLUTO_HIP_F32 && dtype != PLUTO_HIP_BF16)
    return PLUTO_HIP_EUNSUPPORTED;  // attention.cc:403 (FP8 -> Unimplemented)
  if (context_length <= 0 || num_heads <= 0 || embedding_dim <= 0)
    return PLUTO_HIP_EINVAL;  // attention.cc:404-407
  if (embedding_dim % num_heads != 0) return PLUTO_HIP_EINVAL;  // :408-411
  if (rows <= 0 || rows % context_length != 0) return PLUTO_HIP_EINVAL;  // :429
  if (embedding_dim / num_heads > 256) return PLUTO_HIP_EUNSUPPORTED;
  return 0;
}

GenericForwardArgs packed_forward_args(int dtype, const void* qkv, int rows,
                                       int T, int H, int E, void* out,
                                       float* maxima, float* normalizers) {
  (void)rows;
  const int D = E / H;
  const size_t element = dtype == PLUTO_HIP_BF16 ? 2 : 4;
  GenericForwardArgs a;
  const char* base = static_cast<const char*>(qkv);
  a.q = {base, 3LL * E * T, 3LL * E, D, dtype};
  a.k = {base + element * E, 3LL * E * T, 3LL * E, D, dtype};
  a.v = {base + element * 2 * E, 3LL * E * T, 3LL * E, D, dtype};
  a.out = out;
  a.o_seq_stride = 1LL * E * T;
  a.o_row_stride = E;
  a.o_head_stride = D;
  a.o_dtype = dtype;
  a.maxima = maxima;
  a.normalizers = normalizers;
  a.q_rows = T;
  a.kv_rows = T;
  a.start_position = 0;
  a.query_heads = H;
  a.group = 1;
  a.head_dim = D;
  a.scale = 1.0f / std::sqrt(static_cast<float>(D));
  return a;
}

}  // namespace
}  // namespace pluto_hip

using namespace pluto_hip;

extern "C" {

int pluto_hip_test_force_generic(int enabled) {
  const int before = force_generic_flag;
  force_generic_flag = enabled != 0 ? 1 : 0;
  return before;
}

unsigned pluto_hip_test_kernel_classes(unsigned mask) {
  const unsigned before = kernel_class_mask;
  kernel_class_mask = mask;
  return before;
}

int pluto_hip_test_last_path(void) { return last_path; }

int pluto_hip_mha_forward(void* stream, int dtype, const void* qkv, int rows,
                          int context_length, int num_heads, int embedding_dim,
                          void* out, float* maxima, float* normalizers) {
  int status = validate_mha(dtype, rows, context_length, num_heads, embedding_dim);
  if (status != 0) return status;
  if (!qkv || !out || !maxima || !normalizers) return PLUTO_HIP_EINVAL;
  const int T = context_length, H = num_heads, E = embedding_dim, D = E / H;
  const int sequences = rows / T;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == PLUTO_HIP_BF16 && !force_generic()) {
    FlashForwardArgs f;
    const uint16_t* base = static_cast<const uint16_t*>(qkv);
    f.q = base;
    f.k = base + E;
    f.v = base + 2 * E;
    f.q_seq_stride = f.k_seq_stride = f.v_seq_stride = 3LL * E * T;
    f.q_row_stride = f.k_row_stride = f.v_row_stride = 3LL * E;
    f.q_head_stride = f.k_head_stride = f.v_head_stride = D;
    f.out = static_cast<uint16_t*>(out);
    f.o_seq_stride = 1LL * E * T;
    f.o_row_stride = E;
    f.o_head_stride = D;
    f.maxima = maxima;
    f.normalizers = normalizers;
    f.q_rows = T;
    f.kv_rows = T;
    f.query_heads = H;
    f.group = 1;
    f.scale = 1.0f / std::sqrt(static_cast<float>(D));
    if (flash_forward_supported(f, D)) {
      note_path(PLUTO_HIP_PATH_FLASH);
      return launch_flash_forward(s, f, D, sequences);
    }
  }
  const GenericForwardArgs a =
      packed_forward_args(dtype, qkv, rows, T, H, E, out, maxima, normalizers);
  if (!force_generic() && f32_forward_supported(a)) {
    note_path(PLUTO_HIP_PATH_MATRIX_F32);
    return launch_f32_forward(s, a, sequences);
  }
  note_path(PLUTO_HIP_PATH_GENERIC);
  return launch_generic_forward(s, a, sequences);
}

int pluto_hip_mha_probabilities(void* stream, int dtype, const void* qkv,
                                const float* maxima, const float* normalizers,
                                int rows, int context_length, int num_heads,
                                int embedding_dim, float* probabilities) {
  int status = validate_mha(dtype, rows, context_length, num_heads, embedding_dim);
  if (status != 0) return status;
  if (!qkv || !maxima || !normalizers || !probabilities) return PLUTO_HIP_EINVAL;
  // attention.cc:40-61: the quadratic tensor must be addressable.
  const long long tiles = (context_length + 31) / 32;
  if (tiles * tiles > 0x7fffffffLL) return PLUTO_HIP_ERANGE;
  const GenericForwardArgs a = packed_forward_args(
      dtype, qkv, rows, context_length, num_heads, embedding_dim, nullptr,
      const_cast<float*>(maxima), const_cast<float*>(normalizers));
  return launch_generic_probabilities(static_cast<hipStream_t>(stream), a,
                                      rows / context_length, probabilities);
}

size_t pluto_hip_mha_backward_workspace_bytes(int dtype, int rows,
                                              int context_length, int num_heads,
                                              int embedding_dim) {
  if (validate_mha(dtype, rows, context_length, num_heads, embedding_dim) != 0)
    return 0;
  // deltas [rows/T * H, T] fp32; the bf16 path adds the rows' log2-sum-exp
  // (same shape) and a bf16 copy of d_out.
  const size_t stats = align_up(static_cast<size_t>(rows) * num_heads * sizeof(float), 256);
  size_t bytes = stats;
  if (dtype == PLUTO_HIP_BF16)
    bytes += stats + align_up(static_cast<size_t>(rows) * embedding_dim * 2, 256);
  return bytes;
}

int pluto_hip_mha_backward(void* stream, int dtype, const void* qkv,
                           const void* out, const float* d_out,
                           const float* maxima, const float* normalizers,
                           int rows, int context_length, int num_heads,
                           int embedding_dim, float* d_qkv, void* workspace,
                           size_t workspace_bytes) {
  int status = validate_mha(dtype, rows, context_length, num_heads, embedding_dim);
  if (status != 0) return status;
  if (!qkv || !out || !d_out || !maxima || !normalizers || !d_qkv)
    return PLUTO_HIP_EINVAL;
  const size_t needed = pluto_hip_mha_backward_workspace_bytes(
      dtype, rows, context_length, num_heads, embedding_dim);
  if (!workspace || workspace_bytes < needed) return PLUTO_HIP_EWORKSPACE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  GenericBackwardArgs a;
  a.qkv = qkv;
  a.out = out;
  a.dtype = dtype;
  a.d_out = d_out;
  a.maxima = maxima;
  a.normalizers = normalizers;
  a.deltas = static_cast<float*>(workspace);
  a.d_qkv = d_qkv;
  a.rows = rows;
  a.context_length = context_length;
  a.num_heads = num_heads;
  a.embedding_dim = embedding_dim;
  const int D = embedding_dim / num_heads;
  a.scale = 1.0f / std::sqrt(static_cast<float>(D));
  if (dtype == PLUTO_HIP_BF16 && !force_generic() &&
      flash_backward_supported(a)) {
    const size_t stats =
        align_up(static_cast<size_t>(rows) * num_heads * sizeof(float), 256);
    char* scratch = static_cast<char*>(workspace);
    note_path(PLUTO_HIP_PATH_FLASH);
    return launch_flash_backward(s, a, reinterpret_cast<float*>(scratch + stats),
                                 reinterpret_cast<uint16_t*>(scratch + 2 * stats));
  }
  note_path(PLUTO_HIP_PATH_GENERIC);
  return launch_generic_backward(s, a);
}

}  // extern "C"
