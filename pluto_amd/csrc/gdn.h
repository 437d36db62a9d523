// Argument block of the gated delta-net kernels and the per-chunk scratch
// layout shared by the two kernels of the chunked scan.
#pragma once

#include "common.h"

namespace pluto_hip {

// Scratch written by the chunk-parallel kernel for one 64-token chunk of one
// (sequence, head), all in matrix-core register order:
//   U      fp32 [4 token tiles][8 column slices][64 lanes][4]        32 KiB
//   -W     bf16 [4 token tiles][4 key blocks][64 lanes][8]           16 KiB
//   cQ     bf16 same shape (exp(c) * q_scale * Q)                    16 KiB
//   A2     bf16 [4 token tiles][2 token blocks][64 lanes][8]          8 KiB
//   Kt     bf16 [8 key tiles][2 token blocks][64 lanes][8]           16 KiB
//   decay  fp32 exp(c_C)
constexpr size_t kGdnOffsetU = 0;
constexpr size_t kGdnOffsetW = 32768;
constexpr size_t kGdnOffsetQ = 49152;
constexpr size_t kGdnOffsetA2 = 65536;
constexpr size_t kGdnOffsetKt = 73728;
constexpr size_t kGdnOffsetDecay = 90112;
constexpr size_t kGdnChunkBytes = 90368;

struct GdnArgs {
  const uint16_t* q = nullptr;  // bf16 [batch, T, kh, kd]
  const uint16_t* k = nullptr;
  const uint16_t* v = nullptr;  // bf16 [batch, T, vh, vd]
  const float* log_decay = nullptr;  // [batch, T, vh]
  const float* beta = nullptr;
  float* state = nullptr;   // fp32 [batch, vh, kd, vd]
  uint16_t* out = nullptr;  // bf16 [batch, T, vh, vd] (chunked scan)
  void* out_any = nullptr;  // recurrence kernel: bf16 or fp32
  char* workspace = nullptr;
  int batch = 0, length = 0;
  int key_heads = 0, value_heads = 0, key_dim = 0, value_dim = 0;
  int normalize_qk = 0;
  int round_output = 1;
  float q_scale = 1.0f;
};

bool gdn_chunked_supported(const GdnArgs& args, int chunk);
int launch_gdn_chunked(hipStream_t stream, const GdnArgs& args);
int launch_gdn_recurrence(hipStream_t stream, const GdnArgs& args, int out_dtype);

}  // namespace pluto_hip
