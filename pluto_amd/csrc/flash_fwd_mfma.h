// Argument block and launcher of the bf16 MFMA flash-attention forward kernel.
#pragma once

#include "common.h"

namespace pluto_hip {

// All tensors hold bf16 bits.  Element (seq, row, head, c) of a tensor is
// base[seq*seq_stride + row*row_stride + head*head_stride + c]; every stride
// must be a multiple of 8 elements and every base 16-byte aligned.
struct FlashForwardArgs {
  const uint16_t* q = nullptr;
  long long q_seq_stride = 0, q_row_stride = 0, q_head_stride = 0;
  const uint16_t* k = nullptr;
  long long k_seq_stride = 0, k_row_stride = 0, k_head_stride = 0;
  const uint16_t* v = nullptr;
  long long v_seq_stride = 0, v_row_stride = 0, v_head_stride = 0;
  uint16_t* out = nullptr;
  long long o_seq_stride = 0, o_row_stride = 0, o_head_stride = 0;
  uint16_t* core = nullptr;        // optional: the output before the gate, laid out like out
  const uint16_t* gate = nullptr;  // optional sigmoid gate logits
  long long gate_seq_stride = 0, gate_row_stride = 0, gate_head_stride = 0;
  float* maxima = nullptr;       // [(seq*QH + head)*q_rows + row]
  float* normalizers = nullptr;  // same layout
  float* lse = nullptr;          // [(seq*q_rows + row)*QH + head]
  int q_rows = 0;
  int kv_rows = 0;
  int start_position = 0;  // query row i sees keys [0, start_position + i]
  int query_heads = 0;
  int group = 1;
  float scale = 1.0f;
};

bool flash_forward_supported(const FlashForwardArgs& args, int head_dim);
int launch_flash_forward(hipStream_t stream, const FlashForwardArgs& args,
                         int head_dim, int sequences);
// flash_fwd_pipelined.hip: head widths 64 and 128, 256-row query tiles, hand-scheduled
// main loop; what launch_flash_forward picks for long sequences.
int launch_flash_forward_pipelined(hipStream_t stream, const FlashForwardArgs& args,
                                   int head_dim, int sequences);

}  // namespace pluto_hip
