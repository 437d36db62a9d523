// Launcher of the bf16 MFMA flash-attention backward kernels.
#pragma once

#include "attn_generic.h"

namespace pluto_hip {

bool flash_backward_supported(const GenericBackwardArgs& args);
// lse2: scratch [rows/T * H, T] fp32 (log2-sum-exp of every softmax row);
// d_out_bf16: scratch for a bf16 copy of d_out, [rows, E].
int launch_flash_backward(hipStream_t stream, const GenericBackwardArgs& args,
                          float* lse2, uint16_t* d_out_bf16);
// The key-owned kernel for heads of 64 channels with a hand-scheduled main loop
// (flash_dkv_wide.hip); reads what the query-owned kernel left in lse2,
// args.deltas and d_out_bf16.
int launch_flash_dkv_wide(hipStream_t stream, const GenericBackwardArgs& args, const float* lse2,
                          const uint16_t* d_out_bf16);

}  // namespace pluto_hip
