// Shared device/host helpers for the gfx950 kernels of the attention path.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "pluto_hip.h"

namespace pluto_hip {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(2))) float floatx2;
typedef __attribute__((ext_vector_type(4))) uint32_t uint32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t uint32x2;

constexpr int kWave = 64;
// Finite sentinel for masked scores, as in the reference kernels
// (src/llm/layers/attention.cc:132,146).
constexpr float kMasked = -3.402823466e+38f;
constexpr float kLog2e = 1.4426950408889634f;

// bfloat16 <-> float, round to nearest even
// (src/llm/layers/reference_internal.h:109-119).
__host__ __device__ inline float bf16_bits_to_float(uint16_t bits) {
  union {
    uint32_t u;
    float f;
  } c;
  c.u = static_cast<uint32_t>(bits) << 16;
  return c.f;
}

__host__ __device__ inline uint16_t float_to_bf16_bits(float value) {
  union {
    uint32_t u;
    float f;
  } c;
  c.f = value;
  c.u += 0x7fffu + ((c.u >> 16) & 1u);
  return static_cast<uint16_t>(c.u >> 16);
}

__host__ __device__ inline float round_to_bf16(float value) {
  return bf16_bits_to_float(float_to_bf16_bits(value));
}

// Sigmoid of a gate logit, the one form every kernel of the library uses (the
// cached step, the sequence kernels and the any-shape kernels must agree bit
// for bit): one v_exp_f32 and one v_rcp_f32, about two units in the last place
// of FP32 before the result is rounded to bf16.  Saturates to 0 and 1.
__device__ inline float gate_sigmoid(float logit) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-logit * kLog2e));
}

// Runtime-typed element access for the generic (any shape) kernels.
__device__ inline float load_element(const void* base, long long index,
                                     int dtype) {
  if (dtype == PLUTO_HIP_BF16)
    return bf16_bits_to_float(static_cast<const uint16_t*>(base)[index]);
  return static_cast<const float*>(base)[index];
}

__device__ inline void store_element(void* base, long long index, int dtype,
                                     float value) {
  if (dtype == PLUTO_HIP_BF16)
    static_cast<uint16_t*>(base)[index] = float_to_bf16_bits(value);
  else
    static_cast<float*>(base)[index] = value;
}

__device__ inline float wave_half_max(float v) {
  // reduction over 32 consecutive lanes (one half of a wave64)
  for (int offset = 16; offset > 0; offset >>= 1)
    v = fmaxf(v, __shfl_xor(v, offset, 64));
  return v;
}

__device__ inline float wave_half_sum(float v) {
  for (int offset = 16; offset > 0; offset >>= 1)
    v += __shfl_xor(v, offset, 64);
  return v;
}

__device__ inline float wave_sum(float v) {
  for (int offset = 32; offset > 0; offset >>= 1)
    v += __shfl_xor(v, offset, 64);
  return v;
}

__device__ inline float wave_max(float v) {
  for (int offset = 32; offset > 0; offset >>= 1)
    v = fmaxf(v, __shfl_xor(v, offset, 64));
  return v;
}

inline int launch_status() { return static_cast<int>(hipGetLastError()); }

// Measurement hook (pluto_hip_test_kernel_classes): the launchers of the
// specialised kernels ask whether their class is switched on, so that a
// benchmark can time one kernel of a multi-launch entry point with events
// around the call.  All classes are on unless a test or benchmark says so.
enum KernelClass : unsigned {
  kMainKernel = 1u,       // the kernel that bounds the call (flash, split-K, scan ...)
  kQueryKernel = 2u,      // the query-owned half of the attention backward
  kAuxiliaryKernel = 4u,  // preparation, tables, combines
  kEightWave = 16u,       // not a kernel: the hand-scheduled kernels may be taken (pipelined forward, wide dK/dV)
  kFromLength = 32u,      // not a kernel: ... but only from the sequence lengths where they win
};
bool kernel_enabled(KernelClass which);  // mha_capi.hip
// Records the kernel family a compute call chose (pluto_hip_test_last_path).
void note_path(int path);  // mha_capi.hip

inline size_t align_up(size_t value, size_t alignment) {
  return (value + alignment - 1) / alignment * alignment;
}

}  // namespace pluto_hip
