/*
 * pluto_oracle.h -- CPU restatement of the reference's attention hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the benchmark's cpu_baseline leg may link or call it, and
 * only as the checker.  Nothing that ships computes through this library.
 *
 * Every function restates, in scalar C, a function of the reference
 * (sanjoy/pluto); the reference file:line it follows is cited at each
 * declaration.  Arithmetic is done in the same precision and order as the
 * cited code so results agree to the last bit wherever the cited code is
 * itself deterministic scalar code.
 *
 * Pinning status (which independent evidence fixes each function):
 *   mha_fwd / mha_bwd        closed form (attention_test.cc:282-360), float64
 *                            scaled_dot_product_attention + autograd, brute
 *                            force, causality invariants.
 *   gqa_*                    known answers of cached_attention_test.cc:108-156,
 *                            exact gate expectation and uniform 1/L rows of
 *                            cached_attention_ops_test.cc:364-398,472-503,
 *                            an independent float64 numpy restatement.
 *   gqa_sequence_backward    central finite differences of a frozen-rounding
 *                            double-precision forward (the reference's own
 *                            check, qwen_attention_test.cc:22-99,230-300, at
 *                            its bound of 3e-5, both rounding modes) and
 *                            float64 autograd of the unrounded layer.
 *   gdn_sequence_backward    the same two checks (frozen-rounding finite
 *                            differences at 3e-5, float64 autograd) for all
 *                            four inputs and four parameters.
 *   gdn_*                    textbook delta rule special cases (beta=0, g=0
 *                            with orthonormal keys), softplus extremes,
 *                            independent float64 numpy recurrence.
 */
#ifndef PLUTO_ORACLE_H_
#define PLUTO_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Storage type of activations.  The reference's DataType::FP16 policy keeps
 * FP32 storage (src/llm/layer.h:86-88); DataType::BF16 stores bfloat16. */
enum { PLUTO_ORACLE_F32 = 0, PLUTO_ORACLE_BF16 = 1 };

/* src/llm/layers/reference_internal.h:109-119 (round to nearest even). */
uint16_t pluto_oracle_f32_to_bf16(float value);
float pluto_oracle_bf16_to_f32(uint16_t value);
float pluto_oracle_bf16_round(float value);

/* ---- GPT-2 style causal multi-head attention -------------------------- */

/* src/llm/layers/attention_reference.cc:36-114.  qkv is the packed
 * [rows, 3*E] activation, out is [rows, E].  Additionally reports the
 * per-(sequence, head, position) maximum and normalizer of the softmax row
 * ([rows/T * H, T] each, nullable), which the reference's device layer saves
 * (src/llm/layers/attention.cc:448-451) and the CPU class does not.
 * Only sequences [seq_begin, seq_end) and heads [head_begin, head_end) are
 * computed; other outputs are left untouched.  Returns 0, or -1 on a shape
 * the reference rejects. */
int pluto_oracle_mha_fwd(int dtype, const void* qkv, int rows,
                         int context_length, int num_heads, int embedding_dim,
                         void* out, float* maxima, float* normalizers,
                         int seq_begin, int seq_end, int head_begin,
                         int head_end);

/* src/llm/layers/attention_reference.cc:116-230.  d_qkv must be zeroed by
 * the caller ([rows, 3*E] fp32); d_out is fp32 [rows, E]; out is the stored
 * forward output. */
int pluto_oracle_mha_bwd(int dtype, const void* qkv, const void* out,
                         const float* d_out, int rows, int context_length,
                         int num_heads, int embedding_dim, float* d_qkv,
                         int seq_begin, int seq_end, int head_begin,
                         int head_end);

/* ---- Qwen style grouped-query attention ------------------------------- */

/* src/llm/layers/util/cached_attention_ops.h:13-22 */
typedef struct {
  int query_heads;
  int key_value_heads;
  int head_dim;
  int rotary_dim;
  int capacity;
  float rms_norm_epsilon;
  float rope_theta;
  int round_to_bfloat16;
} pluto_oracle_attention_params;

/* Per-head RMSNorm with (1 + weight) and split-half partial RoPE at
 * `position`: src/llm/layers/util/cached_attention_ops_test.cc:56-78 (scalar
 * specification of cached_attention_ops.cc:30-79). */
void pluto_oracle_gqa_normalize_rotate(const pluto_oracle_attention_params* p,
                                       int position, const float* input,
                                       const float* weight, float* output);

/* One cached decode step: cached_attention_ops_test.cc:46-118 (scalar
 * specification of CachedAttentionStep, cached_attention_ops.cc:308-353).
 * cache_keys / cache_values are FP32 [capacity, kv_heads, head_dim]
 * (src/llm/key_value_cache.h:13-16); `position` rows are valid on entry and
 * row `position` is written.  q_gate is [qh, 2, d], k/v are [kh, d], output
 * is [qh, d], probabilities (nullable) is [qh, position + 1].
 * Returns 0, -1 for invalid parameters, -2 when the cache is full. */
int pluto_oracle_gqa_cached_step(const pluto_oracle_attention_params* p,
                                 float* cache_keys, float* cache_values,
                                 int position, const float* q_gate,
                                 const float* k, const float* v,
                                 const float* q_norm, const float* k_norm,
                                 float* output, float* probabilities);

/* Whole-sequence attention with the semantics of
 * QwenAttentionLayer::SequenceForward (src/llm/layers/qwen_attention.cc:
 * 414-448; scalar specification qwen_attention_test.cc:26-95): row t is the
 * cached step at position t.  qg is [T, qh, 2, d], k/v are [T, kh, d]; all
 * inputs are FP32 holding the (bf16 representable) activations.  Writes the
 * prepared keys and rounded values for every row < row_end into key_out /
 * value_out ([T, kh, d], nullable) and the gated output [T, qh, d] for rows
 * [row_begin, row_end) and heads [head_begin, head_end).  lse (nullable,
 * [T, qh]) receives max + log(normalizer) of each softmax row. */
int pluto_oracle_gqa_sequence(const pluto_oracle_attention_params* p,
                              int length, const float* qg, const float* k,
                              const float* v, const float* q_norm,
                              const float* k_norm, float* out, float* key_out,
                              float* value_out, float* lse, int row_begin,
                              int row_end, int head_begin, int head_end);

/* Gradients of pluto_oracle_gqa_sequence with respect to qg, k, v and the two
 * norm weights for an upstream gradient dy [T, qh, d]
 * (QwenAttentionLayer::SequenceBackward, qwen_attention.cc:450-499).  dqg
 * [T, qh, 2, d], dk, dv [T, kh, d] are overwritten; dq_norm, dk_norm (nullable,
 * [d]) are added to. */
int pluto_oracle_gqa_sequence_backward(const pluto_oracle_attention_params* p,
                                       int length, const float* qg, const float* k,
                                       const float* v, const float* q_norm,
                                       const float* k_norm, const float* dy,
                                       float* dqg, float* dk, float* dv,
                                       float* dq_norm, float* dk_norm);

/* Attention of prepared queries against an existing cache, used for the
 * batched decode configuration: q is [qh, d] already normalised and rotated,
 * gate is [qh, d] raw logits, keys/values are [kh, length, d] head-major FP32
 * views of a bf16 cache (row stride = stride_tokens rows per head).  Softmax
 * and gating follow cached_attention_ops_test.cc:86-114. */
int pluto_oracle_gqa_attend(const pluto_oracle_attention_params* p, int length,
                            size_t head_stride, const float* q,
                            const float* gate, const float* keys,
                            const float* values, float* output);

/* ---- Gated delta-net --------------------------------------------------- */

/* src/llm/layers/util/cached_attention_ops.h:49-57 */
typedef struct {
  int key_heads;
  int value_heads;
  int key_head_dim;
  int value_head_dim;
  int conv_kernel_dim;
  float rms_norm_epsilon;
  int round_to_bfloat16;
} pluto_oracle_delta_params;

/* The recurrence alone: sequence_delta_net_test.cc:100-141 (scalar
 * specification of RecurrenceForward, sequence_delta_net.cc:55-102).
 * q, k are [T, kh, kd]; v is [T, vh, vd]; log_decay and beta are [T, vh]
 * (decay = exp(log_decay); beta is used as given).  When normalize_qk is
 * nonzero q and k are L2-normalised as the reference does (1e-6 added to the
 * sum of squares); q is always multiplied by q_scale (the reference uses
 * 1/sqrt(kd)).  state is FP64 [vh, kd, vd], read as the initial state and
 * overwritten with the final state.  core is [T, vh, vd], rounded to bf16
 * when p->round_to_bfloat16.  Heads [head_begin, head_end) only. */
int pluto_oracle_gdn_scan(const pluto_oracle_delta_params* p, int length,
                          const float* q, const float* k, const float* v,
                          const float* log_decay, const float* beta,
                          int normalize_qk, double q_scale, double* state,
                          float* core, int head_begin, int head_end);

/* Whole layer over a sequence: sequence_delta_net_test.cc:66-159 (scalar
 * specification of SequenceDeltaNetLayer::fwd_impl, sequence_delta_net.cc:
 * 435-480).  qkv is [T, 2*kh*kd + vh*vd] packed [all Q | all K | all V],
 * z is [T, vh*vd], a and b are [T, vh]; conv_weight is [channels, kernel];
 * a_log, dt_bias are [vh]; norm is [vd].  output is [T, vh*vd].  core
 * (nullable) receives the pre-norm recurrence output, final_state (nullable)
 * the FP64 [vh, kd, vd] state after the last token. */
int pluto_oracle_gdn_sequence(const pluto_oracle_delta_params* p, int length,
                              const float* qkv, const float* z, const float* a,
                              const float* b, const float* conv_weight,
                              const float* a_log, const float* dt_bias,
                              const float* norm, float* output, float* core,
                              double* final_state);

/* Gradients of pluto_oracle_gdn_sequence with respect to its four activation
 * inputs and four parameters for an upstream gradient dy [T, vh*vd]
 * (SequenceDeltaNetLayer::bwd_impl, sequence_delta_net.cc:482-561).  dqkv
 * [T, channels], dz [T, vh*vd], da, db [T, vh] are overwritten; the parameter
 * gradients (nullable; shapes of the parameters) are added to. */
int pluto_oracle_gdn_sequence_backward(
    const pluto_oracle_delta_params* p, int length, const float* qkv, const float* z,
    const float* a, const float* b, const float* conv_weight, const float* a_log,
    const float* dt_bias, const float* norm, const float* dy, float* dqkv, float* dz,
    float* da, float* db, float* d_conv_weight, float* d_a_log, float* d_dt_bias,
    float* d_norm);

/* Single-token step with persistent state: cached_attention_ops_test.cc:
 * 133-220 (scalar specification of DeltaNetState::Step,
 * cached_attention_ops.cc:401-431).  conv_state is FP32 [channels, kernel],
 * recurrent_state is FP64 [vh, kd, vd]; both are updated in place. */
int pluto_oracle_gdn_step(const pluto_oracle_delta_params* p,
                          float* conv_state, double* recurrent_state,
                          const float* qkv, const float* z, const float* a,
                          const float* b, const float* conv_weight,
                          const float* a_log, const float* dt_bias,
                          const float* norm, float* output);

/* FullyConnectedLayer, trainable path (src/llm/layers/fully_connected.cc:
 * DenseForwardKernel :97-131, DenseInputGradientKernel :134-164,
 * DenseWeightGradientKernel :167-196, the bias gradient :198-247).  dtype is
 * the activation storage: PLUTO_ORACLE_BF16 (0x1) multiplies operands rounded
 * to bf16, PLUTO_ORACLE_F32 (0x0) operands rounded to IEEE half (MmaType,
 * :31-33); sums are kept in double here (FP32 in the reference, order
 * unspecified).  matrix is [input_dim, output_dim], bias [output_dim].
 *   forward:  y[r, o] = bias[o] + sum_i R(x[r, i]) R(w[i, o]), stored in the
 *             activation type (rounded to bf16 for bf16 storage)
 *   backward: dx[r, i] = sum_o R(dy[r, o]) R(w[i, o])
 *             dw[i, o] = sum_r R(x[r, i]) R(dy[r, o])
 *             db[o]    = sum_r dy[r, o]            (dy unrounded)
 * x is given as float values (bf16-representable for bf16 storage). */
float pluto_oracle_half_round(float value);
int pluto_oracle_dense_forward(int dtype, int rows, int input_dim, int output_dim,
                               const float* x, const float* matrix, const float* bias,
                               float* y);
int pluto_oracle_dense_backward(int dtype, int rows, int input_dim, int output_dim,
                                const float* x, const float* matrix, const float* dy,
                                float* dx, float* d_matrix, float* d_bias);

/* Imported (frozen, output-major) projection of FullyConnectedLayer
 * (src/llm/layers/fully_connected.cc:40-94,295-341): one bf16 token
 * [input_dim] against weights [output_dim, input_dim] stored as bf16, fp32 or
 * FP8 E4M3 with FP32 scales [ceil(out/128), ceil(in/128)]; all arithmetic in
 * FP32 (here: double sums, as the scalar projection of
 * fully_connected_imported_test.cc:190-205), output rounded to bf16. */
#define PLUTO_ORACLE_MATRIX_BF16 0
#define PLUTO_ORACLE_MATRIX_F32 1
#define PLUTO_ORACLE_MATRIX_FP8_E4M3 2
/* OCP FP8 E4M3 (no infinities, 0x7f/0xff NaN, largest finite 448). */
float pluto_oracle_fp8_e4m3_to_f32(uint8_t bits);
/* Round to nearest even, saturating to +-448; NaN -> 0x7f. */
uint8_t pluto_oracle_f32_to_fp8_e4m3(float value);
/* QuantizeImportedInputKernel (fully_connected.cc:70-88): per group of 128
 * elements scale = max|x| / 448, out = fp8(x / max(scale, 1e-12)) * scale. */
void pluto_oracle_imported_quantize(const float* x, int n, float* out);
/* x: the token as floats (bf16 values); FP8 storage quantizes it first.
 * y: output_dim floats holding bf16 values. */
int pluto_oracle_imported_matvec(int storage, const void* weights, const float* scales,
                                 const float* x, int input_dim, int output_dim, float* y);

#ifdef __cplusplus
}
#endif
#endif /* PLUTO_ORACLE_H_ */
