/*
 * pluto_hip.h -- C ABI of the MI355X (gfx950) attention path.
 *
 * This is the boundary a maintainer of the reference (sanjoy/pluto) binds to
 * replace the execution pieces of its attention hot path: the stream/buffer
 * runtime of src/cuda and the device kernels of src/llm/layers/{attention,
 * qwen_attention,sequence_delta_net,delta_net}.cc and
 * src/llm/layers/util/cached_attention_ops.cc.  Every entry point cites the
 * reference interface it stands in for.
 *
 * Conventions
 *   - plain C types only: device/host pointers, sizes, ints, floats.
 *   - every function returns 0 on success.  Positive values are hipError_t
 *     codes reported by the HIP runtime; negative values are the PLUTO_HIP_E*
 *     codes below (argument validation, done before any GPU work is queued).
 *   - `stream` is a hipStream_t passed as void*.  Nothing synchronises with
 *     the host and nothing uses the default stream; all work is queued on the
 *     given stream, and calls on different streams may run concurrently.
 *   - kernels never allocate: scratch memory is passed in as `workspace`, whose
 *     required size the matching *_workspace_bytes function reports.
 */
#ifndef PLUTO_HIP_H_
#define PLUTO_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PLUTO_HIP_EINVAL (-1)       /* invalid argument (absl::InvalidArgument) */
#define PLUTO_HIP_ERANGE (-2)       /* capacity exhausted (absl::ResourceExhausted) */
#define PLUTO_HIP_EUNSUPPORTED (-3) /* not implemented (absl::Unimplemented) */
#define PLUTO_HIP_EWORKSPACE (-4)   /* workspace missing or too small */
#define PLUTO_HIP_ELIMIT (-5)       /* request larger than an entry point's fixed scratch */

/* Storage type of an activation buffer.  The reference's DataType::FP16
 * compute policy keeps FP32 storage (src/llm/layer.h:86-88). */
#define PLUTO_HIP_F32 0
#define PLUTO_HIP_BF16 1

/* Human readable text for any value returned by this library. */
const char* pluto_hip_error_name(int code);
const char* pluto_hip_error_string(int code);

/* Library/ABI version and the gfx target the kernels were compiled for.  The
 * version changes whenever an existing signature, struct or workspace layout
 * changes; a caller compares pluto_hip_abi_version() with the
 * PLUTO_HIP_ABI_VERSION of the header it was built against.
 *   2: pluto_hip_gdn_step_batch takes io_dtype and void* activations; the
 *      decode workspace starts with the arrival counters;
 *      pluto_hip_dense_imported_workspace_bytes grew.
 *   3: pluto_hip_gqa_decode_static_reset added.
 *      (pluto_hip_dense_imported_forward_many was added without a bump:
 *      nothing that existed changed.) */
#define PLUTO_HIP_ABI_VERSION 3
int pluto_hip_abi_version(void);
const char* pluto_hip_target_arch(void);

/* ------------------------------------------------------------------------
 * Runtime: replaces src/cuda/executor.{h,cc}, buffer.{h,cc} and
 * page_locked_host_buffer.{h,cc} for this path.
 * --------------------------------------------------------------------- */

typedef struct pluto_hip_executor pluto_hip_executor;

/* cuda::Executor::Create (src/cuda/executor.cc:35-96): one non-blocking
 * compute stream, one non-blocking immediate stream, a pinned-host block
 * cache.  Uses the calling thread's current device. */
int pluto_hip_executor_create(pluto_hip_executor** executor);
/* cuda::Executor::~Executor (src/cuda/executor.cc:98-116): drains both
 * streams, releases cached pinned blocks, destroys the streams. */
int pluto_hip_executor_destroy(pluto_hip_executor* executor);
/* cuda::Executor::Synchronize (src/cuda/executor.cc:118-120). */
int pluto_hip_executor_synchronize(pluto_hip_executor* executor);
/* cuda::Executor::stream / immediate_stream (src/cuda/executor.h:42-51). */
void* pluto_hip_executor_stream(pluto_hip_executor* executor);
void* pluto_hip_executor_immediate_stream(pluto_hip_executor* executor);

/* cuda::Buffer::Allocate (src/cuda/buffer.cc:53-68): stream-ordered device
 * allocation on the compute stream.  bytes == 0 yields *data == NULL. */
int pluto_hip_malloc_async(pluto_hip_executor* executor, size_t bytes,
                           void** data);
/* cuda::Buffer::Allocation::~Allocation (src/cuda/buffer.cc:33-47): the free
 * is ordered after all work queued so far on the compute stream. */
int pluto_hip_free_async(pluto_hip_executor* executor, void* data);

/* cuda::PageLockedHostBuffer::Allocate
 * (src/cuda/page_locked_host_buffer.h:27-29): pinned host memory that the CPU
 * may touch as soon as the call returns, without waiting for compute. */
int pluto_hip_host_alloc(pluto_hip_executor* executor, size_t bytes,
                         void** data);
/* Release of a pinned block: it is recycled only after the work queued on
 * the compute stream at the time of this call has finished
 * (src/cuda/page_locked_host_buffer.h:13-24). */
int pluto_hip_host_free_async(pluto_hip_executor* executor, void* data);

/* cudaMemcpyAsync / cudaMemsetAsync call sites of the path
 * (src/llm/layers/util/cached_attention_ops.cc:433-441,
 *  src/llm/block_parameter.cc:56-66).  kind: 1 H2D, 2 D2H, 3 D2D. */
int pluto_hip_memcpy_async(void* stream, void* dst, const void* src,
                           size_t bytes, int kind);
int pluto_hip_memset_async(void* stream, void* dst, int value, size_t bytes);
int pluto_hip_stream_synchronize(void* stream);

/* CastKernel of src/llm/layers/util.cc:14-40 (ToFloat / ToBFloat16). */
int pluto_hip_cast_bf16_to_f32(void* stream, const void* src, float* dst,
                               size_t count);
int pluto_hip_cast_f32_to_bf16(void* stream, const float* src, void* dst,
                               size_t count);

/* ------------------------------------------------------------------------
 * GPT-2 style causal multi-head attention over packed [rows, 3E] Q|K|V.
 * --------------------------------------------------------------------- */

/* AttentionLayer::fwd_impl + FlashAttentionForwardKernel
 * (src/llm/layers/attention.cc:418-507, 98-170).
 *   qkv          [rows, 3E], head h at columns h*D.. of each third
 *   out          [rows, E]   (same storage type as qkv)
 *   maxima       [rows/T * H, T] fp32, max of the scaled visible scores
 *   normalizers  [rows/T * H, T] fp32, sum of exp(score - max)
 * rows must be a positive multiple of context_length and E of num_heads. */
int pluto_hip_mha_forward(void* stream, int dtype, const void* qkv, int rows,
                          int context_length, int num_heads, int embedding_dim,
                          void* out, float* maxima, float* normalizers);

/* AttentionProbabilitiesKernel (src/llm/layers/attention.cc:176-230):
 * fp32 probabilities [rows/T, H, T, T] rebuilt from the saved statistics,
 * zeros above the diagonal. */
int pluto_hip_mha_probabilities(void* stream, int dtype, const void* qkv,
                                const float* maxima, const float* normalizers,
                                int rows, int context_length, int num_heads,
                                int embedding_dim, float* probabilities);

/* AttentionLayer::bwd_impl + the two backward kernels
 * (src/llm/layers/attention.cc:509-596, 235-396).
 *   d_out   [rows, E] fp32 upstream gradient
 *   d_qkv   [rows, 3E] fp32, every element written exactly once
 * Deterministic: single-writer tiles, fixed reduction order, no atomics.
 * The workspace replaces the `deltas` buffer the reference allocates
 * (attention.cc:544) and holds the bf16 copy of d_out the MFMA path uses. */
size_t pluto_hip_mha_backward_workspace_bytes(int dtype, int rows,
                                              int context_length,
                                              int num_heads,
                                              int embedding_dim);
int pluto_hip_mha_backward(void* stream, int dtype, const void* qkv,
                           const void* out, const float* d_out,
                           const float* maxima, const float* normalizers,
                           int rows, int context_length, int num_heads,
                           int embedding_dim, float* d_qkv, void* workspace,
                           size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * Qwen style grouped-query attention with a contiguous KV cache.
 * --------------------------------------------------------------------- */

/* FullAttentionParameters (src/llm/layers/util/cached_attention_ops.h:13-22);
 * round_to_bfloat16 is an int here. */
typedef struct {
  int query_heads;
  int key_value_heads;
  int head_dim;
  int rotary_dim;
  int capacity;
  float rms_norm_epsilon;
  float rope_theta;
  int round_to_bfloat16;
} pluto_hip_attention_params;

/* One sequence's K and V storage (KeyValueCache, src/llm/key_value_cache.h:
 * 25-57).  Element (token t, kv head h, channel c) of either tensor lives at
 * base[t * token_stride + h * head_stride + c].  The reference layout is FP32
 * token-major (token_stride = kh*d, head_stride = d); the native layout of
 * this library is BF16 head-major [kh, capacity, d] (token_stride = d,
 * head_stride = capacity*d), which is lossless while round_to_bfloat16 is set
 * because every stored value is then bf16 representable
 * (cached_attention_ops.cc:64-67,75-77). */
typedef struct {
  void* keys;
  void* values;
  int dtype; /* PLUTO_HIP_F32 or PLUTO_HIP_BF16 */
  long long token_stride;
  long long head_stride;
} pluto_hip_kv_cache_view;

/* ValidateCachedAttention (cached_attention_ops.cc:283-306), parameter part:
 * PLUTO_HIP_EINVAL for anything the reference rejects. */
int pluto_hip_attention_params_validate(const pluto_hip_attention_params* p);

/* Whole-sequence GQA ("prefill") with the semantics of
 * QwenAttentionLayer::SequenceForward (src/llm/layers/qwen_attention.cc:
 * 414-448: PrepareKernel :30-63, ForwardKernel :68-119) and the cache append
 * of PrepareAttentionKernel (cached_attention_ops.cc:72-77): rows
 * [start_position, start_position + length) of the cache are written, and
 * row i attends to cache rows [0, start_position + i].
 *   qg   bf16 [length, qh, 2, d]  (query at [..,0,:], gate logits at [..,1,:])
 *   k,v  bf16 [length, kh, d]
 *   q_norm, k_norm  fp32 [d], zero centred (multiplier 1 + w)
 *   out  bf16 [length, qh, d] = bf16(bf16(core) * bf16(sigmoid(gate)))
 *   lse  optional fp32 [length, qh]: max + log(normalizer) of each row
 *   saved  optional, pluto_hip_gqa_prefill_saved_bytes(...) bytes: what
 *        pluto_hip_gqa_prefill_backward would otherwise recompute (the
 *        attention output before the gate and the row statistics; the
 *        counterpart of the state SequenceForward hands to SequenceBackward,
 *        qwen_attention.cc:445-447, without its quadratic tensors).  Only for
 *        start_position 0 and where that size is not 0: round_to_bfloat16, a
 *        BF16 cache and head_dim 64 or 128; PLUTO_HIP_EUNSUPPORTED otherwise.
 * The quadratic probability tensor of the reference is not produced. */
size_t pluto_hip_gqa_prefill_workspace_bytes(const pluto_hip_attention_params* p,
                                             int length);
size_t pluto_hip_gqa_prefill_saved_bytes(const pluto_hip_attention_params* p,
                                         int length, int cache_dtype);
int pluto_hip_gqa_prefill(void* stream, const pluto_hip_attention_params* p,
                          int length, int start_position, const void* qg,
                          const void* k, const void* v, const float* q_norm,
                          const float* k_norm,
                          const pluto_hip_kv_cache_view* cache, void* out,
                          float* lse, void* saved, void* workspace,
                          size_t workspace_bytes);

/* Backward of the whole-sequence layer
 * (QwenAttentionLayer::SequenceBackward, qwen_attention.cc:450-499; kernels
 * GateBackward :124-141, QueryBackward :146-174, KeyValueBackward :179-199,
 * NormBackward :201-228, ReduceNorm :230-239).  Self-contained: it takes the
 * layer's inputs and recomputes what the forward pass derived from them, so
 * nothing quadratic (the reference saves probabilities and score gradients,
 * [qh, length, length] each) is kept between the passes.
 *   dy       fp32 [length, qh, d]     gradient of the layer output
 *   saved    optional: the block pluto_hip_gqa_prefill filled for the same
 *            inputs and parameters; the attention forward is then not repeated
 *            (a quarter of the call at length 8192).  NULL recomputes.
 *   dqg      fp32 [length, qh, 2, d]  query gradients at [..,0,:], gate at [..,1,:]
 *   dk, dv   fp32 [length, kh, d]
 *   dq_norm, dk_norm  optional fp32 [d]: the norm weights' gradients are ADDED
 *            to them (shared weights accumulate over calls, as in the
 *            reference); NULL skips that work.
 * Rounding points are treated as identities, with the rounded forward values
 * as operands where the reference uses them.  With round_to_bfloat16 set and
 * head_dim 64 or 128 the attention part runs on the matrix cores with bf16
 * operands; all other cases run FP32 kernels. */
size_t pluto_hip_gqa_prefill_backward_workspace_bytes(const pluto_hip_attention_params* p,
                                                      int length, int q_weight_grad,
                                                      int k_weight_grad);
int pluto_hip_gqa_prefill_backward(void* stream, const pluto_hip_attention_params* p,
                                   int length, const void* qg, const void* k,
                                   const void* v, const float* q_norm,
                                   const float* k_norm, const float* dy,
                                   const void* saved, float* dqg, float* dk,
                                   float* dv, float* dq_norm, float* dk_norm,
                                   void* workspace, size_t workspace_bytes);

/* The FP32 probabilities tensor of the same ForwardKernel
 * (qwen_attention.cc:68-119, reported to attention_probabilities_hook at
 * :441-444), produced on request by a separate two-pass kernel:
 * probabilities [qh, length, start_position + length], zeros after each row's
 * visible prefix.  Must follow pluto_hip_gqa_prefill on the same stream with
 * the same parameters, cache and workspace: it reads the normalised, rotated
 * queries that call left in the workspace and the keys it appended. */
int pluto_hip_gqa_prefill_probabilities(void* stream,
                                        const pluto_hip_attention_params* p,
                                        int length, int start_position,
                                        const pluto_hip_kv_cache_view* cache,
                                        const void* workspace,
                                        size_t workspace_bytes,
                                        float* probabilities);

/* Batched single-token decode: `batch` independent CachedAttentionStep calls
 * (cached_attention_ops.cc:308-353: PrepareAttentionKernel :30-79,
 * FullAttentionKernel :83-126) in one launch sequence.  Sequence b appends
 * its token at row positions[b] of caches[b] and attends to rows
 * [0, positions[b]].  The caller advances its position counters after a
 * successful return (KeyValueCache::Advance).
 *   io_dtype  storage of q_gate, k, v and out: PLUTO_HIP_F32 (the reference's
 *             pointers) or PLUTO_HIP_BF16 (skips the four cast launches of
 *             qwen_attention.cc:381-386,409-411)
 *   q_gate [batch, qh, 2, d], k/v [batch, kh, d], out [batch, qh, d]
 *   positions, caches: HOST arrays of length batch
 *   probabilities: optional HOST array of `batch` device pointers (entries may
 *             be NULL), each fp32 [qh, positions[b] + 1]
 *             (AttentionProbabilitiesKernel, cached_attention_ops.cc:131-178)
 *   split_tokens: cache rows per split-K block: a multiple of 64 up to 512, or
 *             1024 at head width 256; 0 selects the default (512, and 1024
 *             at head width 256).  Anything else is PLUTO_HIP_EINVAL, and the
 *             workspace size is then reported as 0.
 * Returns PLUTO_HIP_ERANGE if any positions[b] >= capacity; nothing is
 * queued in that case. */
size_t pluto_hip_gqa_decode_workspace_bytes(const pluto_hip_attention_params* p,
                                            int batch, const int* positions,
                                            int split_tokens);
int pluto_hip_gqa_decode(void* stream, const pluto_hip_attention_params* p,
                         int batch, int io_dtype, const void* q_gate,
                         const void* k, const void* v, const float* q_norm,
                         const float* k_norm, const int* positions,
                         const pluto_hip_kv_cache_view* caches, void* out,
                         float* const* probabilities, int split_tokens,
                         void* workspace, size_t workspace_bytes);

/* pluto_hip_gqa_decode for callers that cannot allocate device memory or
 * pass a workspace: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  Same
 * arguments, results and errors as pluto_hip_gqa_decode (bit for bit), but the
 * scratch (prepared queries and split-K partial results) is a fixed array of
 * PLUTO_HIP_GQA_DECODE_STATIC_BYTES that the library keeps on every GPU it
 * runs on, and the call allocates nothing.  A call that would need more than
 * that (pluto_hip_gqa_decode_workspace_bytes says how much) returns
 * PLUTO_HIP_ELIMIT and queues nothing; the decode configuration (batch 32,
 * contexts up to 32768, 24 query heads of 128, 512-token blocks) needs about
 * 13 MiB.  All calls on one GPU share the array: calls that overlap there, on
 * whatever streams, race on it.  pluto_hip_gqa_decode_static_prepare looks
 * the array's device address up for the calling thread's current device (the
 * entry point does it itself on its first call there).
 * The array starts with the split-K arrival counters; every call that runs to
 * its end leaves them zero, which the next call relies on.  A call that
 * returns an error after queueing work marks the device, and the next call
 * there clears the counters first.  After anything else that may have left
 * them non-zero (calls that overlapped on one GPU, a kernel that was aborted)
 * queue pluto_hip_gqa_decode_static_reset(stream): one small fill kernel (no
 * memset node, so it may be recorded into a graph) that zeroes them all;
 * later calls on that stream then start clean. */
#define PLUTO_HIP_GQA_DECODE_STATIC_BYTES (16u << 20)
size_t pluto_hip_gqa_decode_static_bytes(void);
int pluto_hip_gqa_decode_static_prepare(void);
int pluto_hip_gqa_decode_static_reset(void* stream);
int pluto_hip_gqa_decode_static(void* stream, const pluto_hip_attention_params* p,
                                int batch, int io_dtype, const void* q_gate,
                                const void* k, const void* v, const float* q_norm,
                                const float* k_norm, const int* positions,
                                const pluto_hip_kv_cache_view* caches, void* out,
                                float* const* probabilities, int split_tokens);

/* ------------------------------------------------------------------------
 * Gated delta-net.
 * --------------------------------------------------------------------- */

/* DeltaNetParameters (cached_attention_ops.h:49-57). */
typedef struct {
  int key_heads;
  int value_heads;
  int key_head_dim;
  int value_head_dim;
  int conv_kernel_dim;
  float rms_norm_epsilon;
  int round_to_bfloat16;
} pluto_hip_delta_params;

/* Chunked scan of the gated delta rule; semantics of RecurrenceForward
 * (src/llm/layers/sequence_delta_net.cc:55-102) for `batch` independent
 * sequences, without the per-token state snapshots:
 *     S <- exp(g_t) S;  delta = (v_t - S^T k_t) beta_t;  S <- S + k_t delta^T
 *     o_t = S^T (q_t * q_scale)
 *   q, k        bf16 [batch, length, kh, kd]
 *   v           bf16 [batch, length, vh, vd]
 *   log_decay   fp32 [batch, length, vh]   (g_t <= 0)
 *   beta        fp32 [batch, length, vh]
 *   normalize_qk  when set, q and k are L2 normalised inside the kernel with
 *               1e-6 added to the sum of squares (sequence_delta_net.cc:84-85)
 *   state       fp32 [batch, vh, kd, vd], read as S_0, overwritten with S_T
 *   out         bf16 [batch, length, vh, vd]
 *   chunk       tokens per chunk (64); 0 selects the default. */
size_t pluto_hip_gdn_scan_workspace_bytes(const pluto_hip_delta_params* p,
                                          int batch, int length, int chunk);
int pluto_hip_gdn_scan(void* stream, const pluto_hip_delta_params* p,
                       int batch, int length, int chunk, const void* q,
                       const void* k, const void* v, const float* log_decay,
                       const float* beta, int normalize_qk, float q_scale,
                       float* state, void* out, void* workspace,
                       size_t workspace_bytes);

/* Token-by-token form of the same recurrence (the reference's own loop
 * structure); used for short sequences and as the device-side cross check
 * of the chunked scan.  Same arguments; out_dtype selects fp32 or bf16 `out`. */
int pluto_hip_gdn_recurrence(void* stream, const pluto_hip_delta_params* p,
                             int batch, int length, const void* q,
                             const void* k, const void* v,
                             const float* log_decay, const float* beta,
                             int normalize_qk, float q_scale, float* state,
                             void* out, int out_dtype);

/* Whole gated delta-net layer over sequences; semantics of
 * SequenceDeltaNetLayer::fwd_impl (src/llm/layers/sequence_delta_net.cc:435-480:
 * ConvForward :31-51, RecurrenceForward :55-102, OutputForward :104-121) for
 * `batch` independent sequences, each starting from an empty convolution history.
 *   qkv  bf16 [batch, length, 2*kh*kd + vh*vd], packed [all Q | all K | all V]
 *   z    bf16 [batch, length, vh*vd];  a, b  bf16 [batch, length, vh]
 *   conv_weight fp32 [channels, kernel]; a_log, dt_bias fp32 [vh]; norm fp32 [vd]
 *   state fp32 [batch, vh, kd, vd], read as the initial recurrent state (zeros for
 *        the reference's behaviour) and overwritten with the final one
 *   out  bf16 [batch, length, vh*vd]
 * The per-token state snapshots the reference saves for its backward pass are
 * not produced. */
size_t pluto_hip_gdn_layer_workspace_bytes(const pluto_hip_delta_params* p,
                                           int batch, int length);
int pluto_hip_gdn_layer_forward(void* stream, const pluto_hip_delta_params* p,
                                int batch, int length, const void* qkv,
                                const void* z, const void* a, const void* b,
                                const float* conv_weight, const float* a_log,
                                const float* dt_bias, const float* norm,
                                float* state, void* out, void* workspace,
                                size_t workspace_bytes);

/* Backward of the whole layer: SequenceDeltaNetLayer::bwd_impl
 * (sequence_delta_net.cc:482-561; kernels OutputBackward :125-155,
 * RecurrenceBackward :171-253, the two gathers :255-305, the convolution
 * backward kernels :307-355).  Self-contained: it takes the layer's inputs and
 * repeats the forward pass.  128 x 128 heads run in 64-token chunks on the
 * FP32 matrix cores and keep one state per chunk (about 0.8 MB of workspace
 * per chunk and value head); other head widths go token by token and keep the
 * recurrent state after every token ((length + 1) * vh * kd * vd floats, as
 * the reference's saved state does).  length <= 65535 and as far as the
 * workspace fits.  FP32 arithmetic throughout.
 *   dy    fp32 [batch, length, vh*vd]
 *   dqkv  fp32 [batch, length, channels];  dz fp32 [batch, length, vh*vd]
 *   da, db  fp32 [batch, length, vh]
 *   d_conv_weight [channels, kernel], d_a_log, d_dt_bias [vh], d_norm [vd]:
 *        optional; the parameters' gradients are ADDED to them. */
size_t pluto_hip_gdn_layer_backward_workspace_bytes(const pluto_hip_delta_params* p,
                                                    int length, int norm_grad);
int pluto_hip_gdn_layer_backward(void* stream, const pluto_hip_delta_params* p,
                                 int batch, int length, const void* qkv,
                                 const void* z, const void* a, const void* b,
                                 const float* conv_weight, const float* a_log,
                                 const float* dt_bias, const float* norm,
                                 const float* dy, float* dqkv, float* dz, float* da,
                                 float* db, float* d_conv_weight, float* d_a_log,
                                 float* d_dt_bias, float* d_norm, void* workspace,
                                 size_t workspace_bytes);

/* DeltaNetState::Step (src/llm/layers/util/cached_attention_ops.cc:401-431:
 * ConvolutionKernel :180-203, DeltaRecurrenceKernel :205-251, DeltaOutputKernel
 * :253-272): one token, contiguous FP32 device arrays as in the reference.
 *   conv_state fp32 [channels, kernel] and recurrent_state fp32 [vh, kd, vd]
 *   are updated in place (DeltaNetState::Reset = zero both). */
size_t pluto_hip_gdn_step_workspace_bytes(const pluto_hip_delta_params* p);
size_t pluto_hip_gdn_step_batch_workspace_bytes(const pluto_hip_delta_params* p,
                                                int batch);
int pluto_hip_gdn_step(void* stream, const pluto_hip_delta_params* p,
                       float* conv_state, float* recurrent_state,
                       const float* qkv, const float* z, const float* a,
                       const float* b, const float* conv_weight,
                       const float* a_log, const float* dt_bias,
                       const float* norm, float* output, void* workspace,
                       size_t workspace_bytes);

/* The same step for `batch` independent sequences in one set of launches: the
 * delta-net half of a decoder step lifted from batch one (Model::Step,
 * src/llm/qwen/model.cc:405-428, drives one DeltaNetState::Step per layer and
 * token) to the batch the cached attention entry point already takes.
 * Sequence s owns conv_states[s] ([batch, channels, kernel]) and
 * recurrent_states[s] ([batch, vh, kd, vd]); qkv [batch, channels], z and
 * output [batch, vh*vd], a and b [batch, vh]; the weights are shared.  Row s
 * of the result is bit for bit what pluto_hip_gdn_step gives for sequence s
 * alone.
 *   io_dtype  PLUTO_HIP_F32 or PLUTO_HIP_BF16: the element type of qkv, z, a,
 *             b and output.  With bf16 the step reads the layer's activations
 *             and writes its result directly, which replaces the four ToFloat
 *             launches and the ToBFloat16 launch of DeltaNetLayer::fwd_impl
 *             (src/llm/layers/delta_net.cc:70-102) with nothing: the result is
 *             bit for bit the FP32 step's output cast to bf16.  The states stay
 *             FP32. */
int pluto_hip_gdn_step_batch(void* stream, const pluto_hip_delta_params* p,
                             int batch, int io_dtype, float* conv_states,
                             float* recurrent_states, const void* qkv,
                             const void* z, const void* a, const void* b,
                             const float* conv_weight, const float* a_log,
                             const float* dt_bias, const float* norm,
                             void* output, void* workspace,
                             size_t workspace_bytes);

/* FullyConnectedLayer, trainable path: the projections either side of the
 * attention layers (src/llm/layers/fully_connected.cc: DenseForwardKernel
 * :97-131, DenseInputGradientKernel :134-164, DenseWeightGradientKernel
 * :167-196, the bias gradient kernels :198-247; fwd_impl :415-454, bwd_impl
 * :456-527).  dtype is the activation type (PLUTO_HIP_BF16 or PLUTO_HIP_F32;
 * anything else PLUTO_HIP_EUNSUPPORTED).  Operands are multiplied as bf16
 * (bf16 activations) or IEEE half (FP32 activations) values and summed in
 * FP32, as the reference's MmaType does (:31-33).
 *   input   [rows, input_dim] in dtype;  matrix fp32 [input_dim, output_dim];
 *   bias fp32 [output_dim];  output [rows, output_dim] in dtype
 *   d_output fp32 [rows, output_dim];  d_input fp32 [rows, input_dim]
 *   d_matrix, d_bias: shapes of the parameters, OVERWRITTEN (:190-196,241-246)
 * With output_dim = 3 * embedding_dim the forward output is the packed
 * [rows, Q | K | V] operand of pluto_hip_mha_forward, in its storage type.
 * Widths that are multiples of 64 run on the matrix cores; any other positive
 * width is accepted and takes a slower kernel with the same arithmetic. */
size_t pluto_hip_dense_workspace_bytes(int dtype, int rows, int input_dim,
                                       int output_dim);
int pluto_hip_dense_forward(void* stream, int dtype, const void* input,
                            const float* matrix, const float* bias, int rows,
                            int input_dim, int output_dim, void* output,
                            void* workspace, size_t workspace_bytes);
int pluto_hip_dense_backward(void* stream, int dtype, const void* input,
                             const float* matrix, const float* d_output,
                             int rows, int input_dim, int output_dim,
                             float* d_input, float* d_matrix, float* d_bias,
                             void* workspace, size_t workspace_bytes);

/* FullyConnectedLayer, imported path (src/llm/layers/fully_connected.cc:
 * ImportedMatVecKernel :40-68, QuantizeImportedInputKernel :70-88, Create
 * :267-293, ImportedForward :295-341; storage enum matrix_common.h:10): a
 * frozen checkpoint matrix, output-major [output_dim, input_dim], stored as
 * bf16, fp32 or OCP FP8 E4M3 with FP32 block scales
 * [ceil(output_dim/128), ceil(input_dim/128)], times ONE bf16 token
 * [input_dim] -> bf16 [output_dim].  All arithmetic is FP32.  With FP8 weights
 * the token is quantized first, in independent groups of 128 elements:
 * scale = max|x| / 448, x -> fp8(x / max(scale, 1e-12)) * scale.  `scales`
 * must be non-NULL exactly for FP8 storage; dimensions in [1, 1048576] (:271).
 * workspace: pluto_hip_dense_imported_workspace_bytes(input_dim) bytes. */
#define PLUTO_HIP_MATRIX_BF16 0
#define PLUTO_HIP_MATRIX_F32 1
#define PLUTO_HIP_MATRIX_FP8_E4M3 2
#define PLUTO_HIP_IMPORTED_MAX_DIM 1048576
#define PLUTO_HIP_IMPORTED_MAX_TOKENS 4096
size_t pluto_hip_dense_imported_workspace_bytes(int input_dim);
int pluto_hip_dense_imported_forward(void* stream, int storage,
                                     const void* weights, const float* scales,
                                     const void* input, int input_dim,
                                     int output_dim, void* output,
                                     void* workspace, size_t workspace_bytes);
/* The same projection for `tokens` independent tokens (the decoder step of
 * several sequences, qwen/model.cc:405-428 lifted from batch one): input bf16
 * [tokens, input_dim] -> output bf16 [tokens, output_dim].  Up to eight tokens
 * share one vector pass over the weights, and row t of the result is bit for
 * bit what the one-token call gives for token t; larger batches of bf16 or
 * FP8 weights with input_dim a multiple of 128 run on the matrix cores and
 * agree with the one-token calls to FP32 summation order. */
size_t pluto_hip_dense_imported_batch_workspace_bytes(int tokens, int input_dim);
int pluto_hip_dense_imported_forward_batch(void* stream, int storage,
                                           const void* weights,
                                           const float* scales,
                                           const void* input, int tokens,
                                           int input_dim, int output_dim,
                                           void* output, void* workspace,
                                           size_t workspace_bytes);
/* `matrices` (1..8) such projections of the SAME tokens in one call: the query
 * | gate, key and value projections of an attention branch, or the four input
 * projections of a delta-net branch, which the reference's block applies to
 * one hidden row one after the other (qwen/model.cc:174-274, each a
 * FullyConnectedLayer of its own; no single call of the reference
 * corresponds to this).  weights, scales (FP8 only, else NULL or all NULL),
 * output_dims and outputs are HOST arrays of `matrices` entries; all matrices
 * share storage and input_dim.  outputs[i] is bf16 [tokens, output_dims[i]] and
 * bit for bit what pluto_hip_dense_imported_forward_batch gives for matrix i;
 * the tokens are prepared once and every pass of 32 tokens is one launch
 * over all matrices (one call a matrix costs a fixed 14 us at 32 tokens,
 * whatever its size).  Workspace as for the batch call. */
#define PLUTO_HIP_IMPORTED_MAX_MATRICES 8
int pluto_hip_dense_imported_forward_many(void* stream, int storage,
                                          int matrices,
                                          const void* const* weights,
                                          const float* const* scales,
                                          const int* output_dims,
                                          const void* input, int tokens,
                                          int input_dim, void* const* outputs,
                                          void* workspace,
                                          size_t workspace_bytes);

/* ------------------------------------------------------------------------
 * Test support.  No counterpart in the reference.
 * --------------------------------------------------------------------- */

/* Routes the later calls of the CALLING THREAD through the any-shape
 * FP32-arithmetic kernels (enabled != 0) or back to normal kernel selection
 * (0), so that tests can compare the two implementations on the device.
 * Returns the thread's previous setting.  Thread-local, like the two hooks
 * below: a thread that never calls them always gets normal kernel selection,
 * and the library keeps no process-wide switches. */
int pluto_hip_test_force_generic(int enabled);

/* Measurement hook: entry points that queue several kernels skip those whose
 * class bit is cleared in `mask` (1 = the kernel that bounds the call: flash
 * attention forward, key-owned attention backward, split-K decode, delta-net
 * scan; 2 = the query-owned attention backward kernel; 4 = auxiliary kernels:
 * preparation, tables, combines; 16 = not a kernel: with this bit cleared the
 * attention forward and the key-owned attention backward keep to their
 * compiler-scheduled kernels whatever the sequence length, which lets a test
 * compare those with the kernels with hand-scheduled loops that longer
 * sequences take (forward: from 2048 rows at head widths 64 and 128, from 256
 * rows at 256; backward: from 4096 rows at head width 64); 32 = not a kernel
 * either: with this bit cleared (and 16 set) the backward and the forward at
 * head width 256 take their hand-scheduled kernels at every sequence length,
 * which extends that comparison, bit for bit, to small shapes).  A benchmark
 * runs the whole call once, then times one class with events around the call.  Returns the previous mask;
 * the default, ~0u, runs everything.  Thread-local like the switch above, and
 * like it written by nothing on the product path. */
unsigned pluto_hip_test_kernel_classes(unsigned mask);

/* Which family of kernels the calling thread's most recent compute call chose
 * (the entry points fall back to the any-shape kernels when a shape, stride
 * or alignment rules the specialised ones out; tests assert that the
 * configurations the library is built for do not).  Thread-local. */
#define PLUTO_HIP_PATH_NONE 0
#define PLUTO_HIP_PATH_GENERIC 1      /* any shape, FP32 arithmetic */
#define PLUTO_HIP_PATH_MATRIX_F32 2   /* FP32 storage on the FP32 matrix cores */
#define PLUTO_HIP_PATH_FLASH 3        /* bf16 flash attention on the matrix cores */
#define PLUTO_HIP_PATH_SPLIT_K 4      /* fused split-K decode */
#define PLUTO_HIP_PATH_CHUNKED 5      /* chunked delta-net (forward scan or backward) */
#define PLUTO_HIP_PATH_RECURRENCE 6   /* token-by-token delta-net */
int pluto_hip_test_last_path(void);

/* The tile lists the attention forward with the hand-scheduled loop would
 * launch with for a shape, computed on the host alone (no device is touched):
 * `items[w * *slots + e]` is entry e of workgroup w's list, (sequence *
 * query_heads + head) * q_tiles + q_tile with q_tiles = ceil(q_rows /
 * tile_rows), or 0xffff past the list's end; tile_rows is 256 at head width
 * 128 and 128 at 64 and 256.  `workgroups_resident` is what the launcher
 * derives from the device (compute units x workgroups a compute unit).
 * Returns 0 and sets *workgroups (0: the launch numbers its tiles by
 * workgroup index instead of lists) and *slots; PLUTO_HIP_EINVAL for a bad
 * argument, PLUTO_HIP_ELIMIT when `capacity` entries do not hold the lists.
 * Lets a test check, for any shape, that every tile is launched exactly once. */
int pluto_hip_test_forward_schedule(int head_dim, int q_rows, int kv_rows, int start_position,
                                    int query_heads, int group, int sequences,
                                    int workgroups_resident, uint16_t* items, int capacity,
                                    int* workgroups, int* slots);

#ifdef __cplusplus
}
#endif
#endif /* PLUTO_HIP_H_ */
