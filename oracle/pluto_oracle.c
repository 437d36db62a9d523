/*
 * pluto_oracle.c -- scalar CPU restatement of the reference's attention path.
 *
 * TEST INFRASTRUCTURE ONLY (see pluto_oracle.h).  Build with
 *   gcc -std=c11 -O2 -ffp-contract=off -fPIC -shared pluto_oracle.c -lm
 * -ffp-contract=off keeps every float operation separately rounded, as the
 * reference's `-O2` x86-64 build does.
 */
#include "pluto_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------------- */
/* bf16 helpers: src/llm/layers/reference_internal.h:109-119              */
/* ---------------------------------------------------------------------- */

uint16_t pluto_oracle_f32_to_bf16(float value) {
  uint32_t bits;
  memcpy(&bits, &value, sizeof bits);
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return (uint16_t)(bits >> 16);
}

float pluto_oracle_bf16_to_f32(uint16_t value) {
  uint32_t bits = (uint32_t)value << 16;
  float result;
  memcpy(&result, &bits, sizeof result);
  return result;
}

/* cached_attention_ops_test.cc:25-29 */
float pluto_oracle_bf16_round(float value) {
  return pluto_oracle_bf16_to_f32(pluto_oracle_f32_to_bf16(value));
}

/* reference_internal.h:190-203 */
static inline float load_activation(const void* buffer, size_t index,
                                    int dtype) {
  if (dtype == PLUTO_ORACLE_BF16)
    return pluto_oracle_bf16_to_f32(((const uint16_t*)buffer)[index]);
  return ((const float*)buffer)[index];
}

static inline void store_activation(void* buffer, size_t index, int dtype,
                                    float value) {
  if (dtype == PLUTO_ORACLE_BF16)
    ((uint16_t*)buffer)[index] = pluto_oracle_f32_to_bf16(value);
  else
    ((float*)buffer)[index] = value;
}

/* ---------------------------------------------------------------------- */
/* GPT-2 causal MHA: src/llm/layers/attention_reference.cc                */
/* ---------------------------------------------------------------------- */

static int mha_shape_ok(int rows, int context_length, int num_heads,
                        int embedding_dim) {
  /* attention_reference.cc:23-31,46-49 */
  if (context_length <= 0 || num_heads <= 0 || embedding_dim <= 0) return 0;
  if (embedding_dim % num_heads != 0) return 0;
  if (rows <= 0 || rows % context_length != 0) return 0;
  return 1;
}

int pluto_oracle_mha_fwd(int dtype, const void* qkv, int rows,
                         int context_length, int num_heads, int embedding_dim,
                         void* out, float* maxima, float* normalizers,
                         int seq_begin, int seq_end, int head_begin,
                         int head_end) {
  if (!mha_shape_ok(rows, context_length, num_heads, embedding_dim)) return -1;
  const int E = embedding_dim;
  const int head_dim = E / num_heads;
  const float scale = 1.0f / sqrtf((float)head_dim);
  float* scores = (float*)malloc(sizeof(float) * (size_t)context_length);
  if (!scores) return -1;
  /* attention_reference.cc:61-110: row, head, key loops in source order. */
  for (int row = seq_begin * context_length; row < seq_end * context_length;
       ++row) {
    const int sequence_start = (row / context_length) * context_length;
    const int query_position = row % context_length;
    for (int head = head_begin; head < head_end; ++head) {
      const int head_start = head * head_dim;
      float maximum = -INFINITY;
      for (int key_position = 0; key_position <= query_position;
           ++key_position) {
        const int key_row = sequence_start + key_position;
        float score = 0.0f;
        for (int dim = 0; dim < head_dim; ++dim) {
          const int column = head_start + dim;
          score += load_activation(qkv, (size_t)row * (3 * E) + column, dtype) *
                   load_activation(
                       qkv, (size_t)key_row * (3 * E) + E + column, dtype);
        }
        scores[key_position] = score * scale;
        maximum = fmaxf(maximum, scores[key_position]);
      }
      float denominator = 0.0f;
      for (int key_position = 0; key_position <= query_position;
           ++key_position) {
        scores[key_position] = expf(scores[key_position] - maximum);
        denominator += scores[key_position];
      }
      for (int dim = 0; dim < head_dim; ++dim) {
        const int column = head_start + dim;
        float value = 0.0f;
        for (int key_position = 0; key_position <= query_position;
             ++key_position) {
          const int key_row = sequence_start + key_position;
          value += (scores[key_position] / denominator) *
                   load_activation(
                       qkv, (size_t)key_row * (3 * E) + 2 * E + column, dtype);
        }
        store_activation(out, (size_t)row * E + column, dtype, value);
      }
      /* Statistics in the device layer's layout [B*H, T]
       * (src/llm/layers/attention.cc:128-131). */
      const size_t stat =
          ((size_t)(row / context_length) * num_heads + head) * context_length +
          query_position;
      if (maxima) maxima[stat] = maximum;
      if (normalizers) normalizers[stat] = denominator;
    }
  }
  free(scores);
  return 0;
}

int pluto_oracle_mha_bwd(int dtype, const void* qkv, const void* out,
                         const float* d_out, int rows, int context_length,
                         int num_heads, int embedding_dim, float* d_qkv,
                         int seq_begin, int seq_end, int head_begin,
                         int head_end) {
  if (!mha_shape_ok(rows, context_length, num_heads, embedding_dim)) return -1;
  const int E = embedding_dim;
  const int head_dim = E / num_heads;
  const float scale = 1.0f / sqrtf((float)head_dim);
  float* probabilities = (float*)malloc(sizeof(float) * (size_t)context_length);
  if (!probabilities) return -1;
  /* attention_reference.cc:146-228 */
  for (int row = seq_begin * context_length; row < seq_end * context_length;
       ++row) {
    const int sequence_start = (row / context_length) * context_length;
    const int query_position = row % context_length;
    for (int head = head_begin; head < head_end; ++head) {
      const int head_start = head * head_dim;
      float maximum = -INFINITY;
      for (int key_position = 0; key_position <= query_position;
           ++key_position) {
        const int key_row = sequence_start + key_position;
        float score = 0.0f;
        for (int dim = 0; dim < head_dim; ++dim) {
          const int column = head_start + dim;
          score += load_activation(qkv, (size_t)row * (3 * E) + column, dtype) *
                   load_activation(
                       qkv, (size_t)key_row * (3 * E) + E + column, dtype);
        }
        probabilities[key_position] = score * scale;
        maximum = fmaxf(maximum, probabilities[key_position]);
      }
      float denominator = 0.0f;
      for (int key_position = 0; key_position <= query_position;
           ++key_position) {
        probabilities[key_position] =
            expf(probabilities[key_position] - maximum);
        denominator += probabilities[key_position];
      }
      for (int key_position = 0; key_position <= query_position;
           ++key_position)
        probabilities[key_position] /= denominator;
      /* delta uses the STORED forward output (attention_reference.cc:181-189). */
      float delta = 0.0f;
      for (int dim = 0; dim < head_dim; ++dim) {
        const int column = head_start + dim;
        delta += d_out[(size_t)row * E + column] *
                 load_activation(out, (size_t)row * E + column, dtype);
      }
      for (int key_position = 0; key_position <= query_position;
           ++key_position) {
        const int key_row = sequence_start + key_position;
        float d_probability = 0.0f;
        for (int dim = 0; dim < head_dim; ++dim) {
          const int column = head_start + dim;
          d_probability +=
              d_out[(size_t)row * E + column] *
              load_activation(
                  qkv, (size_t)key_row * (3 * E) + 2 * E + column, dtype);
        }
        const float d_score =
            probabilities[key_position] * (d_probability - delta);
        for (int dim = 0; dim < head_dim; ++dim) {
          const int column = head_start + dim;
          const size_t q = (size_t)row * (3 * E) + column;
          const size_t k = (size_t)key_row * (3 * E) + E + column;
          const size_t v = (size_t)key_row * (3 * E) + 2 * E + column;
          d_qkv[q] += d_score * load_activation(qkv, k, dtype) * scale;
          d_qkv[k] += d_score * load_activation(qkv, q, dtype) * scale;
          d_qkv[v] +=
              probabilities[key_position] * d_out[(size_t)row * E + column];
        }
      }
    }
  }
  free(probabilities);
  return 0;
}

/* ---------------------------------------------------------------------- */
/* Qwen GQA: cached_attention_ops_test.cc:43-131                          */
/* ---------------------------------------------------------------------- */

static inline float round_if(const pluto_oracle_attention_params* p, float x) {
  return p->round_to_bfloat16 ? pluto_oracle_bf16_round(x) : x;
}

/* cached_attention_ops_test.cc:31 */
static inline float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }
static inline float silu_f32(float x) { return x * sigmoid_f32(x); }

static int attention_params_ok(const pluto_oracle_attention_params* p) {
  /* cached_attention_ops.cc:286-297 */
  if (p->query_heads <= 0 || p->key_value_heads <= 0 ||
      p->query_heads % p->key_value_heads != 0 || p->head_dim <= 0 ||
      p->head_dim > 256 || p->rotary_dim <= 0 ||
      p->rotary_dim > p->head_dim || p->rotary_dim % 2 != 0 ||
      !isfinite(p->rope_theta) || p->rope_theta <= 0.0f ||
      !isfinite(p->rms_norm_epsilon) || p->rms_norm_epsilon <= 0.0f)
    return 0;
  return 1;
}

void pluto_oracle_gqa_normalize_rotate(const pluto_oracle_attention_params* p,
                                       int position, const float* input,
                                       const float* weight, float* output) {
  /* cached_attention_ops_test.cc:56-78 */
  double square = 0.0;
  for (int d = 0; d < p->head_dim; ++d) square += input[d] * input[d];
  const double inverse =
      1.0 / sqrt(square / p->head_dim + p->rms_norm_epsilon);
  for (int d = 0; d < p->head_dim; ++d)
    output[d] = round_if(p, (float)(input[d] * inverse * (1.0 + weight[d])));
  for (int d = 0; d < p->rotary_dim / 2; ++d) {
    const int partner = d + p->rotary_dim / 2;
    const double angle =
        position * pow(p->rope_theta, -2.0 * d / p->rotary_dim);
    const float first = output[d];
    const float second = output[partner];
    const float cosine = round_if(p, (float)cos(angle));
    const float sine = round_if(p, (float)sin(angle));
    output[d] =
        round_if(p, round_if(p, first * cosine) - round_if(p, second * sine));
    output[partner] =
        round_if(p, round_if(p, second * cosine) + round_if(p, first * sine));
  }
}

/* Softmax(q.K/sqrt(d)) V and the sigmoid gate for one query head:
 * cached_attention_ops_test.cc:86-114.  keys/values rows are addressed as
 * base + t*token_stride. */
static void attend_head(const pluto_oracle_attention_params* p, int length,
                        const float* query, const float* gate,
                        const float* keys, const float* values,
                        size_t token_stride, double* scratch, float* output,
                        float* probabilities_out, float* lse_out) {
  const int d = p->head_dim;
  for (int t = 0; t < length; ++t) {
    double score = 0;
    const float* key = keys + (size_t)t * token_stride;
    for (int c = 0; c < d; ++c) score += query[c] * key[c];
    scratch[t] = score / sqrt((double)d);
  }
  double maximum = scratch[0];
  for (int t = 1; t < length; ++t)
    if (scratch[t] > maximum) maximum = scratch[t];
  double normalizer = 0;
  for (int t = 0; t < length; ++t) {
    scratch[t] = exp(scratch[t] - maximum);
    normalizer += scratch[t];
  }
  if (probabilities_out)
    for (int t = 0; t < length; ++t)
      probabilities_out[t] = (float)(scratch[t] / normalizer);
  if (lse_out) *lse_out = (float)(maximum + log(normalizer));
  for (int c = 0; c < d; ++c) {
    double sum = 0;
    for (int t = 0; t < length; ++t)
      sum += scratch[t] * values[(size_t)t * token_stride + c] / normalizer;
    output[c] = round_if(
        p, round_if(p, (float)sum) * round_if(p, sigmoid_f32(gate[c])));
  }
}

int pluto_oracle_gqa_cached_step(const pluto_oracle_attention_params* p,
                                 float* cache_keys, float* cache_values,
                                 int position, const float* q_gate,
                                 const float* k, const float* v,
                                 const float* q_norm, const float* k_norm,
                                 float* output, float* probabilities) {
  if (!attention_params_ok(p) || p->capacity <= 0 || position < 0) return -1;
  if (position >= p->capacity) return -2; /* cached_attention_ops.cc:318-320 */
  const int d = p->head_dim, qh = p->query_heads, kh = p->key_value_heads;
  const int length = position + 1;
  float* queries = (float*)malloc(sizeof(float) * (size_t)qh * d);
  double* scratch = (double*)malloc(sizeof(double) * (size_t)length);
  if (!queries || !scratch) {
    free(queries);
    free(scratch);
    return -1;
  }
  for (int h = 0; h < qh; ++h)
    pluto_oracle_gqa_normalize_rotate(p, position, q_gate + (size_t)h * 2 * d,
                                      q_norm, queries + (size_t)h * d);
  /* Append: row `position` of the token-major cache
   * (cached_attention_ops.cc:72-77). */
  for (int h = 0; h < kh; ++h) {
    float* key_row = cache_keys + ((size_t)position * kh + h) * d;
    float* value_row = cache_values + ((size_t)position * kh + h) * d;
    pluto_oracle_gqa_normalize_rotate(p, position, k + (size_t)h * d, k_norm,
                                      key_row);
    for (int c = 0; c < d; ++c) value_row[c] = round_if(p, v[(size_t)h * d + c]);
  }
  for (int h = 0; h < qh; ++h) {
    const int kv = h / (qh / kh);
    attend_head(p, length, queries + (size_t)h * d,
                q_gate + ((size_t)2 * h + 1) * d, cache_keys + (size_t)kv * d,
                cache_values + (size_t)kv * d, (size_t)kh * d, scratch,
                output + (size_t)h * d,
                probabilities ? probabilities + (size_t)h * length : NULL,
                NULL);
  }
  free(queries);
  free(scratch);
  return 0;
}

int pluto_oracle_gqa_sequence(const pluto_oracle_attention_params* p,
                              int length, const float* qg, const float* k,
                              const float* v, const float* q_norm,
                              const float* k_norm, float* out, float* key_out,
                              float* value_out, float* lse, int row_begin,
                              int row_end, int head_begin, int head_end) {
  if (!attention_params_ok(p) || length <= 0 || row_begin < 0 ||
      row_end > length || head_begin < 0 || head_end > p->query_heads)
    return -1;
  const int d = p->head_dim, qh = p->query_heads, kh = p->key_value_heads;
  const size_t kv_elements = (size_t)row_end * kh * d;
  float* keys = (float*)malloc(sizeof(float) * kv_elements);
  float* values = (float*)malloc(sizeof(float) * kv_elements);
  float* query = (float*)malloc(sizeof(float) * (size_t)d);
  double* scratch = (double*)malloc(sizeof(double) * (size_t)row_end);
  if (!keys || !values || !query || !scratch) {
    free(keys);
    free(values);
    free(query);
    free(scratch);
    return -1;
  }
  /* Row t is prepared at position t (qwen_attention.cc:54, "float(row)"). */
  for (int t = 0; t < row_end; ++t)
    for (int h = 0; h < kh; ++h) {
      const size_t at = ((size_t)t * kh + h) * d;
      pluto_oracle_gqa_normalize_rotate(p, t, k + at, k_norm, keys + at);
      for (int c = 0; c < d; ++c) values[at + c] = round_if(p, v[at + c]);
    }
  if (key_out) memcpy(key_out, keys, sizeof(float) * kv_elements);
  if (value_out) memcpy(value_out, values, sizeof(float) * kv_elements);
  for (int row = row_begin; row < row_end; ++row)
    for (int h = head_begin; h < head_end; ++h) {
      const int kv = h / (qh / kh);
      const size_t base = ((size_t)row * qh + h) * 2 * d;
      pluto_oracle_gqa_normalize_rotate(p, row, qg + base, q_norm, query);
      attend_head(p, row + 1, query, qg + base + d, keys + (size_t)kv * d,
                  values + (size_t)kv * d, (size_t)kh * d, scratch,
                  out + ((size_t)row * qh + h) * d, NULL,
                  lse ? lse + (size_t)row * qh + h : NULL);
    }
  free(keys);
  free(values);
  free(query);
  free(scratch);
  return 0;
}

/* Backward of the whole-sequence layer: the five kernels of
 * qwen_attention.cc:124-239 as launched by SequenceBackward (:450-499), in
 * double precision.  Rounding points have derivative one; the operands are the
 * values the reference's kernels use: dC = dy * Round(sigmoid) and
 * d gate = dy * Round(core) * s(1-s) (:136-140); delta = dC . core with the
 * unrounded core (:160-161); dS = P (dC . V - delta) (:168); dQ = sum dS K
 * scale (:170); dK = sum dS Q scale, dV = sum P dC over the later rows of the
 * kv head's query heads (:189-196); RoPE transposed with the rounded cos/sin
 * and RMSNorm backward (:213-227); weight gradients are added to dq_norm /
 * dk_norm (:230-239). */
static void norm_rope_backward(const pluto_oracle_attention_params* p, int row,
                               const float* input, const float* weight,
                               const double* grad, double* dx, double* dw) {
  const int d = p->head_dim, rotary = p->rotary_dim, half = rotary / 2;
  double normalized[256];
  for (int c = 0; c < d; ++c) {
    double ng = grad[c];
    if (c < rotary) {
      const int frequency = c < half ? c : c - half;
      const double angle = row * pow(p->rope_theta, -2.0 * frequency / rotary);
      const double co = round_if(p, (float)cos(angle));
      const double si = round_if(p, (float)sin(angle));
      const double partner = grad[c < half ? c + half : c - half];
      ng = grad[c] * co + (c < half ? partner * si : -partner * si);
    }
    normalized[c] = ng;
  }
  double square = 0.0;
  for (int c = 0; c < d; ++c) square += (double)input[c] * input[c];
  const double inv = 1.0 / sqrt(square / d + p->rms_norm_epsilon);
  double dot = 0.0;
  for (int c = 0; c < d; ++c) dot += normalized[c] * (1.0 + weight[c]) * input[c];
  for (int c = 0; c < d; ++c) {
    dx[c] = inv * normalized[c] * (1.0 + weight[c]) -
            input[c] * (inv * inv * inv / d) * dot;
    if (dw) dw[c] += normalized[c] * input[c] * inv;
  }
}

int pluto_oracle_gqa_sequence_backward(const pluto_oracle_attention_params* p,
                                       int length, const float* qg, const float* k,
                                       const float* v, const float* q_norm,
                                       const float* k_norm, const float* dy,
                                       float* dqg, float* dk, float* dv,
                                       float* dq_norm, float* dk_norm) {
  if (!attention_params_ok(p) || length <= 0) return -1;
  const int d = p->head_dim, qh = p->query_heads, kh = p->key_value_heads;
  const int group = qh / kh;
  const size_t qn = (size_t)length * qh * d, kn = (size_t)length * kh * d;
  const double scale = 1.0 / sqrt((double)d);
  float* queries = (float*)malloc(sizeof(float) * qn);
  float* keys = (float*)malloc(sizeof(float) * kn);
  float* values = (float*)malloc(sizeof(float) * kn);
  double* dq_rope = (double*)calloc(qn, sizeof(double));
  double* dk_rope = (double*)calloc(kn, sizeof(double));
  double* dv_sum = (double*)calloc(kn, sizeof(double));
  double* prob = (double*)malloc(sizeof(double) * (size_t)length);
  double* dq_weight = (double*)calloc((size_t)d, sizeof(double));
  double* dk_weight = (double*)calloc((size_t)d, sizeof(double));
  if (!queries || !keys || !values || !dq_rope || !dk_rope || !dv_sum || !prob ||
      !dq_weight || !dk_weight) {
    free(queries); free(keys); free(values); free(dq_rope); free(dk_rope);
    free(dv_sum); free(prob); free(dq_weight); free(dk_weight);
    return -1;
  }
  for (int t = 0; t < length; ++t) {
    for (int h = 0; h < kh; ++h) {
      const size_t at = ((size_t)t * kh + h) * d;
      pluto_oracle_gqa_normalize_rotate(p, t, k + at, k_norm, keys + at);
      for (int c = 0; c < d; ++c) values[at + c] = round_if(p, v[at + c]);
    }
    for (int h = 0; h < qh; ++h)
      pluto_oracle_gqa_normalize_rotate(p, t, qg + ((size_t)t * qh + h) * 2 * d, q_norm,
                                        queries + ((size_t)t * qh + h) * d);
  }
  for (int row = 0; row < length; ++row)
    for (int h = 0; h < qh; ++h) {
      const int kv = h / group;
      const float* query = queries + ((size_t)row * qh + h) * d;
      double maximum = -INFINITY;
      for (int t = 0; t <= row; ++t) {
        double score = 0.0;
        const float* key = keys + ((size_t)t * kh + kv) * d;
        for (int c = 0; c < d; ++c) score += (double)query[c] * key[c];
        prob[t] = score * scale;
        if (prob[t] > maximum) maximum = prob[t];
      }
      double normalizer = 0.0;
      for (int t = 0; t <= row; ++t) {
        prob[t] = exp(prob[t] - maximum);
        normalizer += prob[t];
      }
      for (int t = 0; t <= row; ++t) prob[t] /= normalizer;
      double dc[256];
      double delta = 0.0;
      for (int c = 0; c < d; ++c) {
        double sum = 0.0;
        for (int t = 0; t <= row; ++t) sum += prob[t] * values[((size_t)t * kh + kv) * d + c];
        const size_t at = ((size_t)row * qh + h) * d + c;
        const double gate = qg[(((size_t)row * qh + h) * 2 + 1) * d + c];
        const double sigmoid = 1.0 / (1.0 + exp(-gate));
        const double grad = dy[at];
        dc[c] = grad * round_if(p, (float)sigmoid);
        dqg[(((size_t)row * qh + h) * 2 + 1) * d + c] =
            (float)(grad * round_if(p, (float)sum) * sigmoid * (1.0 - sigmoid));
        delta += dc[c] * sum;
      }
      for (int t = 0; t <= row; ++t) {
        const size_t kv_at = ((size_t)t * kh + kv) * d;
        double dp = 0.0;
        for (int c = 0; c < d; ++c) dp += dc[c] * values[kv_at + c];
        const double ds = prob[t] * (dp - delta);
        for (int c = 0; c < d; ++c) {
          dq_rope[((size_t)row * qh + h) * d + c] += ds * keys[kv_at + c] * scale;
          dk_rope[kv_at + c] += ds * query[c] * scale;
          dv_sum[kv_at + c] += prob[t] * dc[c];
        }
      }
    }
  double dx[256];
  for (int row = 0; row < length; ++row) {
    for (int h = 0; h < qh; ++h) {
      const size_t unit = (size_t)row * qh + h;
      norm_rope_backward(p, row, qg + unit * 2 * d, q_norm, dq_rope + unit * d, dx,
                         dq_norm ? dq_weight : NULL);
      for (int c = 0; c < d; ++c) dqg[unit * 2 * d + c] = (float)dx[c];
    }
    for (int h = 0; h < kh; ++h) {
      const size_t unit = (size_t)row * kh + h;
      norm_rope_backward(p, row, k + unit * d, k_norm, dk_rope + unit * d, dx,
                         dk_norm ? dk_weight : NULL);
      for (int c = 0; c < d; ++c) {
        dk[unit * d + c] = (float)dx[c];
        dv[unit * d + c] = (float)dv_sum[unit * d + c];
      }
    }
  }
  for (int c = 0; c < d; ++c) {
    if (dq_norm) dq_norm[c] += (float)dq_weight[c];
    if (dk_norm) dk_norm[c] += (float)dk_weight[c];
  }
  free(queries); free(keys); free(values); free(dq_rope); free(dk_rope);
  free(dv_sum); free(prob); free(dq_weight); free(dk_weight);
  return 0;
}

int pluto_oracle_gqa_attend(const pluto_oracle_attention_params* p, int length,
                            size_t head_stride, const float* q,
                            const float* gate, const float* keys,
                            const float* values, float* output) {
  if (!attention_params_ok(p) || length <= 0) return -1;
  const int d = p->head_dim, qh = p->query_heads, kh = p->key_value_heads;
  double* scratch = (double*)malloc(sizeof(double) * (size_t)length);
  if (!scratch) return -1;
  for (int h = 0; h < qh; ++h) {
    const int kv = h / (qh / kh);
    attend_head(p, length, q + (size_t)h * d, gate + (size_t)h * d,
                keys + (size_t)kv * head_stride,
                values + (size_t)kv * head_stride, (size_t)d, scratch,
                output + (size_t)h * d, NULL, NULL);
  }
  free(scratch);
  return 0;
}

/* ---------------------------------------------------------------------- */
/* Gated delta-net                                                        */
/* ---------------------------------------------------------------------- */

static inline double round_bf16_f64(double x, int enabled) {
  /* sequence_delta_net_test.cc:81-91: narrow to float, then to bf16. */
  if (!enabled) return x;
  return (double)pluto_oracle_bf16_round((float)x);
}

static int delta_params_ok(const pluto_oracle_delta_params* p) {
  /* cached_attention_ops.cc:376-383 */
  if (p->key_heads <= 0 || p->value_heads <= 0 ||
      p->value_heads % p->key_heads != 0 || p->key_head_dim <= 0 ||
      p->value_head_dim <= 0 || p->conv_kernel_dim <= 0 ||
      !isfinite(p->rms_norm_epsilon) || p->rms_norm_epsilon <= 0.0f)
    return 0;
  return 1;
}

/* One token of one head: sequence_delta_net_test.cc:102-140. q and k are the
 * raw key-head vectors; decay and beta are already evaluated. */
static void delta_token(int kd, int vd, const double* q_in, const double* k_in,
                        const double* v, int normalize_qk, double q_scale,
                        double decay, double beta, double* state,
                        double* q_tmp, double* k_tmp, double* core) {
  double q_norm = 1e-6, k_norm = 1e-6;
  for (int d = 0; d < kd; ++d) {
    q_tmp[d] = q_in[d];
    k_tmp[d] = k_in[d];
    q_norm += q_tmp[d] * q_tmp[d];
    k_norm += k_tmp[d] * k_tmp[d];
  }
  for (int d = 0; d < kd; ++d) {
    if (normalize_qk) {
      q_tmp[d] /= sqrt(q_norm);
      k_tmp[d] /= sqrt(k_norm);
    }
    q_tmp[d] *= q_scale;
  }
  for (int channel = 0; channel < vd; ++channel) {
    double prediction = 0;
    for (int d = 0; d < kd; ++d) {
      const size_t i = (size_t)d * vd + channel;
      state[i] *= decay;
      prediction += state[i] * k_tmp[d];
    }
    const double delta = (v[channel] - prediction) * beta;
    double output = 0;
    for (int d = 0; d < kd; ++d) {
      const size_t i = (size_t)d * vd + channel;
      state[i] += k_tmp[d] * delta;
      output += state[i] * q_tmp[d];
    }
    core[channel] = output;
  }
}

int pluto_oracle_gdn_scan(const pluto_oracle_delta_params* p, int length,
                          const float* q, const float* k, const float* v,
                          const float* log_decay, const float* beta,
                          int normalize_qk, double q_scale, double* state,
                          float* core, int head_begin, int head_end) {
  if (!delta_params_ok(p) || length <= 0 || head_begin < 0 ||
      head_end > p->value_heads)
    return -1;
  const int kh = p->key_heads, vh = p->value_heads;
  const int kd = p->key_head_dim, vd = p->value_head_dim;
  double* tmp = (double*)malloc(sizeof(double) * (size_t)(4 * kd + 2 * vd));
  if (!tmp) return -1;
  double *qd = tmp, *kdv = tmp + kd, *qt = tmp + 2 * kd, *kt = tmp + 3 * kd;
  double *vv = tmp + 4 * kd, *out = tmp + 4 * kd + vd;
  for (int head = head_begin; head < head_end; ++head) {
    const int key_head = head / (vh / kh);
    double* head_state = state + (size_t)head * kd * vd;
    for (int t = 0; t < length; ++t) {
      for (int d = 0; d < kd; ++d) {
        qd[d] = q[((size_t)t * kh + key_head) * kd + d];
        kdv[d] = k[((size_t)t * kh + key_head) * kd + d];
      }
      for (int c = 0; c < vd; ++c) vv[c] = v[((size_t)t * vh + head) * vd + c];
      const double decay = exp((double)log_decay[(size_t)t * vh + head]);
      delta_token(kd, vd, qd, kdv, vv, normalize_qk, q_scale, decay,
                  (double)beta[(size_t)t * vh + head], head_state, qt, kt, out);
      for (int c = 0; c < vd; ++c)
        core[((size_t)t * vh + head) * vd + c] =
            (float)round_bf16_f64(out[c], p->round_to_bfloat16);
    }
  }
  free(tmp);
  return 0;
}

int pluto_oracle_gdn_sequence(const pluto_oracle_delta_params* p, int length,
                              const float* qkv, const float* z, const float* a,
                              const float* b, const float* conv_weight,
                              const float* a_log, const float* dt_bias,
                              const float* norm, float* output, float* core_out,
                              double* final_state) {
  if (!delta_params_ok(p) || length <= 0) return -1;
  const int kh = p->key_heads, vh = p->value_heads;
  const int kd = p->key_head_dim, vd = p->value_head_dim;
  const int kernel = p->conv_kernel_dim;
  const int channels = 2 * kh * kd + vh * vd;
  const int round = p->round_to_bfloat16;
  double* convolved =
      (double*)malloc(sizeof(double) * (size_t)length * channels);
  double* states = (double*)calloc((size_t)vh * kd * vd, sizeof(double));
  double* core = (double*)malloc(sizeof(double) * (size_t)length * vh * vd);
  double* tmp = (double*)malloc(sizeof(double) * (size_t)(4 * kd + 2 * vd));
  if (!convolved || !states || !core || !tmp) {
    free(convolved);
    free(states);
    free(core);
    free(tmp);
    return -1;
  }
  /* sequence_delta_net_test.cc:92-104: causal depthwise conv + SiLU. */
  for (int t = 0; t < length; ++t)
    for (int c = 0; c < channels; ++c) {
      double sum = 0;
      for (int tap = 0; tap < kernel; ++tap) {
        const int source = t + tap - kernel + 1;
        if (source >= 0)
          sum += (double)qkv[(size_t)source * channels + c] *
                 (double)conv_weight[(size_t)c * kernel + tap];
      }
      sum = round_bf16_f64(sum, round);
      convolved[(size_t)t * channels + c] =
          round_bf16_f64(sum / (1 + exp(-sum)), round);
    }
  double *qd = tmp, *kdv = tmp + kd, *qt = tmp + 2 * kd, *kt = tmp + 3 * kd;
  double *vv = tmp + 4 * kd, *out = tmp + 4 * kd + vd;
  /* sequence_delta_net_test.cc:107-141 */
  for (int head = 0; head < vh; ++head) {
    const int key_head = head / (vh / kh);
    double* head_state = states + (size_t)head * kd * vd;
    for (int t = 0; t < length; ++t) {
      for (int d = 0; d < kd; ++d) {
        qd[d] = convolved[(size_t)t * channels + key_head * kd + d];
        kdv[d] = convolved[(size_t)t * channels + (kh + key_head) * kd + d];
      }
      for (int c = 0; c < vd; ++c)
        vv[c] = convolved[(size_t)t * channels + 2 * kh * kd + head * vd + c];
      const double alpha =
          (double)a[(size_t)t * vh + head] + (double)dt_bias[head];
      const double softplus =
          fmax(alpha, 0.) + log1p(exp(-fabs(alpha)));
      const double decay = exp(-exp((double)a_log[head]) * softplus);
      const double beta = round_bf16_f64(
          1 / (1 + exp(-(double)b[(size_t)t * vh + head])), round);
      /* sequence_delta_net_test.cc:111-121, literally. */
      double q_norm = 1e-6, k_norm = 1e-6;
      for (int d = 0; d < kd; ++d) {
        q_norm += qd[d] * qd[d];
        k_norm += kdv[d] * kdv[d];
      }
      for (int d = 0; d < kd; ++d) {
        qd[d] /= sqrt(q_norm * kd);
        kdv[d] /= sqrt(k_norm);
      }
      delta_token(kd, vd, qd, kdv, vv, 0, 1.0, decay, beta, head_state, qt, kt,
                  out);
      for (int c = 0; c < vd; ++c)
        core[((size_t)t * vh + head) * vd + c] = round_bf16_f64(out[c], round);
    }
  }
  /* sequence_delta_net_test.cc:143-157: RMSNorm, plain weight, SiLU(z). */
  for (int row = 0; row < length * vh; ++row) {
    double sum = 0;
    for (int d = 0; d < vd; ++d)
      sum += core[(size_t)row * vd + d] * core[(size_t)row * vd + d];
    const double inverse = 1 / sqrt(sum / vd + (double)p->rms_norm_epsilon);
    for (int d = 0; d < vd; ++d) {
      const size_t i = (size_t)row * vd + d;
      const double normalized = round_bf16_f64(core[i] * inverse, round);
      const double affine = round_bf16_f64(normalized * (double)norm[d], round);
      const double gate = (double)z[i];
      output[i] = (float)round_bf16_f64(affine * gate / (1 + exp(-gate)), 1);
    }
  }
  if (core_out)
    for (size_t i = 0; i < (size_t)length * vh * vd; ++i)
      core_out[i] = (float)core[i];
  if (final_state)
    memcpy(final_state, states, sizeof(double) * (size_t)vh * kd * vd);
  free(convolved);
  free(states);
  free(core);
  free(tmp);
  return 0;
}

/* Backward of the whole layer: SequenceDeltaNetLayer::bwd_impl
 * (sequence_delta_net.cc:482-561) with its kernels OutputBackward (:125-155),
 * SumNormGradient (:157-166), RecurrenceBackward (:171-253), GatherQkGradient
 * (:255-276), GatherScalarGradient (:278-305), ConvSiluBackward (:307-318),
 * ConvInputBackward (:320-336), ConvWeightBackward (:338-355), in double
 * precision.  Rounding points have derivative one; the operands are the saved
 * (rounded) forward values where the reference reads them from its saved
 * state.  Parameter gradients (nullable) are added to. */
int pluto_oracle_gdn_sequence_backward(
    const pluto_oracle_delta_params* p, int length, const float* qkv, const float* z,
    const float* a, const float* b, const float* conv_weight, const float* a_log,
    const float* dt_bias, const float* norm, const float* dy, float* dqkv, float* dz,
    float* da, float* db, float* d_conv_weight, float* d_a_log, float* d_dt_bias,
    float* d_norm) {
  if (!delta_params_ok(p) || length <= 0) return -1;
  const int kh = p->key_heads, vh = p->value_heads;
  const int kd = p->key_head_dim, vd = p->value_head_dim;
  const int kernel = p->conv_kernel_dim;
  const int channels = 2 * kh * kd + vh * vd;
  const int round = p->round_to_bfloat16;
  const size_t state_size = (size_t)kd * vd;
  double* pre = (double*)malloc(sizeof(double) * (size_t)length * channels);
  double* post = (double*)malloc(sizeof(double) * (size_t)length * channels);
  double* dpost = (double*)calloc((size_t)length * channels, sizeof(double));
  double* dpre = (double*)malloc(sizeof(double) * (size_t)length * channels);
  double* core = (double*)malloc(sizeof(double) * (size_t)length * vh * vd);
  double* dcore = (double*)malloc(sizeof(double) * (size_t)length * vh * vd);
  double* states = (double*)calloc((size_t)(length + 1) * state_size, sizeof(double));
  double* dm = (double*)malloc(sizeof(double) * state_size);
  double* tmp = (double*)malloc(sizeof(double) * (size_t)(8 * kd + 4 * vd));
  if (!pre || !post || !dpost || !dpre || !core || !dcore || !states || !dm || !tmp) {
    free(pre); free(post); free(dpost); free(dpre); free(core); free(dcore);
    free(states); free(dm); free(tmp);
    return -1;
  }
  for (int t = 0; t < length; ++t)
    for (int c = 0; c < channels; ++c) {
      double sum = 0;
      for (int tap = 0; tap < kernel; ++tap) {
        const int source = t + tap - kernel + 1;
        if (source >= 0)
          sum += (double)qkv[(size_t)source * channels + c] *
                 (double)conv_weight[(size_t)c * kernel + tap];
      }
      sum = round_bf16_f64(sum, round);
      pre[(size_t)t * channels + c] = sum;
      post[(size_t)t * channels + c] = round_bf16_f64(sum / (1 + exp(-sum)), round);
    }
  double *raw_q = tmp, *raw_k = tmp + kd, *q = tmp + 2 * kd, *k = tmp + 3 * kd;
  double *dq = tmp + 4 * kd, *dk = tmp + 5 * kd, *sum_q = tmp + 6 * kd, *sum_k = tmp + 7 * kd;
  double *v = tmp + 8 * kd, *difference = v + vd, *delta = v + 2 * vd, *ddelta = v + 3 * vd;
  for (int t = 0; t < length; ++t) {
    memset(da + (size_t)t * vh, 0, sizeof(float) * (size_t)vh);
    memset(db + (size_t)t * vh, 0, sizeof(float) * (size_t)vh);
  }
  for (int head = 0; head < vh; ++head) {
    const int key_head = head / (vh / kh);
    /* forward with every state kept (RecurrenceForward, :55-102) */
    memset(states, 0, sizeof(double) * state_size);
    for (int t = 0; t < length; ++t) {
      const double* row = post + (size_t)t * channels;
      double q_norm = 1e-6, k_norm = 1e-6;
      for (int d = 0; d < kd; ++d) {
        raw_q[d] = row[key_head * kd + d];
        raw_k[d] = row[(kh + key_head) * kd + d];
        q_norm += raw_q[d] * raw_q[d];
        k_norm += raw_k[d] * raw_k[d];
      }
      for (int d = 0; d < kd; ++d) {
        q[d] = raw_q[d] / sqrt(q_norm) / sqrt((double)kd);
        k[d] = raw_k[d] / sqrt(k_norm);
      }
      const double alpha = (double)a[(size_t)t * vh + head] + (double)dt_bias[head];
      const double softplus = fmax(alpha, 0.) + log1p(exp(-fabs(alpha)));
      const double decay = exp(-exp((double)a_log[head]) * softplus);
      const double beta =
          round_bf16_f64(1 / (1 + exp(-(double)b[(size_t)t * vh + head])), round);
      const double* previous = states + (size_t)t * state_size;
      double* next = states + (size_t)(t + 1) * state_size;
      for (int c = 0; c < vd; ++c) {
        double prediction = 0;
        for (int d = 0; d < kd; ++d) prediction += previous[(size_t)d * vd + c] * decay * k[d];
        const double dl = (row[2 * kh * kd + head * vd + c] - prediction) * beta;
        double out = 0;
        for (int d = 0; d < kd; ++d) {
          const double value = previous[(size_t)d * vd + c] * decay + k[d] * dl;
          next[(size_t)d * vd + c] = value;
          out += value * q[d];
        }
        core[((size_t)t * vh + head) * vd + c] = round_bf16_f64(out, round);
      }
    }
    /* OutputBackward (:125-155) for this head's rows */
    double norm_partial[256];
    for (int c = 0; c < vd; ++c) norm_partial[c] = 0;
    for (int t = 0; t < length; ++t) {
      const size_t base = ((size_t)t * vh + head) * vd;
      double sum = 0;
      for (int c = 0; c < vd; ++c) sum += core[base + c] * core[base + c];
      const double inverse = 1 / sqrt(sum / vd + (double)p->rms_norm_epsilon);
      double dot = 0;
      for (int c = 0; c < vd; ++c) {
        const double gate = (double)z[base + c];
        const double sigmoid = 1 / (1 + exp(-gate));
        const double dn = (double)dy[base + c] * gate * sigmoid * (double)norm[c];
        dot += dn * core[base + c];
      }
      for (int c = 0; c < vd; ++c) {
        const double x = core[base + c];
        const double gate = (double)z[base + c];
        const double sigmoid = 1 / (1 + exp(-gate));
        const double normalized = round_bf16_f64(x * inverse, round);
        const double affine = round_bf16_f64(normalized * (double)norm[c], round);
        const double dn = (double)dy[base + c] * gate * sigmoid * (double)norm[c];
        dcore[base + c] = inverse * dn - x * inverse * inverse * inverse / vd * dot;
        dz[base + c] = (float)((double)dy[base + c] * affine * sigmoid *
                               (1 + gate * (1 - sigmoid)));
        norm_partial[c] += (double)dy[base + c] * gate * sigmoid * normalized;
      }
    }
    if (d_norm)
      for (int c = 0; c < vd; ++c) d_norm[c] += (float)norm_partial[c];
    /* RecurrenceBackward (:171-253) */
    for (size_t i = 0; i < state_size; ++i) dm[i] = 0;
    double head_dalog = 0, head_dbias = 0;
    for (int t = length - 1; t >= 0; --t) {
      const double* row = post + (size_t)t * channels;
      double q_norm = 1e-6, k_norm = 1e-6;
      for (int d = 0; d < kd; ++d) {
        raw_q[d] = row[key_head * kd + d];
        raw_k[d] = row[(kh + key_head) * kd + d];
        q_norm += raw_q[d] * raw_q[d];
        k_norm += raw_k[d] * raw_k[d];
      }
      const double iq = 1 / sqrt(q_norm), ik = 1 / sqrt(k_norm);
      const double norm_scale = sqrt((double)kd);
      for (int d = 0; d < kd; ++d) {
        q[d] = raw_q[d] * iq / norm_scale;
        k[d] = raw_k[d] * ik;
      }
      const double alpha = (double)a[(size_t)t * vh + head] + (double)dt_bias[head];
      const double softplus = fmax(alpha, 0.) + log1p(exp(-fabs(alpha)));
      const double rate = exp((double)a_log[head]);
      const double decay = exp(-rate * softplus);
      const double sigmoid = 1 / (1 + exp(-(double)b[(size_t)t * vh + head]));
      const double beta = round_bf16_f64(sigmoid, round);
      const double* previous = states + (size_t)t * state_size;
      const double* matrix = states + (size_t)(t + 1) * state_size;
      const double* grad = dcore + ((size_t)t * vh + head) * vd;
      for (int c = 0; c < vd; ++c) {
        double prediction = 0;
        for (int d = 0; d < kd; ++d) prediction += previous[(size_t)d * vd + c] * decay * k[d];
        difference[c] = row[2 * kh * kd + head * vd + c] - prediction;
        delta[c] = difference[c] * beta;
      }
      for (int d = 0; d < kd; ++d) {
        double sum = 0;
        for (int c = 0; c < vd; ++c) {
          sum += matrix[(size_t)d * vd + c] * grad[c];
          dm[(size_t)d * vd + c] += q[d] * grad[c];
        }
        dq[d] = sum;
      }
      double dbeta = 0;
      for (int c = 0; c < vd; ++c) {
        double sum = 0;
        for (int d = 0; d < kd; ++d) sum += dm[(size_t)d * vd + c] * k[d];
        ddelta[c] = sum;
        dbeta += sum * difference[c];
        dpost[(size_t)t * channels + 2 * kh * kd + head * vd + c] = sum * beta;
      }
      double dg = 0;
      for (int d = 0; d < kd; ++d) {
        double sum = 0;
        for (int c = 0; c < vd; ++c) {
          const double dvalue = ddelta[c] * beta;
          const double decayed = previous[(size_t)d * vd + c] * decay;
          sum += dm[(size_t)d * vd + c] * delta[c] - decayed * dvalue;
          const double ddecayed = dm[(size_t)d * vd + c] - k[d] * dvalue;
          dg += ddecayed * previous[(size_t)d * vd + c];
          dm[(size_t)d * vd + c] = ddecayed * decay;
        }
        dk[d] = sum;
      }
      const double dalpha = -dg * decay * rate / (1 + exp(-alpha));
      da[(size_t)t * vh + head] = (float)dalpha;
      db[(size_t)t * vh + head] = (float)(dbeta * sigmoid * (1 - sigmoid));
      head_dalog += -dg * decay * rate * softplus;
      head_dbias += dalpha;
      double q_dot = 0, k_dot = 0;
      for (int d = 0; d < kd; ++d) {
        q_dot += dq[d] * raw_q[d];
        k_dot += dk[d] * raw_k[d];
      }
      for (int d = 0; d < kd; ++d) {
        sum_q[d] = (dq[d] * iq - raw_q[d] * iq * iq * iq * q_dot) / norm_scale;
        sum_k[d] = dk[d] * ik - raw_k[d] * ik * ik * ik * k_dot;
        /* GatherQkGradient (:255-276): heads of a key head add up */
        dpost[(size_t)t * channels + key_head * kd + d] += sum_q[d];
        dpost[(size_t)t * channels + (kh + key_head) * kd + d] += sum_k[d];
      }
    }
    if (d_a_log) d_a_log[head] += (float)head_dalog;
    if (d_dt_bias) d_dt_bias[head] += (float)head_dbias;
  }
  /* ConvSiluBackward, ConvInputBackward, ConvWeightBackward (:307-355) */
  for (size_t i = 0; i < (size_t)length * channels; ++i) {
    const double x = pre[i];
    const double sigmoid = 1 / (1 + exp(-x));
    dpre[i] = dpost[i] * sigmoid * (1 + x * (1 - sigmoid));
  }
  for (int t = 0; t < length; ++t)
    for (int c = 0; c < channels; ++c) {
      double sum = 0;
      for (int tap = 0; tap < kernel; ++tap) {
        const int future = t + kernel - 1 - tap;
        if (future < length)
          sum += dpre[(size_t)future * channels + c] *
                 (double)conv_weight[(size_t)c * kernel + tap];
      }
      dqkv[(size_t)t * channels + c] = (float)sum;
    }
  if (d_conv_weight)
    for (int c = 0; c < channels; ++c)
      for (int tap = 0; tap < kernel; ++tap) {
        double sum = 0;
        for (int t = kernel - 1 - tap; t < length; ++t)
          sum += dpre[(size_t)t * channels + c] *
                 (double)qkv[(size_t)(t + tap - kernel + 1) * channels + c];
        d_conv_weight[(size_t)c * kernel + tap] += (float)sum;
      }
  free(pre); free(post); free(dpost); free(dpre); free(core); free(dcore);
  free(states); free(dm); free(tmp);
  return 0;
}

int pluto_oracle_gdn_step(const pluto_oracle_delta_params* p,
                          float* conv_state, double* recurrent_state,
                          const float* qkv, const float* z, const float* a,
                          const float* b, const float* conv_weight,
                          const float* a_log, const float* dt_bias,
                          const float* norm, float* output) {
  if (!delta_params_ok(p)) return -1;
  const int kh = p->key_heads, vh = p->value_heads;
  const int kd = p->key_head_dim, vd = p->value_head_dim;
  const int kernel = p->conv_kernel_dim;
  const int channels = 2 * kh * kd + vh * vd;
  const int round = p->round_to_bfloat16;
#define ROUND_F32(x) (round ? pluto_oracle_bf16_round(x) : (x))
  float* convolved = (float*)malloc(sizeof(float) * (size_t)channels);
  double* q = (double*)malloc(sizeof(double) * (size_t)(2 * kd));
  if (!convolved || !q) {
    free(convolved);
    free(q);
    return -1;
  }
  double* k = q + kd;
  /* cached_attention_ops_test.cc:151-163 */
  for (int c = 0; c < channels; ++c) {
    for (int tap = 0; tap < kernel - 1; ++tap)
      conv_state[(size_t)c * kernel + tap] =
          conv_state[(size_t)c * kernel + tap + 1];
    conv_state[(size_t)(c + 1) * kernel - 1] = ROUND_F32(qkv[c]);
    double sum = 0;
    for (int tap = 0; tap < kernel; ++tap)
      sum += conv_state[(size_t)c * kernel + tap] *
             conv_weight[(size_t)c * kernel + tap];
    const float pre = ROUND_F32((float)sum);
    convolved[c] = ROUND_F32(silu_f32(pre));
  }
  /* cached_attention_ops_test.cc:164-216 */
  for (int h = 0; h < vh; ++h) {
    const int key_head = h / (vh / kh);
    double q_square = 1e-6, k_square = 1e-6;
    for (int d = 0; d < kd; ++d) {
      q[d] = convolved[key_head * kd + d];
      k[d] = convolved[(kh + key_head) * kd + d];
      q_square += q[d] * q[d];
      k_square += k[d] * k[d];
    }
    for (int d = 0; d < kd; ++d) {
      q[d] /= sqrt(q_square * kd);
      k[d] /= sqrt(k_square);
    }
    const double alpha = a[h] + dt_bias[h]; /* float sum, as in the source */
    const double softplus = fmax(alpha, 0.0) + log1p(exp(-fabs(alpha)));
    const double decay = exp(-exp((double)a_log[h]) * softplus);
    const float beta = ROUND_F32(sigmoid_f32(b[h]));
    for (int c = 0; c < vd; ++c) {
      double prediction = 0;
      for (int d = 0; d < kd; ++d) {
        const size_t i = ((size_t)h * kd + d) * vd + c;
        recurrent_state[i] *= decay;
        prediction += recurrent_state[i] * k[d];
      }
      const float value = convolved[2 * kh * kd + h * vd + c];
      const double delta = (value - prediction) * beta;
      double core = 0;
      for (int d = 0; d < kd; ++d) {
        const size_t i = ((size_t)h * kd + d) * vd + c;
        recurrent_state[i] += k[d] * delta;
        core += recurrent_state[i] * q[d];
      }
      output[(size_t)h * vd + c] = ROUND_F32((float)core);
    }
    double variance = 0;
    for (int c = 0; c < vd; ++c) {
      const double x = output[(size_t)h * vd + c];
      variance += x * x;
    }
    const double inverse =
        1.0 / sqrt(variance / vd + (double)p->rms_norm_epsilon);
    for (int c = 0; c < vd; ++c) {
      const size_t i = (size_t)h * vd + c;
      const float normalized = ROUND_F32((float)(output[i] * inverse));
      const float affine = ROUND_F32(normalized * norm[c]);
      output[i] = ROUND_F32(affine * silu_f32(z[i]));
    }
  }
#undef ROUND_F32
  free(convolved);
  free(q);
  return 0;
}

/* ---- FullyConnectedLayer (fully_connected.cc:97-247) -------------------- */

/* float -> IEEE binary16 -> float, round to nearest even, with subnormals and
 * overflow to infinity (what element_cast<__half> does). */
float pluto_oracle_half_round(float value) {
  if (isnan(value) || isinf(value)) return value;
  const float magnitude = fabsf(value);
  if (magnitude >= 65520.0f) return copysignf(INFINITY, value); /* above the largest half + 1/2 ulp */
  float scaled;
  if (magnitude < 6.103515625e-05f) {
    /* subnormal halves: multiples of 2^-24 */
    scaled = nearbyintf(magnitude * 16777216.0f) / 16777216.0f;
  } else {
    int exponent;
    const float mantissa = frexpf(magnitude, &exponent); /* in [0.5, 1) */
    scaled = ldexpf(nearbyintf(ldexpf(mantissa, 11)), exponent - 11);
  }
  return copysignf(scaled, value);
}

static float dense_operand(int dtype, float value) {
  return dtype == PLUTO_ORACLE_BF16 ? pluto_oracle_bf16_round(value)
                                    : pluto_oracle_half_round(value);
}

int pluto_oracle_dense_forward(int dtype, int rows, int input_dim, int output_dim,
                               const float* x, const float* matrix, const float* bias,
                               float* y) {
  if ((dtype != PLUTO_ORACLE_BF16 && dtype != PLUTO_ORACLE_F32) || rows <= 0 || input_dim <= 0 ||
      output_dim <= 0 || !x || !matrix || !bias || !y)
    return 1;
  for (int r = 0; r < rows; ++r)
    for (int o = 0; o < output_dim; ++o) {
      double sum = bias[o];
      for (int i = 0; i < input_dim; ++i)
        sum += (double)dense_operand(dtype, x[(size_t)r * input_dim + i]) *
               (double)dense_operand(dtype, matrix[(size_t)i * output_dim + o]);
      const float value = (float)sum;
      y[(size_t)r * output_dim + o] =
          dtype == PLUTO_ORACLE_BF16 ? pluto_oracle_bf16_round(value) : value;
    }
  return 0;
}

int pluto_oracle_dense_backward(int dtype, int rows, int input_dim, int output_dim,
                                const float* x, const float* matrix, const float* dy,
                                float* dx, float* d_matrix, float* d_bias) {
  if ((dtype != PLUTO_ORACLE_BF16 && dtype != PLUTO_ORACLE_F32) || rows <= 0 || input_dim <= 0 ||
      output_dim <= 0 || !x || !matrix || !dy || !dx || !d_matrix || !d_bias)
    return 1;
  for (int r = 0; r < rows; ++r)
    for (int i = 0; i < input_dim; ++i) {
      double sum = 0.0;
      for (int o = 0; o < output_dim; ++o)
        sum += (double)dense_operand(dtype, dy[(size_t)r * output_dim + o]) *
               (double)dense_operand(dtype, matrix[(size_t)i * output_dim + o]);
      dx[(size_t)r * input_dim + i] = (float)sum;
    }
  for (int i = 0; i < input_dim; ++i)
    for (int o = 0; o < output_dim; ++o) {
      double sum = 0.0;
      for (int r = 0; r < rows; ++r)
        sum += (double)dense_operand(dtype, x[(size_t)r * input_dim + i]) *
               (double)dense_operand(dtype, dy[(size_t)r * output_dim + o]);
      d_matrix[(size_t)i * output_dim + o] = (float)sum;
    }
  for (int o = 0; o < output_dim; ++o) {
    double sum = 0.0;
    for (int r = 0; r < rows; ++r) sum += dy[(size_t)r * output_dim + o];
    d_bias[o] = (float)sum;
  }
  return 0;
}


/* ---- imported projection (fully_connected.cc:40-94,295-341) --------------- */

float pluto_oracle_fp8_e4m3_to_f32(uint8_t bits) {
  const int sign = bits >> 7, exponent = (bits >> 3) & 15, mantissa = bits & 7;
  float magnitude;
  if (exponent == 15 && mantissa == 7) return NAN;
  if (exponent == 0)
    magnitude = ldexpf((float)mantissa, -9); /* subnormal: m/8 * 2^-6 */
  else
    magnitude = ldexpf(1.0f + mantissa / 8.0f, exponent - 7);
  return sign ? -magnitude : magnitude;
}

uint8_t pluto_oracle_f32_to_fp8_e4m3(float value) {
  if (isnan(value)) return 0x7f;
  const uint8_t sign = signbit(value) ? 0x80 : 0;
  const double a = fabs((double)value);
  if (a >= 448.0) return sign | 0x7e; /* saturate (also infinities) */
  /* spacing of the format at a: 2^(e-3) with e = max(floor(log2 a), -6) */
  int e;
  frexp(a, &e); /* a = f * 2^e, f in [0.5, 1) -> floor(log2 a) = e - 1 */
  int exponent = a == 0.0 ? -6 : e - 1;
  if (exponent < -6) exponent = -6;
  const double step = ldexp(1.0, exponent - 3);
  /* nearbyint rounds halfway cases to even in the default rounding mode */
  double steps = nearbyint(a / step);
  double rounded = steps * step;
  if (rounded >= 448.0 + 1e-9) return sign | 0x7e;
  if (rounded == 0.0) return sign;
  frexp(rounded, &e);
  int re = e - 1;
  if (re < -6) { /* subnormal: rounded = m * 2^-9 */
    return sign | (uint8_t)(int)(rounded / ldexp(1.0, -9));
  }
  const int mantissa = (int)((rounded / ldexp(1.0, re) - 1.0) * 8.0 + 0.5);
  return sign | (uint8_t)(((re + 7) << 3) | mantissa);
}

void pluto_oracle_imported_quantize(const float* x, int n, float* out) {
  for (int g0 = 0; g0 < n; g0 += 128) {
    const int g1 = g0 + 128 < n ? g0 + 128 : n;
    float largest = 0.0f;
    for (int i = g0; i < g1; ++i) largest = fmaxf(largest, fabsf(x[i]));
    const float scale = largest / 448.0f;
    const float divisor = fmaxf(scale, 1e-12f);
    for (int i = g0; i < g1; ++i)
      out[i] = pluto_oracle_fp8_e4m3_to_f32(pluto_oracle_f32_to_fp8_e4m3(x[i] / divisor)) * scale;
  }
}

int pluto_oracle_imported_matvec(int storage, const void* weights, const float* scales,
                                 const float* x, int input_dim, int output_dim, float* y) {
  if (storage < PLUTO_ORACLE_MATRIX_BF16 || storage > PLUTO_ORACLE_MATRIX_FP8_E4M3 ||
      input_dim <= 0 || output_dim <= 0 || !weights || !x || !y)
    return -1;
  if ((storage == PLUTO_ORACLE_MATRIX_FP8_E4M3) != (scales != NULL)) return -1;
  float* token = (float*)malloc(sizeof(float) * (size_t)input_dim);
  if (!token) return -2;
  if (storage == PLUTO_ORACLE_MATRIX_FP8_E4M3)
    pluto_oracle_imported_quantize(x, input_dim, token);
  else
    memcpy(token, x, sizeof(float) * (size_t)input_dim);
  const int scale_cols = (input_dim + 127) / 128;
  for (int r = 0; r < output_dim; ++r) {
    double sum = 0.0;
    for (int c = 0; c < input_dim; ++c) {
      const size_t i = (size_t)r * input_dim + c;
      float w;
      if (storage == PLUTO_ORACLE_MATRIX_BF16)
        w = pluto_oracle_bf16_to_f32(((const uint16_t*)weights)[i]);
      else if (storage == PLUTO_ORACLE_MATRIX_F32)
        w = ((const float*)weights)[i];
      else
        w = pluto_oracle_fp8_e4m3_to_f32(((const uint8_t*)weights)[i]) *
            scales[(size_t)(r / 128) * scale_cols + c / 128];
      sum += (double)w * token[c];
    }
    y[r] = pluto_oracle_bf16_round((float)sum);
  }
  free(token);
  return 0;
}
