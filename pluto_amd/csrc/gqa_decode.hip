// Batched single-token GQA decode against a bf16 KV cache: one fused kernel,
// split-K over blocks of the sequence, tuned as an HBM streaming kernel.
//
// Semantics: CachedAttentionStep (src/llm/layers/util/cached_attention_ops.cc:
// 308-353: PrepareAttentionKernel :30-79, FullAttentionKernel :83-126) for
// every sequence of the batch.  One workgroup owns one (sequence, kv head,
// block of `split_tokens` cache rows) and serves ALL query heads of the group,
// so every K and V byte is read from HBM exactly once (the reference launches
// one program per query head and streams the cache once per head of the
// group).
//
//   prepare Every workgroup normalises and rotates the group's query heads
//           itself (a few hundred values; cheaper than a launch of its own)
//           while its first cache rows are already travelling.  The
//           workgroup that owns a sequence's last block also prepares the new
//           K row and the V row, appends them to the cache and keeps a copy
//           in LDS: it is the only one that needs them, and takes them from
//           there.
//   scores  S^T[token, head] = K[token, :] . q[head, :] with
//           v_mfma_f32_16x16x32_bf16: the A operand (16 tokens x 32 channels) is
//           loaded straight from global memory, 16 bytes per lane, the four
//           lanes of a token together one 64-byte sector per load;
//           the group's heads are the (zero padded) 16 columns.
//   values  O[head, :] += p[head, token] * V[token, :] on
//           v_mfma_f32_16x16x16_bf16: V rows stream through 16-row LDS stages
//           (buffer loads that write LDS directly), the probabilities enter as
//           the sum of two bf16 numbers (hi + lo), which keeps the product to
//           FP32 accuracy.  The kernel is bound by HBM, not by this arithmetic.
//   combine Partial (o, m, l) triples are written per block.  Workgroups count
//           their arrivals per (sequence, kv head); the one that arrives last
//           combines that pair's blocks in ascending order (a fixed order,
//           whichever workgroup does it: bitwise repeatable), applies
//           bf16(bf16(core) * bf16(sigmoid(gate))) and leaves the counter zero.
#include <type_traits>

#include "gqa.h"
#include "gqa_rotate.h"
#include "mfma_tile.h"

namespace pluto_hip {
namespace {

constexpr int kMaxSplit = 512;
constexpr int kThreads = 256;
constexpr int kCombineChunk = 128;  // blocks combined per pass over the LDS weights

__device__ inline bf16x8 load_bf16x8(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

__device__ inline int find_sequence(const DecodeBatch& batch, int block) {
  int lo = 0, hi = batch.count - 1;
  while (lo < hi) {  // last b with block_start[b] <= block
    const int mid = (lo + hi + 1) / 2;
    if (batch.block_start[mid] <= block) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// Partial results travel between workgroups on different XCDs, each with an L2
// of its own.  They are stored and loaded as device-scope relaxed atomics,
// which go through to the memory side, so no L2 has to be written back or
// invalidated wholesale (a device-scope fence does both, and costs more than
// the rest of the kernel when four thousand workgroups issue one each).
__device__ inline void store_shared(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline float load_shared(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Workgroup barrier that orders LDS traffic only: unlike __syncthreads() it
// does not wait for the wave's outstanding global loads.
__device__ inline void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// One wave prepares one head vector (RMSNorm with (1 + w), split-half partial
// RoPE, bf16 rounding points as in normalize_rotate) with a single round trip
// to memory: every lane loads its D/64 channels and weights at once, the RoPE
// partner comes from the LDS row the result is left in.  `row` receives the
// bf16 bits; `cosine`/`sine` hold this lane's rounded table entries per slot.
template <int D>
__device__ inline void prepare_head(const void* base, long long offset, int dtype,
                                    const float* weight, int rotary_dim, float epsilon,
                                    const float (&cosine)[D / 64], const float (&sine)[D / 64],
                                    uint16_t* row) {
  constexpr int SLOTS = D / 64;
  const int lane = threadIdx.x % 64;
  float x[SLOTS], w[SLOTS];
  if (dtype == PLUTO_HIP_BF16) {
    const uint16_t* in = static_cast<const uint16_t*>(base) + offset;
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) x[i] = bf16_bits_to_float(in[lane + 64 * i]);
  } else {
    const float* in = static_cast<const float*>(base) + offset;
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) x[i] = in[lane + 64 * i];
  }
#pragma unroll
  for (int i = 0; i < SLOTS; ++i) w[i] = weight[lane + 64 * i];
  double square = 0.0;
#pragma unroll
  for (int i = 0; i < SLOTS; ++i) square += static_cast<double>(x[i] * x[i]);
  square = wave_sum_f64(square);
  const double inverse = 1.0 / sqrt(square / D + static_cast<double>(epsilon));
  float normal[SLOTS];
#pragma unroll
  for (int i = 0; i < SLOTS; ++i) {
    normal[i] = round_to_bf16(
        static_cast<float>(x[i] * inverse * (1.0 + static_cast<double>(w[i]))));
    row[lane + 64 * i] = static_cast<uint16_t>(__float_as_uint(normal[i]) >> 16);
  }
  // the wave's normalised row is in LDS before partners are read from it
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_wave_barrier();
  const int half = rotary_dim / 2;
  float result[SLOTS];
#pragma unroll
  for (int i = 0; i < SLOTS; ++i) {
    const int c = lane + 64 * i;
    result[i] = normal[i];
    if (c < rotary_dim) {
      const float partner = bf16_bits_to_float(row[c < half ? c + half : c - half]);
      const float a = round_to_bf16(normal[i] * cosine[i]);
      const float b = round_to_bf16(partner * sine[i]);
      result[i] = round_to_bf16(c < half ? a - b : a + b);
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int i = 0; i < SLOTS; ++i)
    row[lane + 64 * i] = static_cast<uint16_t>(__float_as_uint(result[i]) >> 16);
}

// Compile-time loop: f(std::integral_constant<int, I>) for I = FIRST .. LAST-1.
template <int FIRST, int LAST, class F>
__device__ inline void static_for(F&& f) {
  if constexpr (FIRST < LAST) {
    f(std::integral_constant<int, FIRST>{});
    static_for<FIRST + 1, LAST>(f);
  }
}

// K rows requested without the compiler's knowledge of when they land: the
// wave's vector-memory queue then holds K rows and V stage fills in an order
// only this file knows, and wait_for_rows() says how many younger requests may
// still be outstanding when a group's rows are needed (requests complete in
// order).  Passing the registers through the wait ties every use to it.
template <int KSTEPS>
__device__ inline void request_rows(const uint16_t* row, bf16x8 (&dst)[KSTEPS]) {
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks)
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst[ks]) : "v"(row + 32 * ks) : "memory");
}
template <int OUTSTANDING, int KSTEPS>
__device__ inline void wait_for_rows(bf16x8 (&k)[KSTEPS]) {
  static_assert(OUTSTANDING >= 0 && OUTSTANDING < 64);
  static_assert(KSTEPS == 2 || KSTEPS == 4 || KSTEPS == 8);
  if constexpr (KSTEPS == 2)
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(k[0]), "+v"(k[1]) : "n"(OUTSTANDING) : "memory");
  else if constexpr (KSTEPS == 4)
    asm volatile("s_waitcnt vmcnt(%4)"
                 : "+v"(k[0]), "+v"(k[1]), "+v"(k[2]), "+v"(k[3])
                 : "n"(OUTSTANDING) : "memory");
  else
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(k[0]), "+v"(k[1]), "+v"(k[2]), "+v"(k[3]), "+v"(k[4]), "+v"(k[5]),
                   "+v"(k[6]), "+v"(k[7])
                 : "n"(OUTSTANDING) : "memory");
}

// What a workgroup knows about its (sequence, kv head, block).
struct BlockContext {
  int tid, wave, lane, hq, n;
  int g, seq, position, length, t0, per_wave;
  uint16_t* keys;    // this kv head's rows of the sequence's cache
  uint16_t* values;
  long long slot;    // where the block's partial results go
};

constexpr int kStageRows = 16;  // V rows per LDS stage of a wave: one contraction step
// Stages per wave (one in use, the others travelling) and K groups requested
// before they are used.  At head width 256 a group and a stage are 8 KiB a
// wave each; two of either let two workgroups share a compute unit (64 KiB
// of LDS and under 256 registers each), which covers one workgroup's start
// and hand-over with the other's stream.
constexpr int stages_of(int head_dim) { return head_dim == 256 ? 2 : 3; }
constexpr int ahead_of(int head_dim) { return head_dim == 256 ? 2 : 4; }

// Request order of a wave when the block size is a compile-time constant: K
// groups 0 .. ahead-1 up front; score step j then requests group j + ahead,
// and once the K rows run out the first V stages instead, one a step, so
// that requests stay in flight from the last score steps into the first value
// steps.  A group and a stage are the same number of requests per lane
// (D / 32); ahead >= stages, so every first stage finds a step.
struct RequestOrder {
  int groups, ahead, stages;
  constexpr int first_fill_step() const { return groups > ahead ? groups - ahead : 0; }
  constexpr bool step_requests_rows(int step) const { return step + ahead < groups; }
  constexpr bool step_requests_stage(int step) const {
    const int stage = step - first_fill_step();
    return !step_requests_rows(step) && stage >= 0 && stage < stages && stage < groups;
  }
  // Units (groups or stages) requested after K group `group` and before score
  // step `group` waits for it.
  constexpr int units_after_group(int group) const {
    const int up_front = groups < ahead ? groups : ahead;
    int after = group < up_front ? up_front - 1 - group : 0;
    for (int step = 0; step < group; ++step) {
      if (step_requests_rows(step)) after += step + ahead > group ? 1 : 0;
      else if (step_requests_stage(step)) after += 1;
    }
    return after;
  }
};

// The same order replayed as a queue, at compile time: every K group is
// requested exactly once and before its score step; when step `group` waits
// with units_after_group(group) units allowed outstanding, the group is no
// longer among them but the unit right after it still is (the wait is exact,
// not just safe); and when the value steps begin, the first
// min(stages, groups) V stages, in order, are all that has been requested after
// the last K group -- what the waits of the value steps count on.
constexpr bool request_order_holds(int groups, int ahead, int stages) {
  const RequestOrder order = {groups, ahead, stages};
  int queue[64] = {};  // unit i of the queue: K group g as g, V stage s as 100 + s
  int issued = 0;
  for (int g = 0; g < groups && g < ahead; ++g) queue[issued++] = g;
  for (int step = 0; step < groups; ++step) {
    int at = -1;
    for (int i = 0; i < issued; ++i)
      if (queue[i] == step) at = at < 0 ? i : 64;
    if (at < 0 || at >= 64) return false;  // not requested yet, or twice
    if (issued - 1 - at != order.units_after_group(step)) return false;
    if (order.step_requests_rows(step)) queue[issued++] = step + ahead;
    else if (order.step_requests_stage(step)) queue[issued++] = 100 + step - order.first_fill_step();
    if (issued > 60) return false;
  }
  const int first_stages = stages < groups ? stages : groups;
  if (issued != groups + first_stages) return false;
  for (int s = 0; s < first_stages; ++s)
    if (queue[groups + s] != 100 + s) return false;  // stages follow every K group, in order
  return true;
}
constexpr bool request_orders_hold() {
  for (int groups = 1; groups <= 16; ++groups)
    if (!request_order_holds(groups, 4, 3) || !request_order_holds(groups, 2, 2)) return false;
  return true;
}
static_assert(request_orders_hold(), "the hand-counted waits of the score steps");

// LDS of a workgroup: per wave kStages stages of 16 V rows (later reused for
// the waves' partial outputs and the combine's block weights).
template <int D>
constexpr int value_area_bytes() { return 4 * stages_of(D) * kStageRows * D * 2; }

// Prepare step, split-K attention over one block and the block's partial
// results.  SPLIT: tokens per block when known at compile time (the loops
// then have no branches the load scheduling would have to stop at), 0
// otherwise.  LAST: the block holds the row this call appends; only then can
// rows lie beyond the sequence, and only then is the new row needed (it is
// taken from LDS, whatever the cache holds yet).
//
// Each wave owns a quarter of the block's tokens from the prepare step to the
// end of phase 2 and waits for no other wave in between.
//   phase 1  S^T[token, head] = K q^T for groups of 16 tokens, K rows straight
//            from global memory into A operands.
//   phase 2  O^T[channel, head] += V^T P^T for stages of 16 tokens
//            (v_mfma_f32_16x16x16_bf16, one contraction step a stage).  V rows
//            travel global -> LDS without registers (kStages stages a wave,
//            the later ones requested while this one is used) and are gathered
//            into A operands by the LDS transpose read; P^T is the group's
//            score accumulator (lane group q holds tokens 4q .. 4q+3, the
//            contraction slots of both operands), so it needs no exchange.
//            Probabilities enter as bf16 hi + lo parts (two products), which
//            keeps the FP32 arithmetic of the reference to about 2^-17.
template <int D, int GROUP, int SPLIT, bool LAST>
__device__ inline void decode_block(const DecodeArgs& a, const BlockContext& ctx,
                                    unsigned char* value_area, float (*wave_max)[16],
                                    float (*wave_sum_lds)[16], uint16_t (*q_lds)[D],
                                    uint16_t (*new_row)[D]) {
  constexpr int KSTEPS = D / 32;
  constexpr int KCH = D / 8;                       // 16-byte chunks per row
  constexpr int GROUPS = (SPLIT ? SPLIT : kMaxSplit) / 64;  // 16-token groups per wave at most
  constexpr int FILLS = kStageRows * KCH / 64;     // 16-byte fills per lane and stage
  constexpr int kStages = stages_of(D), kAhead = ahead_of(D);
  constexpr RequestOrder kOrder = {GROUPS, kAhead, kStages};
  static_assert(kAhead >= kStages);
  constexpr int kStageBytes = kStageRows * D * 2;
  constexpr int CB = D / 16;                       // 16-channel blocks of O^T
  float (*o_lds)[GROUP][D] = reinterpret_cast<float (*)[GROUP][D]>(value_area);
  const int tid = ctx.tid, wave = ctx.wave, lane = ctx.lane, hq = ctx.hq, n = ctx.n;
  const int g = ctx.g, seq = ctx.seq, position = ctx.position, length = ctx.length;
  const int t0 = ctx.t0;
  const int per_wave = SPLIT ? SPLIT / 4 : ctx.per_wave;
  const int kh = a.key_value_heads;
  const uint16_t* keys = ctx.keys;
  const float scale2 = a.scale * kLog2e;
  const int groups = per_wave / 16;  // 16-token groups of this wave (<= GROUPS)
  const int wave_t0 = t0 + wave * per_wave;

  // ---- V stages: requested before anything else when the block size is only
  // known at run time, between the last score steps otherwise ---------------
  unsigned char* stage_base = value_area + wave * kStages * kStageBytes;
  uint32_t fill_offset[FILLS];
#pragma unroll
  for (int i = 0; i < FILLS; ++i) fill_offset[i] = tile_fill_offset<D>(i * 64 + lane, a.token_stride);
  auto fill = [&](int st) {
    // rows beyond the sequence (LAST only) or beyond this call's reach read as
    // zero: the descriptor ends with the last valid row
    const int row0 = wave_t0 + kStageRows * st;
    long long rows = kStageRows;
    if constexpr (SPLIT == 0)  // a wave's quarter may end inside a stage
      rows = min(rows, static_cast<long long>(per_wave) - kStageRows * st);
    if constexpr (LAST) rows = min(rows, static_cast<long long>(length) - row0);
    const uint32_t bytes =
        rows <= 0 ? 0u : static_cast<uint32_t>(((rows - 1) * a.token_stride + D) * 2);
    const int32x4 rsrc = make_rsrc(ctx.values + static_cast<long long>(row0) * a.token_stride, bytes);
#pragma unroll
    for (int i = 0; i < FILLS; ++i)
      lds_fill<16>(rsrc, stage_base + (st % kStages) * kStageBytes + i * 1024, fill_offset[i]);
  };
  if constexpr (SPLIT == 0) {
#pragma unroll
    for (int st = 0; st < kStages; ++st)
      if (st < groups) fill(st);
  }

  // ---- then the first K rows ------------------------------------------------
  // A operand row = lane % 16; rows beyond the valid prefix repeat its last row
  auto k_token = [&](int grp) {
    const int t = wave_t0 + 16 * grp + n;
    return LAST ? min(t, length - 1) : t;
  };
  auto load_k = [&](int grp, bf16x8 (&dst)[KSTEPS]) {
    // contraction step ks covers channels 32 ks .. 32 ks + 31: the four lanes
    // of a token read one 64-byte sector per load
    const uint16_t* row = keys + static_cast<long long>(k_token(grp)) * a.token_stride + 8 * hq;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) dst[ks] = load_bf16x8(row + 32 * ks);
  };
  auto request_k = [&](int grp, bf16x8 (&dst)[KSTEPS]) {
    request_rows<KSTEPS>(keys + static_cast<long long>(k_token(grp)) * a.token_stride + 8 * hq,
                         dst);
  };
  bf16x8 k_rows[kAhead][KSTEPS];
#pragma unroll
  for (int grp = 0; grp < kAhead; ++grp) {
    if constexpr (SPLIT == 0) {
      if (grp < groups) load_k(grp, k_rows[grp]);
    } else {
      if (grp < GROUPS) request_k(grp, k_rows[grp]);
    }
  }

  // ---- prepare: the group's queries, and the new cache row ----------------
  {
    // this lane's rotation table entries: channel c = lane + 64 i uses
    // frequency c mod (rotary / 2)
    const int half = a.rotary_dim / 2;
    float cosine[D / 64], sine[D / 64];
#pragma unroll
    for (int i = 0; i < D / 64; ++i) {
      const int c = lane + 64 * i;
      cosine[i] = 1.0f;
      sine[i] = 0.0f;
      if (c < a.rotary_dim && (wave < GROUP || LAST)) {
        const double angle =
            static_cast<double>(position) * a.inverse_frequency[c < half ? c : c - half];
        cosine[i] = round_to_bf16(static_cast<float>(cos(angle)));
        sine[i] = round_to_bf16(static_cast<float>(sin(angle)));
      }
    }
    for (int hh = wave; hh < GROUP; hh += 4)
      prepare_head<D>(a.q_gate,
                      (static_cast<long long>(seq) * a.query_heads + g * GROUP + hh) * 2 * D,
                      a.io_dtype, a.q_norm, a.rotary_dim, a.epsilon, cosine, sine, q_lds[hh]);
    if constexpr (LAST) {
      // cached_attention_ops.cc:64-77: the rotated key and the rounded value
      // become row `position` of the cache
      const long long in = (static_cast<long long>(seq) * kh + g) * D;
      const long long at = static_cast<long long>(position) * a.token_stride;
      if (wave == 3) {
        prepare_head<D>(a.k, in, a.io_dtype, a.k_norm, a.rotary_dim, a.epsilon, cosine, sine,
                        new_row[0]);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        for (int c = lane; c < D; c += 64) ctx.keys[at + c] = new_row[0][c];
      } else if (wave == 2) {
        for (int c = lane; c < D; c += 64) {
          const uint16_t bits = float_to_bf16_bits(load_element(a.v, in + c, a.io_dtype));
          new_row[1][c] = bits;
          ctx.values[at + c] = bits;
        }
      }
    }
    lds_barrier();
  }

  // ---- phase 1: scores -------------------------------------------------
  bf16x8 qf[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) {
    uint4 bits = make_uint4(0, 0, 0, 0);
    if (n < GROUP) bits = *reinterpret_cast<const uint4*>(&q_lds[n][32 * ks + 8 * hq]);
    qf[ks] = __builtin_bit_cast(bf16x8, bits);
  }
  bf16x8 k_new[KSTEPS];  // the appended row, as this lane would load it
  if constexpr (LAST) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) k_new[ks] = load_bf16x8(&new_row[0][32 * ks + 8 * hq]);
  }
  floatx4 s[GROUPS];
  float local_max = kMasked;
  auto score_group = [&](int grp, const bf16x8 (&rows)[KSTEPS]) {
    floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      bf16x8 k_use = rows[ks];
      if constexpr (LAST) k_use = k_token(grp) == position ? k_new[ks] : k_use;
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_use, qf[ks], acc, 0, 0, 0);
    }
    return acc;
  };
  // accumulator register r = (token 4*hq + r of the group, head n)
  auto scaled = [&](int grp, floatx4 acc) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int t = wave_t0 + 16 * grp + 4 * hq + r;
      const float v = (!LAST || t < length) ? acc[r] * scale2 : kMasked;
      acc[r] = v;
      local_max = fmaxf(local_max, v);
    }
    return acc;
  };
  if constexpr (SPLIT == 0) {
#pragma unroll
    for (int grp = 0; grp < GROUPS; ++grp) {
      s[grp] = floatx4{kMasked, kMasked, kMasked, kMasked};
      if (grp < groups) {
        const floatx4 acc = score_group(grp, k_rows[grp % kAhead]);
        // this group's registers take the rows of the group kAhead further on
        if (grp + kAhead < groups) load_k(grp + kAhead, k_rows[grp % kAhead]);
        s[grp] = scaled(grp, acc);
      }
    }
  } else {
    static_for<0, GROUPS>([&](auto index) {
      constexpr int grp = decltype(index)::value;
      wait_for_rows<kOrder.units_after_group(grp) * KSTEPS>(k_rows[grp % kAhead]);
      const floatx4 acc = score_group(grp, k_rows[grp % kAhead]);
      // this group's registers take the rows of the group kAhead further on;
      // when the rows have run out, a V stage is requested in their place
      if constexpr (kOrder.step_requests_rows(grp))
        request_k(grp + kAhead, k_rows[grp % kAhead]);
      else if constexpr (kOrder.step_requests_stage(grp))
        fill(grp - kOrder.first_fill_step());
      s[grp] = scaled(grp, acc);
    });
  }
  // Each wave normalises its quarter of the block by its own maximum.
  local_max = fmaxf(local_max, __shfl_xor(local_max, 16, 64));
  local_max = fmaxf(local_max, __shfl_xor(local_max, 32, 64));
  if (hq == 0) wave_max[wave][n] = local_max;

  // ---- phase 2: O^T += V^T P^T -------------------------------------------
  floatx4 o_acc[CB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) o_acc[cb] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
  float local_sum = 0.0f;
  // transpose read of this lane: as a source it supplies row 4 hq + kk of the
  // stage, channels 4b .. 4b+3 of a 16-channel block; it receives rows
  // 4 hq .. 4 hq + 3 of channel 16 cb + lane % 16
  const int kk = (lane % 16) / 4, bsel = lane % 4;
  int read_offset[CB];
  {
    const int row = 4 * hq + kk;
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
      read_offset[cb] =
          (row * KCH + ((2 * cb + bsel / 2) ^ tile_swizzle(row))) * 16 + (bsel % 2) * 8;
  }
#pragma unroll
  for (int st = 0; st < GROUPS; ++st) {
    if (st < groups) {
      unsigned char* stage = stage_base + (st % kStages) * kStageBytes;
      // this stage's rows have landed (those of the later stages may still
      // travel: kStages - 1 of them unless the block ends first)
      const int younger = min(kStages - 1, groups - 1 - st);
      if (younger >= 2)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * FILLS) : "memory");
      else if (younger == 1)
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(FILLS) : "memory");
      else
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if constexpr (LAST) {
        const int local = position - (wave_t0 + kStageRows * st);
        if (local >= 0 && local < kStageRows) {
          // the appended V row: from LDS to its place in the stage
          if (lane < KCH)
            *reinterpret_cast<uint4*>(stage + (local * KCH + (lane ^ tile_swizzle(local))) * 16) =
                *reinterpret_cast<const uint4*>(&new_row[1][8 * lane]);
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        }
      }
      __builtin_amdgcn_wave_barrier();
      // P^T of the stage's group as hi + lo bf16 B operands
      float p[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float score = s[st][e];
        // (a wave whose tokens all lie beyond the sequence has local_max ==
        // kMasked: its probabilities are zero, not 2^0)
        p[e] = (LAST && score == kMasked) ? 0.0f : __builtin_amdgcn_exp2f(score - local_max);
        local_sum += p[e];
      }
      uint32_t hi[2], lo[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        hi[e] = pack_bf16(p[2 * e], p[2 * e + 1]);
        lo[e] = pack_bf16(p[2 * e] - __uint_as_float(hi[e] << 16),
                          p[2 * e + 1] - __uint_as_float(hi[e] & 0xffff0000u));
      }
      const shortx4 p_hi = __builtin_bit_cast(shortx4, make_uint2(hi[0], hi[1]));
      const shortx4 p_lo = __builtin_bit_cast(shortx4, make_uint2(lo[0], lo[1]));
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        const shortx4 v_t =
            __builtin_bit_cast(shortx4, lds_transpose_read(stage, read_offset[cb]));
        o_acc[cb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v_t, p_hi, o_acc[cb], 0, 0, 0);
        o_acc[cb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(v_t, p_lo, o_acc[cb], 0, 0, 0);
      }
      // the stage kStages further on takes this stage's place
      if (st + kStages < groups) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        fill(st + kStages);
      }
    }
  }
  local_sum += __shfl_xor(local_sum, 16, 64);
  local_sum += __shfl_xor(local_sum, 32, 64);
  if (hq == 0) wave_sum_lds[wave][n] = local_sum;
  __syncthreads();  // every wave is done with its V stages
  // o_acc[cb][r] = O^T[channel 16 cb + 4 hq + r][head n]
  if (n < GROUP) {
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
      *reinterpret_cast<float4*>(&o_lds[wave][n][16 * cb + 4 * hq]) =
          make_float4(o_acc[cb][0], o_acc[cb][1], o_acc[cb][2], o_acc[cb][3]);
  }
  __syncthreads();
  // the four waves' results, each relative to its own maximum, become the
  // block's: o = sum_w o_w 2^(m_w - m), l likewise, m = max_w m_w
  const long long slot = ctx.slot;
  for (int i = tid; i < GROUP * D; i += kThreads) {
    const int hh = i / D, c = i % D;
    const float m = fmaxf(fmaxf(wave_max[0][hh], wave_max[1][hh]),
                          fmaxf(wave_max[2][hh], wave_max[3][hh]));
    float w[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) w[q] = __builtin_amdgcn_exp2f(wave_max[q][hh] - m);
    store_shared(&a.part_o[(slot * GROUP + hh) * D + c],
                 (o_lds[0][hh][c] * w[0] + o_lds[1][hh][c] * w[1]) +
                     (o_lds[2][hh][c] * w[2] + o_lds[3][hh][c] * w[3]));
  }
  if (tid < GROUP) {
    const float m = fmaxf(fmaxf(wave_max[0][tid], wave_max[1][tid]),
                          fmaxf(wave_max[2][tid], wave_max[3][tid]));
    float w[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) w[q] = __builtin_amdgcn_exp2f(wave_max[q][tid] - m);
    store_shared(&a.part_m[slot * GROUP + tid], m);
    store_shared(&a.part_l[slot * GROUP + tid],
                 (wave_sum_lds[0][tid] * w[0] + wave_sum_lds[1][tid] * w[1]) +
                     (wave_sum_lds[2][tid] * w[2] + wave_sum_lds[3][tid] * w[3]));
  }
}

template <int D, int GROUP>
__global__ void __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(D == 256 ? 2 : 3, D == 256 ? 2 : 3)))
decode_fused_kernel(DecodeArgs a, DecodeBatch batch) {
  __shared__ __attribute__((aligned(1024))) unsigned char value_area[value_area_bytes<D>()];
  float* shared_area = reinterpret_cast<float*>(value_area);
  __shared__ float wave_max[4][16];
  __shared__ float wave_sum_lds[4][16];
  __shared__ __attribute__((aligned(16))) uint16_t q_lds[GROUP][D];  // prepared queries
  __shared__ __attribute__((aligned(16))) uint16_t new_row[2][D];    // appended K and V rows
  __shared__ int final_flag;

  const int tid = threadIdx.x;
  const int kh = a.key_value_heads;
  const int g = blockIdx.x % kh;
  const int block = blockIdx.x / kh;
  const int b = find_sequence(batch, block);
  const int seq = batch.sequence[b];
  const int blocks_here = batch.block_start[b + 1] - batch.block_start[b];
  const int j = block - batch.block_start[b];
  BlockContext ctx;
  ctx.tid = tid;
  ctx.wave = tid / 64;
  ctx.lane = tid % 64;
  ctx.hq = ctx.lane / 16;
  ctx.n = ctx.lane % 16;
  ctx.g = g;
  ctx.seq = seq;
  ctx.position = batch.positions[b];
  ctx.length = ctx.position + 1;
  ctx.t0 = j * a.split_tokens;
  ctx.per_wave = a.split_tokens / 4;
  ctx.keys = static_cast<uint16_t*>(batch.keys[b]) + g * a.head_stride;
  ctx.values = static_cast<uint16_t*>(batch.values[b]) + g * a.head_stride;
  ctx.slot = (a.block_base + block) * kh + g;
  const bool is_last = j == blocks_here - 1;  // this block holds row `position`
  constexpr int kFixed = decode_split_default(D);
  if (a.split_tokens == kFixed) {
    if (is_last)
      decode_block<D, GROUP, kFixed, true>(a, ctx, value_area, wave_max, wave_sum_lds, q_lds, new_row);
    else
      decode_block<D, GROUP, kFixed, false>(a, ctx, value_area, wave_max, wave_sum_lds, q_lds, new_row);
  } else {
    if (is_last)
      decode_block<D, GROUP, 0, true>(a, ctx, value_area, wave_max, wave_sum_lds, q_lds, new_row);
    else
      decode_block<D, GROUP, 0, false>(a, ctx, value_area, wave_max, wave_sum_lds, q_lds, new_row);
  }

  // ---- who combines: the workgroup of this (sequence, kv head) that arrives last
  if (blocks_here > 1) {
    // every store of this wave has been acknowledged by the memory side ...
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // ... and so has the whole workgroup's, before it is counted
    if (tid == 0) {
      unsigned* counter = a.arrivals + static_cast<long long>(seq) * kh + g;
      const unsigned before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT);
      const bool final_one = before == static_cast<unsigned>(blocks_here - 1);
      // nobody else touches the counter any more: leave it zero for the next call
      if (final_one) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      final_flag = final_one ? 1 : 0;
    }
    __syncthreads();
    if (!final_flag) return;
    // the partial results are read below with device-scope loads, which do
    // not take stale lines from this XCD's L2
  } else {
    __syncthreads();  // own partial results, read back below
  }

  // ---- combine: blocks in ascending order, kCombineChunk at a time --------
  // LDS: m, l and then the weights of the chunk's blocks per head; running
  // maximum, normalizer and rescale factor per head.
  float* chunk_m = shared_area;                           // [kCombineChunk][GROUP]
  float* chunk_l = shared_area + kCombineChunk * GROUP;   // [kCombineChunk][GROUP]
  float* head_state = shared_area + 2 * kCombineChunk * GROUP;  // [3][GROUP]
  static_assert((2 * kCombineChunk * GROUP + 3 * GROUP) * 4 <= value_area_bytes<D>());
  static_assert(4 * GROUP * D * 4 <= value_area_bytes<D>());
  constexpr int kOutputs = (GROUP * D + kThreads - 1) / kThreads;  // per thread
  const long long first_slot = (a.block_base + batch.block_start[b]) * kh + g;
  const long long slot_step = kh;  // consecutive blocks of one kv head
  float o[kOutputs];
#pragma unroll
  for (int u = 0; u < kOutputs; ++u) o[u] = 0.0f;
  if (tid < GROUP) {
    head_state[0 * GROUP + tid] = kMasked;  // running maximum
    head_state[1 * GROUP + tid] = 0.0f;     // running normalizer
  }
  for (int j0 = 0; j0 < blocks_here; j0 += kCombineChunk) {
    const int count = min(kCombineChunk, blocks_here - j0);
    __syncthreads();  // the previous chunk's weights are no longer read
    for (int i = tid; i < count * GROUP; i += kThreads) {
      const long long at = (first_slot + (j0 + i / GROUP) * slot_step) * GROUP + i % GROUP;
      chunk_m[i] = load_shared(&a.part_m[at]);
      chunk_l[i] = load_shared(&a.part_l[at]);
    }
    __syncthreads();
    if (tid < GROUP) {
      const float old_max = head_state[0 * GROUP + tid];
      float maximum = old_max;
      for (int jj = 0; jj < count; ++jj) maximum = fmaxf(maximum, chunk_m[jj * GROUP + tid]);
      const float rescale = __builtin_amdgcn_exp2f(old_max - maximum);
      float normalizer = head_state[1 * GROUP + tid] * rescale;
      for (int jj = 0; jj < count; ++jj) {
        const float w = __builtin_amdgcn_exp2f(chunk_m[jj * GROUP + tid] - maximum);
        normalizer += chunk_l[jj * GROUP + tid] * w;
        chunk_m[jj * GROUP + tid] = w;  // from here on: the block's weight
      }
      head_state[0 * GROUP + tid] = maximum;
      head_state[1 * GROUP + tid] = normalizer;
      head_state[2 * GROUP + tid] = rescale;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kOutputs; ++u) {
      const int i = tid + u * kThreads;
      if (i < GROUP * D) o[u] *= head_state[2 * GROUP + i / D];
    }
    // eight blocks per step: their loads are issued before their use
    for (int jj = 0; jj < count; jj += 8) {
      float part[8][kOutputs];
#pragma unroll
      for (int step = 0; step < 8; ++step) {
        const int block_j = min(jj + step, count - 1);
        const float* base = a.part_o + (first_slot + (j0 + block_j) * slot_step) * GROUP * D;
#pragma unroll
        for (int u = 0; u < kOutputs; ++u) {
          const int i = tid + u * kThreads;
          part[step][u] = i < GROUP * D ? load_shared(&base[i]) : 0.0f;
        }
      }
#pragma unroll
      for (int step = 0; step < 8; ++step) {
        if (jj + step < count) {
#pragma unroll
          for (int u = 0; u < kOutputs; ++u) {
            const int i = tid + u * kThreads;
            if (i < GROUP * D) o[u] += part[step][u] * chunk_m[(jj + step) * GROUP + i / D];
          }
        }
      }
    }
  }
  // gate: cached_attention_ops.cc:119-125
#pragma unroll
  for (int u = 0; u < kOutputs; ++u) {
    const int i = tid + u * kThreads;
    if (i >= GROUP * D) continue;
    const int hh = i / D, c = i % D;
    const float core = o[u] / head_state[1 * GROUP + hh];
    const long long at = static_cast<long long>(seq) * a.query_heads + g * GROUP + hh;
    const float logit = load_element(a.q_gate, (at * 2 + 1) * D + c, a.io_dtype);
    const float sigmoid = gate_sigmoid(logit);
    store_element(a.out, at * D + c, a.io_dtype,
                  round_to_bf16(round_to_bf16(core) * round_to_bf16(sigmoid)));
  }
}

__global__ void __launch_bounds__(256) decode_clear_kernel(unsigned* arrivals, int count) {
  for (int i = blockIdx.x * 256 + threadIdx.x; i < count; i += gridDim.x * 256) arrivals[i] = 0u;
}

// Two-pass probability rows for inspection: one workgroup per (query head,
// query row).  Row r sees the first `first_visible + r` cache rows and is
// stored at probabilities[(head * rows + r) * row_width ..], zero beyond the
// visible prefix.
__global__ void __launch_bounds__(256)
attention_probabilities_kernel(const void* q, int q_dtype, CacheView cache, int query_heads,
                               int key_value_heads, int head_dim, int rows, int first_visible,
                               int row_width, float scale, float* probabilities) {
  __shared__ float query[256];
  __shared__ float reduce[4];
  const int head = blockIdx.x;
  const int r = blockIdx.y;
  const int length = first_visible + r;
  const int kv = head / (query_heads / key_value_heads);
  float* row = probabilities + (static_cast<long long>(head) * rows + r) * row_width;
  for (int c = threadIdx.x; c < head_dim; c += 256)
    query[c] = load_element(
        q, (static_cast<long long>(r) * query_heads + head) * head_dim + c, q_dtype);
  __syncthreads();
  float maximum = kMasked;
  for (int t = threadIdx.x; t < length; t += 256) {
    const long long base = t * cache.token_stride + kv * cache.head_stride;
    float score = 0.0f;
    for (int c = 0; c < head_dim; ++c)
      score += load_element(cache.keys, base + c, cache.dtype) * query[c];
    score *= scale;
    row[t] = score;
    maximum = fmaxf(maximum, score);
  }
  maximum = wave_max(maximum);
  if (threadIdx.x % 64 == 0) reduce[threadIdx.x / 64] = maximum;
  __syncthreads();
  maximum = fmaxf(fmaxf(reduce[0], reduce[1]), fmaxf(reduce[2], reduce[3]));
  __syncthreads();
  float sum = 0.0f;
  for (int t = threadIdx.x; t < length; t += 256) {
    const float p = expf(row[t] - maximum);
    row[t] = p;
    sum += p;
  }
  sum = wave_sum(sum);
  if (threadIdx.x % 64 == 0) reduce[threadIdx.x / 64] = sum;
  __syncthreads();
  sum = (reduce[0] + reduce[1]) + (reduce[2] + reduce[3]);
  for (int t = threadIdx.x; t < length; t += 256) row[t] = row[t] / sum;
  for (int t = length + threadIdx.x; t < row_width; t += 256) row[t] = 0.0f;
}

template <int D>
int launch_for_group(hipStream_t stream, const DecodeArgs& a, const DecodeBatch& batch,
                     int group, unsigned blocks) {
  switch (group) {
    case 1: decode_fused_kernel<D, 1><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    case 2: decode_fused_kernel<D, 2><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    case 4: decode_fused_kernel<D, 4><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    case 6: decode_fused_kernel<D, 6><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    case 8: decode_fused_kernel<D, 8><<<blocks, kThreads, 0, stream>>>(a, batch); break;
    default: return PLUTO_HIP_EUNSUPPORTED;
  }
  return launch_status();
}

}  // namespace

bool decode_fast_supported(int head_dim, int group) {
  const bool dim_ok = head_dim == 64 || head_dim == 128 || head_dim == 256;
  const bool group_ok = group == 1 || group == 2 || group == 4 || group == 6 || group == 8;
  return dim_ok && group_ok;
}

int launch_decode_fast(hipStream_t stream, const DecodeArgs& a, const DecodeBatch& batch) {
  const int group = a.query_heads / a.key_value_heads;
  const long long blocks =
      static_cast<long long>(batch.block_start[batch.count]) * a.key_value_heads;
  if (blocks <= 0 || blocks > 0x7fffffffLL) return PLUTO_HIP_EINVAL;
  if (!decode_split_valid(a.head_dim, a.split_tokens)) return PLUTO_HIP_EINVAL;
  if (a.rotary_dim / 2 > 128) return PLUTO_HIP_EUNSUPPORTED;
  if (!kernel_enabled(kMainKernel)) return 0;
  switch (a.head_dim) {
    case 64: return launch_for_group<64>(stream, a, batch, group, static_cast<unsigned>(blocks));
    case 128: return launch_for_group<128>(stream, a, batch, group, static_cast<unsigned>(blocks));
    case 256: return launch_for_group<256>(stream, a, batch, group, static_cast<unsigned>(blocks));
    default: return PLUTO_HIP_EUNSUPPORTED;
  }
}

int launch_decode_clear(hipStream_t stream, unsigned* arrivals, int count, bool always) {
  if (!always && !kernel_enabled(kAuxiliaryKernel)) return 0;
  decode_clear_kernel<<<(count + 255) / 256, 256, 0, stream>>>(arrivals, count);
  return launch_status();
}

int launch_attention_probabilities(hipStream_t stream, const void* q, int q_dtype,
                                   const CacheView& cache, int query_heads,
                                   int key_value_heads, int head_dim, int rows,
                                   int first_visible, int row_width, float scale,
                                   float* probabilities) {
  if (rows <= 0 || rows > 65535 || first_visible <= 0 ||
      static_cast<long long>(first_visible) + rows - 1 > row_width)
    return PLUTO_HIP_EINVAL;
  attention_probabilities_kernel<<<dim3(query_heads, rows), 256, 0, stream>>>(
      q, q_dtype, cache, query_heads, key_value_heads, head_dim, rows, first_visible, row_width,
      scale, probabilities);
  return launch_status();
}

}  // namespace pluto_hip
