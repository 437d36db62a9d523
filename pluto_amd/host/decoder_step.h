// One decoding step for several sequences at once: the counterpart of
// Model::Step (src/llm/qwen/model.cc:405-428), lifted from one sequence to
// `batch` sequences that each own their caches and recurrent states.
//
// The reference's step uploads a token, runs the decoder graph (embedding
// lookup, then per layer Residual(norm -> attention branch) and
// Residual(feed-forward), model.cc:281-312) and keeps the hidden row for the
// head.  Here the decoder is a list of layers the caller composes: the batched
// attention branches of decoder_branch.h and, around them, whatever norm,
// residual and feed-forward layers the caller has (they are other layers of the
// reference and are not part of this library).  Every layer maps bf16 rows
// [batch, 1, width] to rows of the same type.  What this class owns is the
// step's contract:
//   * nothing runs when a sequence has no room left or the input does not fit
//     (InvalidArgument, as model.cc:410-412), or after a step that failed
//     (FailedPrecondition until Reset, model.cc:407-409);
//   * the object is poisoned from the first launch to the last: a layer or hook
//     that fails after some caches advanced never leaves a half-advanced history
//     in use (model.cc:413-415,425-426);
//   * positions advance per sequence, and a sequence that ended is reset alone
//     and starts again at position 0 while the others go on.
#pragma once

#include <memory>
#include <optional>
#include <vector>

#include "pluto_amd/host/decoder_branch.h"
#include "pluto_amd/host/layer.h"

namespace pluto::llm {

class BatchedDecoderStep final {
 public:
  BatchedDecoderStep(const BatchedDecoderStep&) = delete;
  BatchedDecoderStep& operator=(const BatchedDecoderStep&) = delete;

  // `layers` run in order.  `attention` and `delta_net` name the branches
  // inside them (not owned; they must live as long as the layers do: the
  // reference keeps the same kind of handles, model.cc:318-331) whose caches
  // and states Reset restores.  `capacity` tokens fit a sequence: at most the
  // capacity of every attention branch's caches.
  static StatusOr<std::unique_ptr<BatchedDecoderStep>> Create(
      hip::Executor& executor, int batch, int width, int capacity,
      std::vector<std::unique_ptr<Layer>> layers,
      std::vector<BatchedFullAttentionBranch*> attention,
      std::vector<BatchedDeltaNetBranch*> delta_net);

  int batch() const { return static_cast<int>(positions_.size()); }
  int capacity() const { return capacity_; }
  // Tokens sequence s has consumed since it was last reset.
  int position(int sequence) const { return positions_[sequence]; }
  bool poisoned() const { return poisoned_; }

  // hidden: bf16 [batch, width], one row per sequence (the embedded token, or
  // whatever the caller's first layer expects).
  Status Step(const Buffer& hidden, LayerHooks* hooks = nullptr);
  // The rows the last layer left; FailedPrecondition unless the last Step
  // succeeded (Model::Logits, model.cc:430-435).
  StatusOr<Buffer> Hidden() const;

  // Every sequence back to position 0; clears the poison (Model::Reset).
  Status Reset();
  // One sequence back to position 0, the others untouched.  Not after a failed
  // step: only a full Reset restores a history that may be half advanced.
  Status Reset(int sequence);

 private:
  BatchedDecoderStep(hip::Executor& executor, int width, int capacity)
      : executor_(executor), width_(width), capacity_(capacity) {}

  hip::Executor& executor_;
  int width_, capacity_;
  bool poisoned_ = false;
  std::vector<int> positions_;
  std::vector<std::unique_ptr<Layer>> layers_;
  std::vector<BatchedFullAttentionBranch*> attention_;
  std::vector<BatchedDeltaNetBranch*> delta_net_;
  std::optional<Buffer> hidden_;
};

}  // namespace pluto::llm
