// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::compute::Embedding, the reference's op interface (include/compute/embedding.h:24-79).
//
// init draws the table from N(0, 1) ([num_embeddings, embedding_dim]), turns a negative
// padding_idx into its row number and rejects max_norm, as the reference does.  forward
// gathers rows for int32 or int64 indices of any shape (the result has the indices' shape
// plus the embedding dimension) and keeps the indices.  backward runs on the assist stream
// and leaves the dense gradient in state->forward.grad_weight: rows that were never indexed
// are zero, the padding row gets nothing, and the sum over the tokens of a row is taken in a
// fixed order (sort and segment, no floating point atomics), so two runs give the same bits.
// A defined grad_weight is accumulated into, an undefined one assigned.
#pragma once
#include "arg.h"
#include "module/state.h"
#include "tensor.h"
#include "threading/scheduler.h"

namespace cs::compute {
struct CS_API Embedding {
  struct State : virtual module::State {
    struct Forward {
      Tensor weight;         // [num_embeddings, embedding_dim]
      Tensor grad_weight{};  // same shape; undefined until the first backward
    } forward;
    struct Backward {
      ReadOnlyTensor indices;  // saved by forward, released by backward
    } backward;
    struct Args {
      int64_t num_weights;
      int64_t padding_idx;  // -1: none
      c10::optional<double> max_norm;
      double norm_type;
      bool scale_grad_by_freq;
      bool sparse;
    } args;

    State(const Forward &forward, const Backward &backward, const Args &args);
    [[nodiscard]] OrderedDict<std::string, Tensor> parameters() const override;  // "weight"
    [[nodiscard]] OrderedDict<std::string, Tensor> gradients() const override;
    [[nodiscard]] OrderedDict<std::string, Increment> increments() const override;
    void zero_grad() override;
  };

  struct Options {
    Options(const int64_t num_embeddings, const int64_t embedding_dim)
        : num_embeddings_{num_embeddings}, embedding_dim_{embedding_dim} {}
    CS_ARG(int64_t, num_embeddings);
    CS_ARG(int64_t, embedding_dim);
    CS_ARG(c10::optional<int64_t>, padding_idx) = {};
    CS_ARG(c10::optional<double>, max_norm) = {};
    CS_ARG(double, norm_type) = 2.;
    CS_ARG(bool, scale_grad_by_freq) = false;
    CS_ARG(bool, sparse) = false;
    CS_ARG(c10::optional<at::Device>, device) = {};
    CS_ARG(c10::optional<at::ScalarType>, dtype) = {};
  };

  static std::shared_ptr<State> init(const Scheduler &scheduler, const Options &options);

  static Tensor forward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                        const ReadOnlyTensor &indices);

  static void backward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                       const ReadOnlyTensor &grad_output);

  // Not in the reference: token + position embedding in one task each way, replacing the
  // gather, gather, broadcast_to, add of example/gpt2/gpt2_single_device.cpp:541-545 and the
  // sum, backward, backward of :565-567.  `tokens` and `positions` are two Embedding states.
  static Tensor forward_with_positions(const Scheduler &scheduler, const std::shared_ptr<State> &tokens,
                                       const std::shared_ptr<State> &positions,
                                       const ReadOnlyTensor &indices);
  static void backward_with_positions(const Scheduler &scheduler, const std::shared_ptr<State> &tokens,
                                      const std::shared_ptr<State> &positions,
                                      const ReadOnlyTensor &grad_output);
};
}  // namespace cs::compute
