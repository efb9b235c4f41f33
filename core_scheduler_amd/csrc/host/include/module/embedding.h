// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::module::Embedding (the reference's include/module/embedding.h:22-39): the op's state
// registered in a module tree ("wte.weight" in named_parameters()).  forward and backward pass
// straight through to cs::compute::Embedding; backward returns nothing, the gradient of the
// table is left in the state (on the assist stream) for the optimizer to pick up.
#pragma once
#include "compute/embedding.h"
#include "module/module.h"
#include "module/pimpl.h"

namespace cs::module {
struct CS_API EmbeddingImpl : Module {
  using Options = compute::Embedding::Options;

  explicit EmbeddingImpl(const Scheduler &scheduler, const Options &options);
  Tensor forward(const Scheduler &scheduler, const ReadOnlyTensor &input) const;
  void backward(const Scheduler &scheduler, const ReadOnlyTensor &grad_output) const;
  // the registered state with its concrete type (table, its gradient, the saved indices)
  std::shared_ptr<compute::Embedding::State> state() const;

 protected:
  EmbeddingImpl() = default;
};

CS_MODULE(Embedding);  // cs::module::Embedding: a shared-pointer holder of EmbeddingImpl
}  // namespace cs::module
