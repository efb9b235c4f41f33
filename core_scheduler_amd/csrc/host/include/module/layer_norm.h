// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::module::LayerNorm (the reference's include/module/layer_norm.h:22-39): the op's state
// registered in a module tree, so that its parameters appear in named_parameters() under the
// module's path ("h.0.ln_1.weight") and an optimizer module finds them.  forward and backward
// pass straight through to cs::compute::LayerNorm with the registered state.
#pragma once
#include "compute/layer_norm.h"
#include "module/module.h"
#include "module/pimpl.h"

namespace cs::module {
struct CS_API LayerNormImpl : Module {
  using Options = compute::LayerNorm::Options;

  explicit LayerNormImpl(const Scheduler &scheduler, const Options &options);
  Tensor forward(const Scheduler &scheduler, const ReadOnlyTensor &input) const;
  Tensor backward(const Scheduler &scheduler, const ReadOnlyTensor &grad_output) const;
  // the registered state with its concrete type (weight, bias, their gradients, saved tensors)
  std::shared_ptr<compute::LayerNorm::State> state() const;

 protected:
  LayerNormImpl() = default;
};

CS_MODULE(LayerNorm);  // cs::module::LayerNorm: a shared-pointer holder of LayerNormImpl
}  // namespace cs::module
