// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::compute::GeLU, the reference's op interface (include/compute/gelu.h:23-42):
// init / forward / backward, the input saved in state->backward for the backward pass.
#pragma once
#include "arg.h"
#include "tensor.h"
#include "threading/scheduler.h"

namespace cs::compute {
struct CS_API GeLU {
  struct State {
    struct Forward {
    } forward;
    struct Backward {
      ReadOnlyTensor input;
    } backward;
    struct Args {
      // 0: exact (erf) form, what the reference always computes; 1: at::gelu(x, "tanh").
      // Not in the reference's Args; it defaults to the reference's behaviour.
      int approximate = 0;
    } args;
  };

  struct Options {
    Options() {}
    CS_ARG(int, approximate) = 0;
  };

  static std::shared_ptr<State> init(const Scheduler &scheduler);
  static std::shared_ptr<State> init(const Scheduler &scheduler, const Options &options);

  static Tensor forward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                        const ReadOnlyTensor &input);

  static Tensor backward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                         const ReadOnlyTensor &grad_output);
};
}  // namespace cs::compute
