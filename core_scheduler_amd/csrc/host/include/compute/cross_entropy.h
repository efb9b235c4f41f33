// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::compute::CrossEntropy, the reference's op interface (include/compute/cross_entropy.h:25-60).
// forward returns the loss; backward returns the gradient of the logits (no upstream gradient
// argument: the reference feeds ones_like(loss)).  Here forward computes both in one pass and
// keeps the gradient in state->backward.log_probs; backward hands it out.
//
// Logits are [N, columns] (two dimensions), targets [N] int64.  Rows whose target equals
// ignore_index, or lies outside the class range, add nothing to the loss and get a zero
// gradient; the mean is over the other rows.  label_smoothing other than 0 aborts in init, as
// in the reference.  Inside the autocast guard the gradient of 16-bit logits is fp32 (what
// ATen's autocast rule gives the reference); outside it keeps the logits' type.
#pragma once
#include <ATen/core/Reduction.h>

#include "arg.h"
#include "tensor.h"
#include "threading/scheduler.h"

namespace cs::compute {
struct CS_API CrossEntropy {
  struct State {
    struct Forward {
      ReadOnlyTensor weight;  // per-class weights: never set by any caller of the reference
    } forward;
    struct Backward {  // filled by forward, released by backward
      ReadOnlyTensor total_weight;  // number of rows that counted, as a 0-d fp32 tensor
      ReadOnlyTensor log_probs;     // holds d(loss)/d(logits) after forward
      ReadOnlyTensor target;
      ReadOnlyTensor loss;
    } backward;
    struct Args {
      int64_t reduction;  // at::Reduction::{None, Mean, Sum}
      int64_t ignore_index;
      double label_smoothing;
      int64_t num_classes;  // class columns of the logits; < 0: all of them (the reference)
    } args;
  };

  struct Options {
    Options() {}
    CS_ARG(at::Reduction::Reduction, reduction) = at::Reduction::Mean;
    CS_ARG(int64_t, ignore_index) = -100;
    CS_ARG(double, label_smoothing) = 0.0;
    // not in the reference: softmax over the first num_classes columns only (lm_head pads
    // 50257 classes to 50304 columns, example/gpt2/gpt2_single_device.cpp:60)
    CS_ARG(int64_t, num_classes) = -1;
  };

  static std::shared_ptr<State> init(const Scheduler &scheduler, const Options &options = {});

  static Tensor forward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                        const ReadOnlyTensor &input, const ReadOnlyTensor &target);

  static Tensor backward(const Scheduler &scheduler, const std::shared_ptr<State> &state);
};
}  // namespace cs::compute
