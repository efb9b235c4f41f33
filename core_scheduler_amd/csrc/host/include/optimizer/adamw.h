// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::optimizer::AdamW, the reference's optimizer interface (include/optimizer/adamw.h:33-75).
#pragma once
#include <vector>

#include "arg.h"
#include "module/state.h"
#include "tensor.h"
#include "threading/scheduler.h"

namespace cs::optimizer {
struct CS_API AdamW {
  AdamW() = delete;

  struct State final : module::OptimizerState {
    struct Tensors {
      Tensor m;
      Tensor v;
      Tensor v_max{};
    } tensors;
    struct Options {
      mutable double lr = 1e-3;
      const double beta1 = 0.9;
      const double beta2 = 0.999;
      const double eps = 1e-8;
      const double weight_decay = 1e-2;
      const bool amsgrad = false;
      long t = 0;
    } options;

    State(const Tensors &tensors, const Options &options);
    void set_lr(double lr) const override;
    double get_lr() const override;
  };

  struct Options {
    CS_ARG(double, lr) = 1e-3;
    CS_ARG(double, beta1) = 0.9;
    CS_ARG(double, beta2) = 0.999;
    CS_ARG(double, eps) = 1e-8;
    CS_ARG(double, weight_decay) = 1e-2;
    CS_ARG(bool, amsgrad) = false;
    CS_ARG(long, t) = 0;
    // Not in the reference (its example leaves clipping as a TODO,
    // example/gpt2/gpt2_single_device.cpp:706): module::AdamW clips the global gradient norm to
    // this value inside its step.
    CS_ARG(c10::optional<double>, max_grad_norm) = {};
    // example/gpt2/gpt2_single_device.cpp:619 sets `.fused(true)`, an option the reference's own
    // header does not declare; it is accepted here so that the example builds.  module::AdamW
    // updates all parameters in one launch either way.
    CS_ARG(bool, fused) = true;
  };

  static std::shared_ptr<State> init(const Scheduler &scheduler, const ReadOnlyTensor &parameter,
                                     const Options &options);

  static void step(const Scheduler &scheduler, const std::shared_ptr<module::OptimizerState> &state,
                   const Tensor &w, const ReadOnlyTensor &dw);

  // Not in the reference: every parameter of a model in one task and one kernel launch
  // (the loop of src/module/adamw.cpp:32-38).  All states must share hyper-parameters and
  // step count; parameters with an undefined gradient are skipped with a warning, as the
  // single-tensor step does.
  static void step(const Scheduler &scheduler,
                   const std::vector<std::shared_ptr<module::OptimizerState>> &states,
                   const std::vector<Tensor> &ws, const std::vector<ReadOnlyTensor> &dws);

  // The same with Utils::clip_grad_norm_ (src/compute/utils.cpp:700-746) folded in: the global
  // norm is taken first and the step scales each gradient as it reads it, so the gradients
  // themselves are left as they were.  Returns the 0-d norm (undefined handle if nothing ran).
  static Tensor step(const Scheduler &scheduler,
                     const std::vector<std::shared_ptr<module::OptimizerState>> &states,
                     const std::vector<Tensor> &ws, const std::vector<ReadOnlyTensor> &dws,
                     c10::optional<double> max_grad_norm, double norm_type = 2.0);
};
}  // namespace cs::optimizer
