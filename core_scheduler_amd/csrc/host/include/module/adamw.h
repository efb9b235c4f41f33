// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::module::AdamW (the reference's include/module/adamw.h:22-41).  step() updates every
// parameter of the module tree; where the reference submits one task and one kernel launch
// per parameter (src/module/adamw.cpp:32-38), this one submits one task with one launch for
// each group of parameters that share dtype, hyper-parameters and step count: one launch for
// a model built the usual way.
#pragma once
#include "module/optimizer_module.h"
#include "module/pimpl.h"
#include "optimizer/adamw.h"

namespace cs::module {
struct CS_API AdamWImpl : OptimizerModule {
  using Options = optimizer::AdamW::Options;

  explicit AdamWImpl(const Scheduler &scheduler, const Module &module, const Options &options);

  template <typename ModuleHolder, typename = std::enable_if_t<!std::is_base_of_v<module::Module, ModuleHolder>>>
  explicit AdamWImpl(const Scheduler &scheduler, const ModuleHolder &module, const Options &options)
      : AdamWImpl{scheduler, *module, options} {}

  void step(const Scheduler &scheduler) const override;

  // With Options::max_grad_norm set: the global gradient norm of the last step (an undefined
  // handle before the first one).  Clipping needs all parameters in one launch group.
  [[nodiscard]] Tensor last_grad_norm() const { return last_grad_norm_; }

 protected:
  AdamWImpl() = default;
  c10::optional<double> max_grad_norm_{};
  mutable Tensor last_grad_norm_{};
};

CS_MODULE(AdamW);
}  // namespace cs::module
