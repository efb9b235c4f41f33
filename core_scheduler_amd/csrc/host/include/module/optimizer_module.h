// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::module::OptimizerModule: the optimizer states of every parameter of a module tree
// (the reference's include/module/optimizer_module.h:29-52, src/module/optimizer_module.cpp:22-41).
#pragma once
#include <memory>
#include <string>

#include "module/module.h"
#include "module/state.h"
#include "threading/scheduler.h"

namespace cs::module {
struct CS_API OptimizerModule : std::enable_shared_from_this<OptimizerModule> {
  virtual ~OptimizerModule() = default;

  OrderedDict<std::string, std::shared_ptr<OptimizerState>> named_states() const;
  void set_lr(double lr) const;
  double get_lr() const;
  virtual void step(const Scheduler &scheduler) const = 0;
  // gradients are set to undefined, not to zero
  void zero_grad(const Scheduler &scheduler) const;

 protected:
  OrderedDict<std::string, std::shared_ptr<OptimizerState>> states_;
  std::weak_ptr<const Module> module_;
};
}  // namespace cs::module

// Optimizer checkpoints (declared in the reference's include/module/optimizer_module.h:54-60; its
// definitions abort with "not implemented", src/module/optimizer_module.cpp:45-51).  Here:
// AdamW's m, v (and v_max) and step count per parameter, in the layout of cs::save(Module).
namespace cs {
CS_API void save(const module::OptimizerModule &module, const std::string &path);
CS_API void load(const module::OptimizerModule &module, const std::string &path);
}  // namespace cs
