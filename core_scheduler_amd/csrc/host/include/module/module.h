// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::module::Module: a tree of named submodules, each with at most one parameter state
// (the reference's include/module/module.h:27-69, src/module/module.cpp:33-127).
//
// The tree exists to name things.  A leaf (Embedding, LayerNorm) registers the State of its
// op; a container registers children under names without dots.  named_states() walks the tree
// depth first in registration order and joins the names with '.', and named_parameters /
// named_gradients / named_increments append the key the state uses for each tensor, which
// gives the "h.0.ln_1.weight" names that checkpoints and optimizers go by.  Modules hold no
// device memory of their own; zero_grad() and to() forward to the states.
#pragma once
#include <torch/nn/pimpl.h>

#include <functional>
#include <memory>
#include <stdexcept>
#include <string>

#include "module/state.h"

namespace cs::module {
struct CS_API Module : std::enable_shared_from_this<Module> {
  virtual ~Module() = default;
  using NamedModulePointerApplyFunction = std::function<void(const std::string &, const std::shared_ptr<Module> &)>;
  using ConstNamedModuleApplyFunction = std::function<void(const std::string &, const Module &)>;

  // depth-first over the children, names joined with '.'
  void apply_to_submodules(const NamedModulePointerApplyFunction &function,
                           const std::string &name_prefix = std::string(), std::size_t depth = 0) const;
  // this module first (under `name_prefix`), then every submodule
  void apply(const ConstNamedModuleApplyFunction &function, const std::string &name_prefix = {}) const;

  // at most one state per module: a second call replaces the first
  void register_state(std::shared_ptr<State> state);

  // Adds a child and returns it.  Throws std::runtime_error for an empty name, a name with a
  // dot in it or a name already taken.  The second form takes a holder (cs::module::LayerNorm).
  template <typename ModuleType>
  std::shared_ptr<ModuleType> register_module(std::string name, std::shared_ptr<ModuleType> module);
  template <typename ModuleType>
  std::shared_ptr<ModuleType> register_module(std::string name, torch::nn::ModuleHolder<ModuleType> module_holder);

  // keys are module paths ("h.0.ln_1"); modules without a state do not appear
  OrderedDict<std::string, std::shared_ptr<State>> named_states() const;
  // keys are "<module path>.<name inside the state>", e.g. "wte.weight"
  OrderedDict<std::string, Tensor> named_parameters(bool recurse = true) const;
  OrderedDict<std::string, Tensor> named_gradients(bool recurse = true) const;
  OrderedDict<std::string, State::Increment> named_increments(bool recurse = true) const;

  void zero_grad() const;  // gradients become undefined handles
  // converts every parameter (dtype / device of `options`); gradients are dropped
  void to(TensorOptions options) const;

 protected:
  OrderedDict<std::string, std::shared_ptr<Module>> children_;
  std::shared_ptr<State> state_;
};

template <typename ModuleType>
std::shared_ptr<ModuleType> Module::register_module(std::string name, std::shared_ptr<ModuleType> module) {
  if (name.empty()) throw std::runtime_error("Submodule name must not be empty");
  if (name.find('.') != std::string::npos)
    throw std::runtime_error("Submodule name must not contain a dot (got '" + name + "')");
  auto &base = children_.insert(std::move(name), std::move(module));
  return std::dynamic_pointer_cast<ModuleType>(base);
}

template <typename ModuleType>
std::shared_ptr<ModuleType> Module::register_module(std::string name,
                                                    torch::nn::ModuleHolder<ModuleType> module_holder) {
  return register_module(std::move(name), module_holder.ptr());
}
}  // namespace cs::module

// Checkpoints in the reference's Parquet layout (the reference's include/module/module.h:92-108,
// src/module/module.cpp:129-220): one row per parameter, `key` = qualified name, `value` = the
// parameter flattened as float32.  load copies every row of the file into the parameter of that
// name (converted to its dtype, device and shape); a name the module does not have aborts.
// Both wait for the tensors they touch; the second form takes a holder (cs::module::LayerNorm).
namespace cs {
CS_API void save(const module::Module &module, const std::string &path);

template <typename Module, typename = std::enable_if_t<!std::is_base_of_v<module::Module, Module> &&
                                                       !std::is_base_of_v<ReadOnlyTensor, Module>>>
static void save(const Module &module, const std::string &path) {
  save(*module, path);
}

CS_API void load(const module::Module &module, const std::string &path);

template <typename Module, typename = std::enable_if_t<!std::is_base_of_v<module::Module, Module> &&
                                                       !std::is_base_of_v<ReadOnlyTensor, Module>>>
static void load(const Module &module, const std::string &path) {
  load(*module, path);
}
}  // namespace cs
