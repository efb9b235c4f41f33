// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Parameter / gradient bookkeeping interfaces (the reference's include/module/state.h:36-52).
//
// An op that owns parameters (Embedding, LayerNorm) derives its State from module::State and
// names what it holds: parameters() and gradients() use the same keys ("weight", "bias"), and
// increments() pairs each parameter with its gradient, which is what an optimizer walks.
// A gradient handle is undefined until a backward task has produced it; the first backward
// after zero_grad() assigns (`=`), later ones accumulate (`+=`).  zero_grad() makes the handles
// undefined again rather than filling them with zeros, as the reference does
// (src/compute/embedding.cpp:54, src/compute/layer_norm.cpp:69-74).
#pragma once
#include <torch/ordered_dict.h>

#include <string>

#include "tensor.h"

namespace cs {
template <typename Key, typename Value>
using OrderedDict = torch::OrderedDict<Key, Value>;
}

namespace cs::module {
// What an optimizer keeps per parameter (moments, step count, hyper-parameters).
struct OptimizerState {
  virtual ~OptimizerState() = default;
  virtual void set_lr(double lr) const = 0;
  virtual double get_lr() const = 0;
};

struct CS_API State {
  struct Increment {
    Tensor parameter;
    Tensor gradient;  // undefined: the parameter took no part in the last backward pass
  };
  virtual ~State() = default;
  [[nodiscard]] virtual OrderedDict<std::string, Tensor> parameters() const = 0;
  [[nodiscard]] virtual OrderedDict<std::string, Tensor> gradients() const = 0;
  [[nodiscard]] virtual OrderedDict<std::string, Increment> increments() const = 0;
  virtual void zero_grad() = 0;
};
}  // namespace cs::module
