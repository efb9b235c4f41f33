// Parameter / gradient bookkeeping interfaces (the reference's include/module/state.h:36-52).
#pragma once
#include <torch/ordered_dict.h>

#include <string>

#include "tensor.h"

namespace cs {
template <typename Key, typename Value>
using OrderedDict = torch::OrderedDict<Key, Value>;
}

namespace cs::module {
struct OptimizerState {
  virtual ~OptimizerState() = default;
  virtual void set_lr(double lr) const = 0;
  virtual double get_lr() const = 0;
};

struct CS_API State {
  struct Increment {
    Tensor parameter;
    Tensor gradient;
  };
  virtual ~State() = default;
  [[nodiscard]] virtual OrderedDict<std::string, Tensor> parameters() const = 0;
  [[nodiscard]] virtual OrderedDict<std::string, Tensor> gradients() const = 0;
  [[nodiscard]] virtual OrderedDict<std::string, Increment> increments() const = 0;
  virtual void zero_grad() = 0;
};
}  // namespace cs::module
