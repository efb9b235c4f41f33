// Task body interface (the reference's include/internal/threading/task_impl.h:23-61).
#pragma once
#include <ATen/core/TensorBody.h>

#include <utility>
#include <vector>

#include "threading/task.h"

namespace cs {
struct Task::Impl {
  enum Type { kConfig = 0, kCompute, kLoader, kMemcpy, kNccl, kNumType };
  enum Priority { kMain = 0, kAssist, kComm, kNumPriority };

  virtual ~Impl() = default;
  Impl(std::vector<Tensor> output, std::vector<ReadOnlyTensor> input, const Priority priority,
       const Type type)
      : output_{std::move(output)}, input_{std::move(input)}, priority_{priority}, type_{type} {}

  [[nodiscard]] auto &input() const { return input_; }
  [[nodiscard]] auto &output() const { return output_; }
  // device memory a side-stream task must keep alive until its stream has run
  [[nodiscard]] auto &intermediate() const { return intermediate_; }
  [[nodiscard]] auto &type() const { return type_; }
  [[nodiscard]] auto &priority() const { return priority_; }

  virtual void operator()() const = 0;
  [[nodiscard]] virtual const char *name() const = 0;

 private:
  std::vector<Tensor> output_;
  std::vector<ReadOnlyTensor> input_;
  mutable std::vector<at::Tensor> intermediate_;
  Priority priority_;
  Type type_;
};
}  // namespace cs
