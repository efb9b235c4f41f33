// What a tensor handle points to (the reference's include/internal/tensor_impl.h:30-59).
#pragma once
#include <ATen/core/TensorBody.h>

#include "tensor.h"
#include "threading/event.h"
#include "threading/task_impl.h"

namespace cs {
struct ReadOnlyTensor::Impl {
  Task::Impl::Priority priority_ = Task::Impl::kMain;
  auto &priority() { return priority_; }
  auto &priority() const { return priority_; }

  Event event_;
  auto &event() { return event_; }
  auto &event() const { return event_; }

  struct {
    bool enable = false;
    c10::ScalarType dtype = c10::ScalarType::Undefined;
  } auto_cast_;
  auto &auto_cast() { return auto_cast_; }
  auto &auto_cast() const { return auto_cast_; }

  Impl() = default;
  [[nodiscard]] auto options() const { return tensor_.options(); }
  [[nodiscard]] auto sizes() const { return tensor_.sizes(); }
  [[nodiscard]] auto size(const int64_t dim) const { return tensor_.size(dim); }
  [[nodiscard]] auto numel() const { return tensor_.numel(); }
  auto &tensor() { return tensor_; }

  at::Tensor tensor_{};
};
}  // namespace cs
