// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// What a tensor handle points to (the reference's include/internal/tensor_impl.h:30-59).
//
// Three things travel with the device tensor: the lane (stream) whose task produced it, the
// event recorded on that stream after the task, and the autocast request in force when the
// handle was made.  A consumer on another lane makes its stream wait for the event unless the
// event has completed already; a consumer on the same lane relies on stream order.
#pragma once
#include <memory>
#include <ATen/core/TensorBody.h>

#include "tensor.h"
#include "threading/event.h"
#include "threading/task_impl.h"

namespace cs {
struct ReadOnlyTensor::Impl {
  // lane of the producing task; kNumPriority for tensors that came from outside (from_torch),
  // which every consumer then waits for
  Task::Impl::Priority priority_ = Task::Impl::kMain;
  auto &priority() { return priority_; }
  auto &priority() const { return priority_; }

  // recorded by the scheduler after the producing task's body has enqueued its kernels
  Event event_;
  auto &event() { return event_; }
  auto &event() const { return event_; }

  // Launches that still have to be enqueued before the tensor holds its value: the column sums
  // of a LayerNorm backward are added up inside the NEXT LayerNorm backward launch, so until
  // that launch (or a launch of their own) the weight and bias gradients are only partial rows.
  // Whoever is about to read or write the tensor - the scheduler for a task's inputs and
  // outputs, wait() for the host - calls settle() first; it enqueues what is missing on the
  // stream of the producing task and stamps the tensor with a fresh event.
  struct Deferred {
    virtual ~Deferred() = default;
    virtual void settle() = 0;  // also clears deferred_ of every tensor it completes
  };
  std::shared_ptr<Deferred> deferred_;
  auto &deferred() { return deferred_; }
  void settle() {
    if (deferred_) {
      const auto keep = deferred_;
      keep->settle();
    }
  }

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
  // task bodies assign here; undefined until the producing task has been submitted
  auto &tensor() { return tensor_; }

  at::Tensor tensor_{};
};
}  // namespace cs
