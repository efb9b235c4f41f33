// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Scheduler implementation interface (the reference's include/internal/threading/scheduler_impl.h).
#pragma once
#include "threading/scheduler.h"
#include "threading/task.h"

namespace cs {
struct Scheduler::Impl {
  explicit Impl(int64_t deviceRank) : device_rank_{deviceRank} {}
  virtual ~Impl() = default;
  virtual void submit(Task &&task);
  [[nodiscard]] int64_t device_rank() const { return device_rank_; }

 protected:
  const int64_t device_rank_;
};
}  // namespace cs
