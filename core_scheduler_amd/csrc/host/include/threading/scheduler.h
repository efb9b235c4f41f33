// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Scheduler handle (the reference's include/threading/scheduler.h).
#pragma once
#include <cstdint>
#include <memory>

#include "export.h"

namespace cs {
struct Scheduler {
  struct Impl;
  [[nodiscard]] const std::shared_ptr<Impl> &impl() const { return impl_; }
  CS_API [[nodiscard]] int64_t get_device_rank() const;

 protected:
  std::shared_ptr<Impl> impl_;
};
}  // namespace cs
