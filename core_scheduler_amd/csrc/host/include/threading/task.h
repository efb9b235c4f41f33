// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// A unit of work handed to a scheduler (the reference's include/threading/task.h).
#pragma once
#include <memory>
#include <vector>

#include "tensor.h"

namespace cs {
struct Task {
  struct Impl;
  CS_API explicit Task(std::shared_ptr<Impl> impl);
  CS_API void operator()() const;
  [[nodiscard]] const std::shared_ptr<Impl> &impl() const;
  CS_API void reset();

 private:
  std::shared_ptr<Impl> impl_;
};
}  // namespace cs
