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
