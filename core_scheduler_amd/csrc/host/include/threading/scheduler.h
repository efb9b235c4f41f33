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
