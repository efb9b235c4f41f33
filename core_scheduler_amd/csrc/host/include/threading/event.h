// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Stream event handle (the reference's include/threading/event.h).
#pragma once
#include <memory>

#include "export.h"

namespace cs {
struct Event {
  struct Impl;
  CS_API Event();
  CS_API explicit Event(std::shared_ptr<Impl> impl);
  CS_API ~Event();
  CS_API void block() const;        // the current stream waits for the event
  CS_API void record() const;       // record on the current stream
  CS_API [[nodiscard]] bool query() const;
  CS_API void synchronize() const;  // the host waits for the event
  [[nodiscard]] const std::shared_ptr<Impl> &impl() const;

 private:
  std::shared_ptr<Impl> impl_;
};
}  // namespace cs
