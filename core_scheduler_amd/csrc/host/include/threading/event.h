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
