// The three-stream scheduler (the reference's include/threading/dynamic_scheduler.h).
#pragma once
#include "threading/scheduler.h"

namespace cs {
struct DynamicScheduler : Scheduler {
  CS_API explicit DynamicScheduler(int localRank);
};
}  // namespace cs
