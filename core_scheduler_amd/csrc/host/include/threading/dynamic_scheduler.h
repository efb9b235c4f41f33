// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// The three-stream scheduler (the reference's include/threading/dynamic_scheduler.h).
#pragma once
#include "threading/scheduler.h"

namespace cs {
struct DynamicScheduler : Scheduler {
  CS_API explicit DynamicScheduler(int localRank);
};
}  // namespace cs
