// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// RAII switch for ATen autocast on the submitting thread (the reference's include/autocast.h).
// The ops below consult at::autocast::is_enabled() the way ATen's own policy would apply to
// the calls the reference makes: LayerNorm and the cross-entropy gradient come out in fp32.
#pragma once
#include <ATen/core/TensorBody.h>

#include "export.h"
#include "threading/scheduler.h"

namespace cs::autocast {
struct CS_API ContextGuard {
  ContextGuard(const Scheduler &scheduler, at::ScalarType dtype);
  ~ContextGuard();

 private:
  bool previous_;
  at::ScalarType previous_dtype_;
};
}  // namespace cs::autocast
