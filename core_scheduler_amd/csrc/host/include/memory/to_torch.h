// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Copy of a cs tensor as an at::Tensor (the reference's test helper, include/memory/to_torch.h).
#pragma once
#include <ATen/core/TensorBody.h>

#include "tensor.h"
#include "threading/scheduler.h"

namespace cs::memory {
CS_API at::Tensor to_torch(const Scheduler &scheduler, const ReadOnlyTensor &tensor);
// The other direction, for callers that already hold device data: a task that makes `handle`
// refer to `tensor` (no copy).
CS_API Tensor from_torch(const Scheduler &scheduler, const at::Tensor &tensor);
}  // namespace cs::memory
