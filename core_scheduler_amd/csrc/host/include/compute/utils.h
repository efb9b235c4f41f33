// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// The part of cs::compute::Utils that belongs to the optimizer path (the reference's
// include/compute/utils.h:106-108, src/compute/utils.cpp:700-746).
#pragma once
#include <vector>

#include "tensor.h"
#include "threading/scheduler.h"

namespace cs::compute::Utils {
// total = || all gradients ||_p (p = 2 or +infinity), every gradient is multiplied in place by
// min(1, max_norm / (total + 1e-6)); returns the 0-d norm.  Undefined gradients are skipped.
CS_API Tensor clip_grad_norm_(const Scheduler &scheduler, const std::vector<Tensor> &tensor, double max_norm,
                              double norm_type);
}  // namespace cs::compute::Utils
