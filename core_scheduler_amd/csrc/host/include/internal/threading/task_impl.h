// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Task body interface (the reference's include/internal/threading/task_impl.h:23-61).
//
// A task is what an op call turns into: the handles it will fill (output), the handles it
// reads (input), the scheduler lane it runs on (priority) and a body.  The scheduler runs the
// body inline on the submitting thread, under a guard that makes the lane's HIP stream
// current, after it has made that stream wait for every input produced on another lane; when
// the body returns it stamps every output with the lane and a fresh event.  A body therefore
// only allocates (at::empty) and enqueues kernels on the current stream: it never
// synchronises and never touches another stream.
#pragma once
#include <ATen/core/TensorBody.h>

#include <memory>
#include <utility>
#include <vector>

#include "threading/task.h"

namespace cs {
struct Task::Impl {
  // What a task does.  Only kConfig changes scheduling: such a task runs at once, outside
  // any lane (the autocast guard is one).  The other values are labels for tracing.
  enum Type { kConfig = 0, kCompute, kLoader, kMemcpy, kNccl, kNumType };
  // The lane: main carries the forward/backward chain, assist the work that may trail it
  // (parameter gradients, optimizer state initialisation), comm would carry collectives.
  // kNumPriority doubles as "produced outside any lane" for handles made from torch tensors.
  enum Priority { kMain = 0, kAssist, kComm, kNumPriority };

  virtual ~Impl() = default;
  Impl(std::vector<Tensor> output, std::vector<ReadOnlyTensor> input, const Priority priority,
       const Type type)
      : output_{std::move(output)}, input_{std::move(input)}, priority_{priority}, type_{type} {}

  // Handles the body reads.  The scheduler looks at their lane and event before the body runs.
  [[nodiscard]] auto &input() const { return input_; }
  // Handles the body fills: it assigns impl()->tensor(); lane and event are the scheduler's.
  [[nodiscard]] auto &output() const { return output_; }
  // Device memory that is neither input nor output (workspaces, descriptor tables).  A body on
  // a side lane pushes such tensors here: the scheduler keeps them, with inputs and outputs,
  // until the main stream has been made to wait for the task, so the caching allocator cannot
  // hand the blocks to main-stream work while the side stream still uses them.
  [[nodiscard]] auto &intermediate() const { return intermediate_; }
  // Tensors of EARLIER tasks whose contents this body's launches completed (a LayerNorm backward
  // adds up the column sums the previous one left).  The body pushes them here; the scheduler
  // stamps them with this task's lane and event, as it stamps the outputs.
  [[nodiscard]] auto &completed() const { return completed_; }
  [[nodiscard]] auto &type() const { return type_; }
  [[nodiscard]] auto &priority() const { return priority_; }

  virtual void operator()() const = 0;
  // "cs::compute::GeLU::forward" and the like; appears in the abort message when a body throws.
  [[nodiscard]] virtual const char *name() const = 0;

 private:
  std::vector<Tensor> output_;
  std::vector<ReadOnlyTensor> input_;
  mutable std::vector<at::Tensor> intermediate_;
  mutable std::vector<std::shared_ptr<ReadOnlyTensor::Impl>> completed_;
  Priority priority_;
  Type type_;
};
}  // namespace cs
