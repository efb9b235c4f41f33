// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Tensor handles of the op API (the reference's include/tensor.h:36-63).
//
// A handle is a shared pointer to {at::Tensor, completion event, the lane of the stream that
// produced it} (internal/tensor_impl.h).  Ops return empty handles at once; the task they
// submit fills the at::Tensor in and the scheduler records the event, so a handle can be
// passed to the next op before anything has run on the device.  Copying a handle shares the
// state; reset() detaches it (the ops do that with what they saved for backward, so the
// memory goes back to the allocator as soon as the last task using it has been submitted).
// ReadOnlyTensor is what an op takes as input, Tensor what it returns and may write.
#pragma once
#include <ATen/core/TensorBody.h>

#include <memory>
#include <ostream>

#include "export.h"

namespace cs {
using Scalar = at::Scalar;
using IntArrayRef = at::IntArrayRef;
using IntArray = c10::SmallVector<IntArrayRef::value_type>;
using TensorOptions = at::TensorOptions;
template <typename Element>
using optional = c10::optional<Element>;

struct ReadOnlyTensor {
  CS_API ReadOnlyTensor();  // an empty handle: an undefined at::Tensor, nothing to wait for

  // Shape and type of the tensor behind the handle.  They are known once the producing task
  // has been submitted (tasks run inline on the submitting thread), not only after wait().
  CS_API [[nodiscard]] TensorOptions options() const;
  CS_API [[nodiscard]] IntArrayRef sizes() const;
  CS_API [[nodiscard]] int64_t size(int64_t dim) const;
  CS_API [[nodiscard]] int64_t numel() const;

  // Blocks the calling thread until the device has finished the task that produced the
  // tensor.  The only host-side synchronisation in the API; ops never need it between them.
  CS_API void wait() const;

  struct Impl;
  CS_API [[nodiscard]] const std::shared_ptr<Impl> &impl() const;
  CS_API void reset();

 protected:
  std::shared_ptr<Impl> impl_;
};

struct Tensor : ReadOnlyTensor {
  CS_API Tensor() = default;
  CS_API void wait() const;
};

// Waits for the tensor, then prints it the way at::print does (`linesize` characters per line).
CS_API std::ostream &print(std::ostream &stream, const ReadOnlyTensor &tensor, int64_t linesize);

inline std::ostream &operator<<(std::ostream &out, const ReadOnlyTensor &t) { return print(out, t, 80); }
}  // namespace cs

// The comparisons the reference's tests use on handles: wait, then at::allclose with its defaults.
namespace at {
CS_API bool allclose(const cs::ReadOnlyTensor &t1, const at::Tensor &t2, double rtol = 1e-05,
                     double atol = 1e-08, bool equal_nan = false);
CS_API bool allclose(const cs::ReadOnlyTensor &t1, const cs::ReadOnlyTensor &t2, double rtol = 1e-05,
                     double atol = 1e-08, bool equal_nan = false);
CS_API bool allclose(const at::Tensor &t1, const cs::ReadOnlyTensor &t2, double rtol = 1e-05,
                     double atol = 1e-08, bool equal_nan = false);
}  // namespace at
