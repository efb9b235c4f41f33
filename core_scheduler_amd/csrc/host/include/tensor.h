// Tensor handles of the op API (the reference's include/tensor.h:36-63).
// A handle is a shared pointer to {at::Tensor, completion event, the priority of
// the stream that produced it}.  Ops return empty handles at once and a task
// fills them in; wait() blocks the host until the producing task has run.
#pragma once
#include <ATen/core/TensorBody.h>

#include <memory>

#include "export.h"

namespace cs {
using Scalar = at::Scalar;
using IntArrayRef = at::IntArrayRef;
using IntArray = c10::SmallVector<IntArrayRef::value_type>;
using TensorOptions = at::TensorOptions;
template <typename Element>
using optional = c10::optional<Element>;

struct ReadOnlyTensor {
  CS_API ReadOnlyTensor();
  CS_API [[nodiscard]] TensorOptions options() const;
  CS_API [[nodiscard]] IntArrayRef sizes() const;
  CS_API [[nodiscard]] int64_t size(int64_t dim) const;
  CS_API [[nodiscard]] int64_t numel() const;
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
}  // namespace cs

namespace at {
CS_API bool allclose(const cs::ReadOnlyTensor &t1, const at::Tensor &t2, double rtol = 1e-05,
                     double atol = 1e-08, bool equal_nan = false);
CS_API bool allclose(const cs::ReadOnlyTensor &t1, const cs::ReadOnlyTensor &t2, double rtol = 1e-05,
                     double atol = 1e-08, bool equal_nan = false);
CS_API bool allclose(const at::Tensor &t1, const cs::ReadOnlyTensor &t2, double rtol = 1e-05,
                     double atol = 1e-08, bool equal_nan = false);
}  // namespace at
