// cs::module::Embedding (the reference's include/module/embedding.h:22-39).
#pragma once
#include "compute/embedding.h"
#include "module/module.h"
#include "module/pimpl.h"

namespace cs::module {
struct CS_API EmbeddingImpl : Module {
  using Options = compute::Embedding::Options;

  explicit EmbeddingImpl(const Scheduler &scheduler, const Options &options);
  Tensor forward(const Scheduler &scheduler, const ReadOnlyTensor &input) const;
  void backward(const Scheduler &scheduler, const ReadOnlyTensor &grad_output) const;
  std::shared_ptr<compute::Embedding::State> state() const;

 protected:
  EmbeddingImpl() = default;
};

CS_MODULE(Embedding);
}  // namespace cs::module
