// cs::module::LayerNorm (the reference's include/module/layer_norm.h:22-39).
#pragma once
#include "compute/layer_norm.h"
#include "module/module.h"
#include "module/pimpl.h"

namespace cs::module {
struct CS_API LayerNormImpl : Module {
  using Options = compute::LayerNorm::Options;

  explicit LayerNormImpl(const Scheduler &scheduler, const Options &options);
  Tensor forward(const Scheduler &scheduler, const ReadOnlyTensor &input) const;
  Tensor backward(const Scheduler &scheduler, const ReadOnlyTensor &grad_output) const;
  std::shared_ptr<compute::LayerNorm::State> state() const;

 protected:
  LayerNormImpl() = default;
};

CS_MODULE(LayerNorm);
}  // namespace cs::module
