// cs::compute::LayerNorm, the reference's op interface (include/compute/layer_norm.h:24-87).
#pragma once
#include "arg.h"
#include "module/state.h"
#include "tensor.h"
#include "threading/scheduler.h"

namespace cs::compute {
struct CS_API LayerNorm {
  struct State : virtual module::State {
    struct Forward {
      Tensor weight;
      Tensor bias{};
      Tensor grad_weight{};
      Tensor grad_bias{};
    } forward;
    struct Backward {
      ReadOnlyTensor input{};
      ReadOnlyTensor mean{};
      ReadOnlyTensor rstd{};
    } backward;
    struct Args {
      const IntArray normalized_shape;
      const double eps;
      const bool elementwise_affine;
      const bool bias;
    } args;

    State(const Forward &forward, const Backward &backward, const Args &args);
    [[nodiscard]] OrderedDict<std::string, Tensor> parameters() const override;
    [[nodiscard]] OrderedDict<std::string, Tensor> gradients() const override;
    [[nodiscard]] OrderedDict<std::string, Increment> increments() const override;
    void zero_grad() override;
  };

  struct Options {
    Options(IntArrayRef normalized_shape) : normalized_shape_{normalized_shape} {}
    CS_ARG(IntArray, normalized_shape);
    CS_ARG(double, eps) = 1e-05;
    CS_ARG(bool, elementwise_affine) = true;
    CS_ARG(bool, bias) = true;
    CS_ARG(c10::optional<at::Device>, device) = {};
    CS_ARG(c10::optional<at::ScalarType>, dtype) = {};
  };

  static std::shared_ptr<State> init(const Scheduler &scheduler, const Options &options);

  static Tensor forward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                        const ReadOnlyTensor &input);

  // One task on the main stream producing dx, dgamma and dbeta from a single pass over dy
  // and x (the reference submits a parameter task on the assist stream and an input task on
  // the main stream, each a full native_layer_norm_backward call).
  static Tensor backward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                         const ReadOnlyTensor &grad_output);
};
}  // namespace cs::compute
