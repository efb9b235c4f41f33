// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// cs::compute::LayerNorm, the reference's op interface (include/compute/layer_norm.h:24-87).
//
// init makes gamma = 1 and beta = 0 of `normalized_shape` (one trailing dimension here: the
// kernels normalise rows of C = normalized_shape[0] columns).  forward writes y and keeps the
// input and the per-row statistics for backward: mean and rstd = 1/sqrt(biased variance + eps),
// fp32 whatever the input type.  backward returns dx and leaves dgamma / dbeta in
// state->forward.grad_weight / grad_bias: assigned when those handles are undefined,
// accumulated into otherwise.  Under the autocast guard y and dx are fp32 for 16-bit inputs,
// as at::native_layer_norm behaves with fp32 parameters.
#pragma once
#include "arg.h"
#include "module/state.h"
#include "tensor.h"
#include "threading/scheduler.h"

namespace cs::compute {
struct CS_API LayerNorm {
  struct State : virtual module::State {
    struct Forward {
      Tensor weight;         // gamma [C]
      Tensor bias{};         // beta [C]; stays an empty handle with Options::bias(false)
      Tensor grad_weight{};  // dgamma, undefined until the first backward
      Tensor grad_bias{};    // dbeta
    } forward;
    struct Backward {  // filled by forward, released once backward has been submitted
      ReadOnlyTensor input{};
      ReadOnlyTensor mean{};  // [rows] fp32
      ReadOnlyTensor rstd{};  // [rows] fp32
    } backward;
    struct Args {
      const IntArray normalized_shape;
      const double eps;
      const bool elementwise_affine;
      const bool bias;
    } args;

    State(const Forward &forward, const Backward &backward, const Args &args);
    // "weight" and, if there is one, "bias"
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
  // the main stream, each a full native_layer_norm_backward call; the second stream costs the
  // main stream more in waiting than the 4 us of summing it would take over).
  static Tensor backward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                         const ReadOnlyTensor &grad_output);

  // Extensions (no counterpart in the reference's header): the residual stream around a norm
  // as one task each way.  The reference's GPT-2 block adds and then normalises
  // (example/gpt2/gpt2_single_device.cpp:459-460) and, going back, differentiates and then adds
  // (:468-469); the sum and the norm here come out of one kernel with the bits of the two.
  struct WithResidual {
    Tensor output;    // LayerNorm(input + residual)
    Tensor residual;  // input + residual, rounded once to the input's type: the new residual stream
  };
  static WithResidual forward_with_residual(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                                            const ReadOnlyTensor &input, const ReadOnlyTensor &residual);
  // backward(grad_output) + grad_residual; grad_residual has the shape and type of the result
  static Tensor backward_with_residual(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                                       const ReadOnlyTensor &grad_output, const ReadOnlyTensor &grad_residual);
};
}  // namespace cs::compute
