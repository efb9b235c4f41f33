// The five ops of the hot path behind the reference's cs::compute / cs::optimizer interface.
// Every task body allocates its outputs with at::empty (libtorch is used for storage, the
// caching allocator and streams only) and enqueues gfx950 kernels through the C ABI of
// libcs_hip_kernels.so on the stream the scheduler made current.  There is no ATen compute
// call on these paths; the init tasks (random / ones / zeros fills) use ATen as the reference does.
#include <ATen/autocast_mode.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <ATen/ops/empty.h>
#include <ATen/ops/add.h>
#include <ATen/ops/empty_like.h>
#include <ATen/ops/normal.h>
#include <ATen/ops/ones.h>
#include <ATen/ops/zeros.h>
#include <ATen/ops/zeros_like.h>
#include <c10/util/Exception.h>

#include <cstring>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <vector>

#include "autocast.h"
#include "compute/cross_entropy.h"
#include "compute/embedding.h"
#include "compute/gelu.h"
#include "compute/layer_norm.h"
#include "compute/utils.h"
#include "cs_hip_kernels.h"
#include "logger.h"
#include "memory/to_torch.h"
#include "optimizer/adamw.h"
#include "tensor_impl.h"
#include "threading/event.h"
#include "threading/scheduler_impl.h"
#include "threading/task_impl.h"

namespace cs {
namespace {
using Priority = Task::Impl::Priority;
constexpr auto kMain = Task::Impl::kMain;
constexpr auto kAssist = Task::Impl::kAssist;
constexpr auto kCompute = Task::Impl::kCompute;

void *current_stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

int dtype_of(const at::ScalarType t) {
  switch (t) {
    case at::kFloat: return CS_F32;
    case at::kDouble: return CS_F64;
    case at::kHalf: return CS_F16;
    case at::kBFloat16: return CS_BF16;
    default: return -1;
  }
}
int itype_of(const at::ScalarType t) {
  switch (t) {
    case at::kInt: return CS_I32;
    case at::kLong: return CS_I64;
    default: return -1;
  }
}
void check(const int rc, const char *what) {
  CS_ASSERT_TRUE(rc == CS_OK, std::string(what) + ": " + cs_hip_error_string(rc));
}
at::Tensor workspace(const size_t bytes, const at::Tensor &like) {
  return at::empty({static_cast<int64_t>(bytes < 256 ? 256 : bytes)}, like.options().dtype(at::kByte));
}
bool autocast_on() { return at::autocast::is_autocast_enabled(at::kCUDA); }
at::Tensor &T(const ReadOnlyTensor &t) { return t.impl()->tensor(); }

// ---- LayerNorm backward: column sums that ride in the next LayerNorm backward launch
//
// A LayerNorm backward launch leaves one fp32 partial row of dgamma and dbeta per workgroup.
// Adding those rows up is 3 us of work that, as a launch of its own, costs the stream more than
// that; the kernels can instead add them up in the first workgroups of the NEXT LayerNorm
// backward launch (cs_layernorm_backward_rows_pending).  A training step runs one backward per
// norm on the main stream, so only the last norm of the step pays for a launch of its own.
//
// Between the two launches the weight and bias gradients are marked (ReadOnlyTensor::Impl::
// deferred): the scheduler settles a marked tensor before any task that lists it as input or
// output, and wait() before the host reads it, with a launch of cs_layernorm_backward_finalize
// on the stream of the backward task.  One record per device is outstanding at a time.
struct LnSums final : ReadOnlyTensor::Impl::Deferred {
  at::Tensor partials, dgamma, dbeta;              // dbeta undefined for a norm without bias
  std::weak_ptr<ReadOnlyTensor::Impl> gw, gb;      // the handles to stamp once the sums are in
  int64_t C = 0;
  int x_dtype = 0, p_dtype = 0, accumulate = 0;
  std::optional<c10::hip::HIPStreamMasqueradingAsCUDA> stream;

  static std::recursive_mutex &mutex() {
    static auto *m = new std::recursive_mutex;
    return *m;
  }
  // the record of the device, if one is outstanding (never destroyed: it holds device memory,
  // which must not be released during static teardown)
  static std::shared_ptr<LnSums> &slot(const int device) {
    static auto *slots = new std::vector<std::shared_ptr<LnSums>>(64);
    CS_ASSERT_TRUE(device >= 0 && device < 64, "device index out of range");
    return (*slots)[static_cast<size_t>(device)];
  }
  // the gradients are no longer waiting for this record
  void detach() {
    for (const auto &w : {gw, gb})
      if (const auto impl = w.lock(); impl && impl->deferred().get() == this) impl->deferred().reset();
    auto &s = slot(stream->device_index());
    if (s.get() == this) s.reset();
  }
  void settle() override {
    std::lock_guard<std::recursive_mutex> lock{mutex()};
    if (!partials.defined()) return;  // folded into a launch or settled already
    const auto keep = slot(stream->device_index());  // detach() may drop the last other owner
    detach();
    c10::hip::HIPGuardMasqueradingAsCUDA device_guard{stream->device_index()};
    c10::hip::HIPStreamGuardMasqueradingAsCUDA stream_guard{*stream};
    check(cs_layernorm_backward_finalize(partials.data_ptr(), partials.size(0), dgamma.data_ptr(),
                                         dbeta.defined() ? dbeta.data_ptr() : nullptr, C, x_dtype, p_dtype, accumulate,
                                         stream->stream()),
          "cs_layernorm_backward_finalize");
    Event stamp;
    stamp.record();
    for (const auto &w : {gw, gb})
      if (const auto impl = w.lock()) {
        impl->priority() = kMain;
        impl->event() = stamp;
      }
    partials = at::Tensor{};
  }
};
}  // namespace

// ============================================================ CrossEntropy
namespace compute {
std::shared_ptr<CrossEntropy::State> CrossEntropy::init(const Scheduler &scheduler, const Options &options) {
  CS_ASSERT_TRUE(options.label_smoothing() == 0.0, "We do not support label_smoothing");
  return std::make_shared<State>(State{{}, {}, {static_cast<int64_t>(options.reduction()), options.ignore_index(),
                                                options.label_smoothing(), options.num_classes()}});
}

Tensor CrossEntropy::forward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                             const ReadOnlyTensor &input, const ReadOnlyTensor &target) {
  struct Body final : Task::Impl {
    State::Args args;
    Body(std::vector<Tensor> out /* grad, loss, total_weight */,
         std::vector<ReadOnlyTensor> in /* weight, input, target */, const State::Args &a)
        : Task::Impl{std::move(out), std::move(in), kMain, kCompute}, args{a} {}
    void operator()() const override {
      // state->forward.weight: nll_loss's per-class weights (src/compute/cross_entropy.cpp:52-55), fp32 for the kernel
      const at::Tensor cw = T(input()[0]).defined() ? T(input()[0]).to(at::kFloat).contiguous() : at::Tensor{};
      const at::Tensor x = T(input()[1]).contiguous();
      const at::Tensor t = T(input()[2]).contiguous();
      TORCH_CHECK(x.dim() == 2, "CrossEntropy expects [N, C] logits");
      TORCH_CHECK(t.scalar_type() == at::kLong && t.numel() == x.size(0), "targets must be int64 [N]");
      const int64_t N = x.size(0), stride = x.size(1);
      const int64_t V = args.num_classes < 0 ? stride : args.num_classes;
      // ATen's policy for the reference's calls: under autocast the gradient is fp32
      const auto g_type = (autocast_on() && x.scalar_type() != at::kDouble) ? at::kFloat : x.scalar_type();
      at::Tensor grad = at::empty(x.sizes(), x.options().dtype(g_type));
      const auto f32 = x.options().dtype(at::kFloat);
      at::Tensor rows = at::empty({N}, f32), loss = at::empty({}, f32), total = at::empty({}, f32);
      at::Tensor ws = workspace(cs_fused_classifier_workspace_bytes(N), x);
      TORCH_CHECK(!cw.defined() || cw.numel() == V, "CrossEntropy: weight must have one entry per class");
      check(cs_fused_classifier_weighted(x.data_ptr(), grad.data_ptr(), t.data_ptr<int64_t>(),
                                         cw.defined() ? cw.data_ptr<float>() : nullptr, rows.data_ptr<float>(),
                                         loss.data_ptr<float>(), total.data_ptr<float>(), ws.data_ptr(), ws.numel(), N,
                                         V, stride, args.ignore_index, static_cast<int>(args.reduction), 1.f,
                                         dtype_of(x.scalar_type()), dtype_of(g_type), current_stream()),
            name());
      if (cw.defined()) intermediate().push_back(cw);
      T(output()[0]) = grad;
      // The reference hands out what nll_loss_forward returns: loss and total weight in the dtype
      // of the log-probabilities (cross_entropy.cpp:57-66), which is 16-bit for 16-bit logits
      // outside autocast.  The kernel sums in fp32; the rounding to that dtype happens once, here.
      const at::Tensor &result = args.reduction == at::Reduction::None ? rows : loss;
      T(output()[1]) = g_type == at::kFloat ? result : result.to(g_type);
      T(output()[2]) = g_type == at::kFloat ? total : total.to(g_type);
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::CrossEntropy::forward"; }
  };
  Tensor loss{}, grad{}, total_weight{};
  state->backward.log_probs = grad;
  state->backward.total_weight = total_weight;
  state->backward.target = target;
  state->backward.loss = loss;
  scheduler.impl()->submit(Task{std::make_shared<Body>(
      std::vector<Tensor>{grad, loss, total_weight},
      std::vector<ReadOnlyTensor>{state->forward.weight, input, target}, state->args)});
  return loss;
}

Tensor CrossEntropy::backward(const Scheduler &scheduler, const std::shared_ptr<State> &state) {
  struct Body final : Task::Impl {
    Body(std::vector<Tensor> out /* grad_input */, std::vector<ReadOnlyTensor> in /* stored gradient */)
        : Task::Impl{std::move(out), std::move(in), kMain, kCompute} {}
    void operator()() const override { T(output()[0]) = T(input()[0]); }
    [[nodiscard]] const char *name() const override { return "cs::compute::CrossEntropy::backward"; }
  };
  Tensor grad_input{};
  scheduler.impl()->submit(Task{std::make_shared<Body>(std::vector<Tensor>{grad_input},
                                                        std::vector<ReadOnlyTensor>{state->backward.log_probs})});
  state->backward.log_probs.reset();
  state->backward.total_weight.reset();
  state->backward.target.reset();
  state->backward.loss.reset();
  return grad_input;
}

// ==================================================================== GeLU
std::shared_ptr<GeLU::State> GeLU::init(const Scheduler &scheduler) { return std::make_shared<State>(); }
std::shared_ptr<GeLU::State> GeLU::init(const Scheduler &scheduler, const Options &options) {
  CS_ASSERT_TRUE(options.approximate() == 0 || options.approximate() == 1, "approximate must be 0 (erf) or 1 (tanh)");
  auto state = std::make_shared<State>();
  state->args.approximate = options.approximate();
  return state;
}

Tensor GeLU::forward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                     const ReadOnlyTensor &input) {
  struct Body final : Task::Impl {
    int mode;
    Body(std::vector<Tensor> out, std::vector<ReadOnlyTensor> in, const int m)
        : Task::Impl{std::move(out), std::move(in), kMain, kCompute}, mode{m} {}
    void operator()() const override {
      const at::Tensor x = T(input()[0]).contiguous();
      at::Tensor y = at::empty_like(x);
      check(cs_gelu_forward(x.data_ptr(), y.data_ptr(), x.numel(), dtype_of(x.scalar_type()), mode, current_stream()),
            name());
      T(output()[0]) = y;
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::GeLU::forward"; }
  };
  Tensor output{};
  state->backward.input = input;
  scheduler.impl()->submit(Task{std::make_shared<Body>(std::vector<Tensor>{output},
                                                        std::vector<ReadOnlyTensor>{input}, state->args.approximate)});
  return output;
}

Tensor GeLU::backward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                      const ReadOnlyTensor &grad_output) {
  struct Body final : Task::Impl {
    int mode;
    Body(std::vector<Tensor> out, std::vector<ReadOnlyTensor> in /* grad_output, input */, const int m)
        : Task::Impl{std::move(out), std::move(in), kMain, kCompute}, mode{m} {}
    void operator()() const override {
      const at::Tensor x = T(input()[1]).contiguous();
      const at::Tensor dy = T(input()[0]).to(x.scalar_type()).contiguous();
      TORCH_CHECK(dy.numel() == x.numel(), "grad_output does not match the saved input");
      at::Tensor dx = at::empty_like(x);
      check(cs_gelu_backward(dy.data_ptr(), x.data_ptr(), dx.data_ptr(), x.numel(), dtype_of(x.scalar_type()), mode,
                             current_stream()),
            name());
      T(output()[0]) = dx;
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::GeLU::backward"; }
  };
  Tensor grad_input{};
  scheduler.impl()->submit(Task{std::make_shared<Body>(
      std::vector<Tensor>{grad_input}, std::vector<ReadOnlyTensor>{grad_output, state->backward.input},
      state->args.approximate)});
  state->backward.input.reset();
  return grad_input;
}

// =============================================================== Embedding
Embedding::State::State(const Forward &forward, const Backward &backward, const Args &args)
    : forward{forward}, backward{backward}, args{args} {}
OrderedDict<std::string, Tensor> Embedding::State::parameters() const {
  OrderedDict<std::string, Tensor> d;
  d.insert("weight", forward.weight);
  return d;
}
OrderedDict<std::string, Tensor> Embedding::State::gradients() const {
  OrderedDict<std::string, Tensor> d;
  d.insert("weight", forward.grad_weight);
  return d;
}
OrderedDict<std::string, module::State::Increment> Embedding::State::increments() const {
  OrderedDict<std::string, Increment> d;
  d.insert("weight", {forward.weight, forward.grad_weight});
  return d;
}
void Embedding::State::zero_grad() { forward.grad_weight = {}; }

std::shared_ptr<Embedding::State> Embedding::init(const Scheduler &scheduler, const Options &options) {
  struct Body final : Task::Impl {
    const Options options;
    Body(std::vector<Tensor> out, const Options &o) : Task::Impl{std::move(out), {}, kMain, kCompute}, options{o} {}
    void operator()() const override {
      T(output()[0]) = at::normal(0, 1, {options.num_embeddings(), options.embedding_dim()}, {}, options.dtype(), {},
                                  options.device(), {});
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::Embedding::init"; }
  };
  int64_t padding_idx = -1;
  if (options.padding_idx().has_value()) {
    const int64_t p = *options.padding_idx();
    // As in the reference (src/compute/embedding.cpp:80-90): a positive index is only checked
    // and a zero one ignored, so State::Args::padding_idx stays -1 for both and that row keeps
    // its gradient; only a negative index is normalised and takes effect in backward.
    if (p > 0) {
      TORCH_CHECK(p < options.num_embeddings(), "Padding_idx must be within num_embeddings");
    } else if (p < 0) {
      TORCH_CHECK(p >= -options.num_embeddings(), "Padding_idx must be within num_embedding");
      padding_idx = options.num_embeddings() + p;
    }
  }
  TORCH_CHECK(!options.max_norm().has_value(), "max_norm is not supported");
  Tensor weight;
  scheduler.impl()->submit(Task{std::make_shared<Body>(std::vector<Tensor>{weight}, options)});
  return std::make_shared<State>(State::Forward{weight}, State::Backward{},
                                 State::Args{options.num_embeddings(), padding_idx, options.max_norm(),
                                             options.norm_type(), options.scale_grad_by_freq(), options.sparse()});
}

Tensor Embedding::forward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                          const ReadOnlyTensor &indices) {
  struct Body final : Task::Impl {
    Body(std::vector<Tensor> out, std::vector<ReadOnlyTensor> in /* weight, indices */)
        : Task::Impl{std::move(out), std::move(in), kMain, kCompute} {}
    void operator()() const override {
      const at::Tensor w = T(input()[0]).contiguous();
      const at::Tensor idx = T(input()[1]).contiguous();
      TORCH_CHECK(itype_of(idx.scalar_type()) >= 0, "indices must be int32 or int64");
      // the reference views the indices as [-1, last] before the gather
      const int64_t last = idx.size(-1);
      at::Tensor out = at::empty({idx.numel() / last, last, w.size(1)}, w.options());
      check(cs_embedding_forward(w.data_ptr(), idx.data_ptr(), out.data_ptr(), idx.numel(), w.size(1), w.size(0),
                                 dtype_of(w.scalar_type()), itype_of(idx.scalar_type()), current_stream()),
            name());
      T(output()[0]) = out;
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::Embedding::forward"; }
  };
  Tensor output{};
  state->backward.indices = indices;
  scheduler.impl()->submit(Task{std::make_shared<Body>(std::vector<Tensor>{output},
                                                        std::vector<ReadOnlyTensor>{state->forward.weight, indices})});
  return output;
}

void Embedding::backward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                         const ReadOnlyTensor &grad_output) {
  struct Body final : Task::Impl {
    State::Args args;
    Body(std::vector<Tensor> out /* grad_weight */, std::vector<ReadOnlyTensor> in /* grad_output, indices */,
         const State::Args &a)
        : Task::Impl{std::move(out), std::move(in), kAssist, kCompute}, args{a} {}
    void operator()() const override {
      // `sparse` would return a sparse tensor (at::embedding_backward's other branch): not built
      CS_ASSERT_TRUE(!args.sparse, "sparse embedding gradients are not supported");
      const at::Tensor dout = T(input()[0]).contiguous();
      const at::Tensor idx = T(input()[1]).contiguous();
      at::Tensor &gw = T(output()[0]);
      const bool accumulate = gw.defined();  // `=` for a fresh gradient, `+=` otherwise
      const int64_t C = dout.size(-1);
      if (!accumulate) gw = at::empty({args.num_weights, C}, dout.options());
      // the kernel adds into the existing gradient with dout's element type and row length
      TORCH_CHECK(gw.scalar_type() == dout.scalar_type() && gw.dim() == 2 && gw.size(0) == args.num_weights &&
                      gw.size(1) == C && gw.is_contiguous(),
                  "Embedding::backward: the existing gradient must be a contiguous [num_embeddings, C] tensor of "
                  "grad_output's dtype");
      at::Tensor ws = workspace(cs_embedding_backward_workspace_bytes(idx.numel(), C, args.num_weights), dout);
      const auto kernel = args.scale_grad_by_freq ? cs_embedding_backward_scaled : cs_embedding_backward;
      check(kernel(dout.data_ptr(), idx.data_ptr(), gw.data_ptr(), ws.data_ptr(), ws.numel(), idx.numel(), C,
                   args.num_weights, args.padding_idx, dtype_of(dout.scalar_type()), itype_of(idx.scalar_type()),
                   accumulate ? 1 : 0, current_stream()),
            name());
      intermediate().push_back(ws);
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::Embedding::backward"; }
  };
  scheduler.impl()->submit(Task{std::make_shared<Body>(std::vector<Tensor>{state->forward.grad_weight},
                                                        std::vector<ReadOnlyTensor>{grad_output, state->backward.indices},
                                                        state->args)});
  state->backward.indices.reset();
}

Tensor Embedding::forward_with_positions(const Scheduler &scheduler, const std::shared_ptr<State> &tokens,
                                         const std::shared_ptr<State> &positions, const ReadOnlyTensor &indices) {
  struct Body final : Task::Impl {
    Body(std::vector<Tensor> out, std::vector<ReadOnlyTensor> in /* wte, wpe, indices */)
        : Task::Impl{std::move(out), std::move(in), kMain, kCompute} {}
    void operator()() const override {
      const at::Tensor wte = T(input()[0]).contiguous(), wpe = T(input()[1]).contiguous();
      const at::Tensor idx = T(input()[2]).contiguous();
      TORCH_CHECK(idx.dim() == 2 && wpe.size(0) >= idx.size(1) && wpe.size(1) == wte.size(1) &&
                      wpe.scalar_type() == wte.scalar_type(),
                  "expects [B, T] indices and a position table of at least T rows");
      at::Tensor out = at::empty({idx.size(0), idx.size(1), wte.size(1)}, wte.options());
      check(cs_embedding_forward_add(wte.data_ptr(), wpe.data_ptr(), idx.data_ptr(), out.data_ptr(), idx.size(0),
                                     idx.size(1), wte.size(1), wte.size(0), dtype_of(wte.scalar_type()),
                                     itype_of(idx.scalar_type()), current_stream()),
            name());
      T(output()[0]) = out;
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::Embedding::forward_with_positions"; }
  };
  Tensor output{};
  tokens->backward.indices = indices;
  scheduler.impl()->submit(Task{std::make_shared<Body>(
      std::vector<Tensor>{output},
      std::vector<ReadOnlyTensor>{tokens->forward.weight, positions->forward.weight, indices})});
  return output;
}

void Embedding::backward_with_positions(const Scheduler &scheduler, const std::shared_ptr<State> &tokens,
                                        const std::shared_ptr<State> &positions,
                                        const ReadOnlyTensor &grad_output) {
  struct Body final : Task::Impl {
    int64_t num_weights;
    Body(std::vector<Tensor> out /* dwte, dwpe */, std::vector<ReadOnlyTensor> in /* grad_output, indices */,
         const int64_t n)
        : Task::Impl{std::move(out), std::move(in), kAssist, kCompute}, num_weights{n} {}
    void operator()() const override {
      const at::Tensor dout = T(input()[0]).contiguous();
      const at::Tensor idx = T(input()[1]).contiguous();
      at::Tensor &dwte = T(output()[0]), &dwpe = T(output()[1]);
      CS_ASSERT_TRUE(dwte.defined() == dwpe.defined(), "token and position gradients must be accumulated together");
      const bool accumulate = dwte.defined();
      const int64_t B = dout.size(0), Tn = dout.size(1), C = dout.size(2);
      if (!accumulate) {
        dwte = at::empty({num_weights, C}, dout.options());
        dwpe = at::empty({Tn, C}, dout.options());
      }
      at::Tensor ws = workspace(cs_embedding_backward_workspace_bytes(B * Tn, C, num_weights), dout);
      check(cs_embedding_backward_fused(dout.data_ptr(), idx.data_ptr(), dwte.data_ptr(), dwpe.data_ptr(), ws.data_ptr(),
                                        ws.numel(), B, Tn, C, num_weights, dtype_of(dout.scalar_type()),
                                        itype_of(idx.scalar_type()), accumulate ? 1 : 0, current_stream()),
            name());
      intermediate().push_back(ws);
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::Embedding::backward_with_positions"; }
  };
  scheduler.impl()->submit(Task{std::make_shared<Body>(
      std::vector<Tensor>{tokens->forward.grad_weight, positions->forward.grad_weight},
      std::vector<ReadOnlyTensor>{grad_output, tokens->backward.indices}, tokens->args.num_weights)});
  tokens->backward.indices.reset();
}

// =============================================================== LayerNorm
LayerNorm::State::State(const Forward &forward, const Backward &backward, const Args &args)
    : forward{forward}, backward{backward}, args{args} {}
OrderedDict<std::string, Tensor> LayerNorm::State::parameters() const {
  OrderedDict<std::string, Tensor> d;
  d.insert("weight", forward.weight);
  if (args.bias) d.insert("bias", forward.bias);
  return d;
}
OrderedDict<std::string, Tensor> LayerNorm::State::gradients() const {
  OrderedDict<std::string, Tensor> d;
  d.insert("weight", forward.grad_weight);
  if (args.bias) d.insert("bias", forward.grad_bias);
  return d;
}
OrderedDict<std::string, module::State::Increment> LayerNorm::State::increments() const {
  OrderedDict<std::string, Increment> d;
  d.insert("weight", {forward.weight, forward.grad_weight});
  if (args.bias) d.insert("bias", {forward.bias, forward.grad_bias});
  return d;
}
void LayerNorm::State::zero_grad() {
  forward.grad_weight = {};
  if (args.bias) forward.grad_bias = {};
}

std::shared_ptr<LayerNorm::State> LayerNorm::init(const Scheduler &scheduler, const Options &options) {
  CS_ASSERT_TRUE(options.elementwise_affine() == true, "elementwise_affine must be enabled now");
  CS_ASSERT_TRUE(options.normalized_shape().size() == 1, "only the last dimension can be normalised");
  struct Body final : Task::Impl {
    const Options options;
    Body(std::vector<Tensor> out /* weight[, bias] */, const Options &o)
        : Task::Impl{std::move(out), {}, kMain, kCompute}, options{o} {}
    void operator()() const override {
      at::TensorOptions opts{};
      if (options.device().has_value()) opts = opts.device(options.device().value());
      if (options.dtype().has_value()) opts = opts.dtype(options.dtype().value());
      T(output()[0]) = at::ones(options.normalized_shape(), opts);
      if (output().size() > 1) T(output()[1]) = at::zeros(options.normalized_shape(), opts);
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::LayerNorm::init"; }
  };
  Tensor weight, bias;
  std::vector<Tensor> outs{weight};
  if (options.bias()) outs.push_back(bias);
  scheduler.impl()->submit(Task{std::make_shared<Body>(std::move(outs), options)});
  State::Forward fwd{weight};
  if (options.bias()) fwd.bias = bias;
  return std::make_shared<State>(fwd, State::Backward{},
                                 State::Args{options.normalized_shape(), options.eps(), options.elementwise_affine(),
                                             options.bias()});
}

namespace {
// forward and forward_with_residual: the second takes one more input (after the parameters)
// and fills one more output (the sum)
struct LnForwardBody final : Task::Impl {
  double eps;
  bool has_bias, has_residual;
  LnForwardBody(std::vector<Tensor> out /* y, mean, rstd[, sum] */,
                std::vector<ReadOnlyTensor> in /* x, weight[, bias][, residual] */, const double e, const bool b,
                const bool r)
      : Task::Impl{std::move(out), std::move(in), kMain, kCompute}, eps{e}, has_bias{b}, has_residual{r} {}
  void operator()() const override {
    const at::Tensor x = T(input()[0]).contiguous();
    const at::Tensor g = T(input()[1]).contiguous();
    const at::Tensor b = has_bias ? T(input()[2]).contiguous() : at::Tensor{};
    const int64_t C = x.size(-1), rows = x.numel() / C;
    TORCH_CHECK(g.numel() == C, "weight does not match the normalised dimension");
    // native_layer_norm is on ATen's fp32 autocast list: y is fp32 under autocast
    const auto y_type = (autocast_on() && x.scalar_type() != at::kDouble) ? at::kFloat : x.scalar_type();
    const auto stat_type = x.scalar_type() == at::kDouble ? at::kDouble : at::kFloat;
    at::Tensor y = at::empty(x.sizes(), x.options().dtype(y_type));
    auto stat_sizes = x.sizes().vec();
    stat_sizes.back() = 1;
    at::Tensor mean = at::empty(stat_sizes, x.options().dtype(stat_type));
    at::Tensor rstd = at::empty(stat_sizes, x.options().dtype(stat_type));
    if (has_residual) {
      at::Tensor res = T(input().back()).contiguous();
      TORCH_CHECK(res.sizes() == x.sizes(), "residual must have the input's shape");
      if (res.scalar_type() != x.scalar_type()) res = res.to(x.scalar_type());
      at::Tensor sum = at::empty_like(x);
      check(cs_add_layernorm_forward(x.data_ptr(), res.data_ptr(), sum.data_ptr(), g.data_ptr(),
                                     has_bias ? b.data_ptr() : nullptr, y.data_ptr(), mean.data_ptr(), rstd.data_ptr(),
                                     rows, C, eps, dtype_of(x.scalar_type()), dtype_of(y_type),
                                     dtype_of(g.scalar_type()), current_stream()),
            name());
      T(output()[3]) = sum;
    } else {
      check(cs_layernorm_forward(x.data_ptr(), g.data_ptr(), has_bias ? b.data_ptr() : nullptr, y.data_ptr(),
                                 mean.data_ptr(), rstd.data_ptr(), rows, C, eps, dtype_of(x.scalar_type()),
                                 dtype_of(y_type), dtype_of(g.scalar_type()), current_stream()),
            name());
    }
    T(output()[0]) = y;
    T(output()[1]) = mean;
    T(output()[2]) = rstd;
  }
  [[nodiscard]] const char *name() const override {
    return has_residual ? "cs::compute::LayerNorm::forward_with_residual" : "cs::compute::LayerNorm::forward";
  }
};
}  // namespace

Tensor LayerNorm::forward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                          const ReadOnlyTensor &input) {
  Tensor output, mean, rstd;
  std::vector<ReadOnlyTensor> ins{input, state->forward.weight};
  if (state->args.bias) ins.push_back(state->forward.bias);
  state->backward.input = input;
  state->backward.mean = mean;
  state->backward.rstd = rstd;
  scheduler.impl()->submit(Task{std::make_shared<LnForwardBody>(std::vector<Tensor>{output, mean, rstd}, std::move(ins),
                                                                 state->args.eps, state->args.bias, false)});
  return output;
}

LayerNorm::WithResidual LayerNorm::forward_with_residual(const Scheduler &scheduler,
                                                         const std::shared_ptr<State> &state,
                                                         const ReadOnlyTensor &input,
                                                         const ReadOnlyTensor &residual) {
  Tensor output, mean, rstd, sum;
  std::vector<ReadOnlyTensor> ins{input, state->forward.weight};
  if (state->args.bias) ins.push_back(state->forward.bias);
  ins.push_back(residual);
  state->backward.input = sum;  // the norm's input is the sum
  state->backward.mean = mean;
  state->backward.rstd = rstd;
  scheduler.impl()->submit(Task{std::make_shared<LnForwardBody>(std::vector<Tensor>{output, mean, rstd, sum},
                                                                 std::move(ins), state->args.eps, state->args.bias,
                                                                 true)});
  return {output, sum};
}

namespace {
// One task on the main stream.  The reference submits two (parameter gradients on the assist
// stream, src/compute/layer_norm.cpp:228-233), and the kernels can be called that way
// (cs_layernorm_backward_rows / _finalize), but the second kernel is 4 us of work, while making
// the main stream wait for another stream's event costs it 7 us on this part: at [8192, 768]
// the main stream is busy 13.9 us per call with one task and 18.8 us with two.  Where the shape
// allows, the task launches the row pass only and the column sums ride in the next LayerNorm
// backward launch of the stream (LnSums above): 11.3 us per call.
struct LnBackwardBody final : Task::Impl {
  bool has_bias, has_residual;
  LnBackwardBody(std::vector<Tensor> out /* dx, grad_weight[, grad_bias] */,
                 std::vector<ReadOnlyTensor> in /* grad_output, x, mean, rstd, weight[, grad_residual] */,
                 const bool b, const bool r)
      : Task::Impl{std::move(out), std::move(in), kMain, kCompute}, has_bias{b}, has_residual{r} {}
  void operator()() const override {
    const at::Tensor x = T(input()[1]).contiguous();
    at::Tensor dy = T(input()[0]).contiguous();
    const at::Tensor mean = T(input()[2]), rstd = T(input()[3]);
    const at::Tensor g = T(input()[4]).contiguous();
    // dy is either x's type or fp32 (autocast over 16-bit x); anything else is brought to x's type
    const bool narrow_x = x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16;
    if (dy.scalar_type() != x.scalar_type() && !(narrow_x && dy.scalar_type() == at::kFloat))
      dy = dy.to(x.scalar_type());
    const int64_t C = x.size(-1), rows = x.numel() / C;
    at::Tensor dx = at::empty(x.sizes(), x.options().dtype(dy.scalar_type()));
    // backward_with_residual: the gradient that flows past the norm is added to dx in the same pass
    at::Tensor dres;
    if (has_residual) {
      dres = T(input()[5]).contiguous();
      TORCH_CHECK(dres.sizes() == x.sizes(), "grad_residual must have the input's shape");
      if (dres.scalar_type() != dx.scalar_type()) dres = dres.to(dx.scalar_type());
    }
    at::Tensor &gw = T(output()[1]);
    at::Tensor *gb = has_bias ? &T(output()[2]) : nullptr;
    const bool accumulate = gw.defined();  // += into gradients that already exist
    if (has_bias) CS_ASSERT_TRUE(gb->defined() == accumulate, "weight and bias gradients must exist together");
    // fp32 dy with 16-bit parameters (autocast over a model whose LayerNorm weights are 16 bit):
    // the kernels take fp32 parameters with fp32 dy, so gamma is widened and the parameter
    // gradients come out in fp32 and are narrowed (or added) afterwards, [C] elements each
    const bool widen = dy.scalar_type() == at::kFloat && g.scalar_type() != at::kFloat && narrow_x;
    const at::Tensor gk = widen ? g.to(at::kFloat) : g;
    at::Tensor dgk, dbk;
    if (widen || !accumulate) {
      // an empty batch leaves the gradients untouched: they are zero then
      dgk = rows == 0 ? at::zeros({C}, gk.options()) : at::empty({C}, gk.options());
      if (has_bias) dbk = rows == 0 ? at::zeros({C}, gk.options()) : at::empty({C}, gk.options());
    } else {
      dgk = gw;
      if (has_bias) dbk = *gb;
    }
    const bool kernel_accumulates = accumulate && !widen;
    if (!widen && rows > 0 && chained(dy, x, mean, rstd, gk, dres, dx, dgk, dbk, kernel_accumulates, rows, C)) {
      if (!accumulate) {
        gw = dgk;
        if (has_bias) *gb = dbk;
      }
      T(output()[0]) = dx;
      return;
    }
    at::Tensor ws = workspace(cs_layernorm_backward_workspace_bytes(rows, C), x);
    if (has_residual && rows > 0) {
      check(cs_layernorm_backward_add(dy.data_ptr(), x.data_ptr(), mean.data_ptr(), rstd.data_ptr(), gk.data_ptr(),
                                      dres.data_ptr(), dx.data_ptr(), dgk.data_ptr(),
                                      has_bias ? dbk.data_ptr() : nullptr, ws.data_ptr(), ws.numel(), rows, C,
                                      dtype_of(dy.scalar_type()), dtype_of(x.scalar_type()),
                                      dtype_of(dx.scalar_type()), dtype_of(gk.scalar_type()),
                                      kernel_accumulates ? 1 : 0, current_stream()),
            name());
    } else {
      check(cs_layernorm_backward(dy.data_ptr(), x.data_ptr(), mean.data_ptr(), rstd.data_ptr(), gk.data_ptr(),
                                  dx.data_ptr(), dgk.data_ptr(), has_bias ? dbk.data_ptr() : nullptr, ws.data_ptr(),
                                  ws.numel(), rows, C, dtype_of(dy.scalar_type()), dtype_of(x.scalar_type()),
                                  dtype_of(dx.scalar_type()), dtype_of(gk.scalar_type()), kernel_accumulates ? 1 : 0,
                                  current_stream()),
            name());
    }
    if (widen) {
      gw = accumulate ? gw + dgk.to(g.scalar_type()) : dgk.to(g.scalar_type());
      if (has_bias) *gb = accumulate ? *gb + dbk.to(g.scalar_type()) : dbk.to(g.scalar_type());
    } else if (!accumulate) {
      gw = dgk;
      if (has_bias) *gb = dbk;
    }
    T(output()[0]) = dx;
  }
  // The row pass alone, with the column sums of the previous LayerNorm backward of this stream
  // added up in the same launch; this call's own sums stay partial rows until the next backward
  // or until somebody needs the gradients.  False when the shape has no such form.
  bool chained(const at::Tensor &dy, const at::Tensor &x, const at::Tensor &mean, const at::Tensor &rstd,
               const at::Tensor &g, const at::Tensor &dres, const at::Tensor &dx, const at::Tensor &dg,
               const at::Tensor &db, const bool kernel_accumulates, const int64_t rows, const int64_t C) const {
    const int xt = dtype_of(x.scalar_type()), pt = dtype_of(g.scalar_type());
    const int64_t n = cs_layernorm_backward_partial_rows(rows, C, xt);
    if (n <= 0) return false;
    for (const at::Tensor *t : {&dy, &x, &g, &dx, &dres})
      if (t->defined() && reinterpret_cast<uintptr_t>(t->data_ptr()) % 16 != 0) return false;
    std::lock_guard<std::recursive_mutex> lock{LnSums::mutex()};
    const auto here = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    std::shared_ptr<LnSums> prev = LnSums::slot(here.device_index());
    if (prev && !(*prev->stream == here && prev->C == C && prev->x_dtype == xt && prev->p_dtype == pt)) {
      prev->settle();  // another stream, width or type: its sums cannot ride in this launch
      prev.reset();
    }
    at::Tensor partials = at::empty({n, 2, C}, x.options().dtype(at::kFloat));
    check(cs_layernorm_backward_rows_pending(
              dy.data_ptr(), x.data_ptr(), mean.data_ptr(), rstd.data_ptr(), g.data_ptr(),
              dres.defined() ? dres.data_ptr() : nullptr, dx.data_ptr(), partials.data_ptr(), static_cast<size_t>(partials.numel()) * 4,
              prev ? prev->partials.data_ptr() : nullptr, prev ? prev->partials.size(0) : 0,
              prev ? prev->dgamma.data_ptr() : nullptr,
              prev && prev->dbeta.defined() ? prev->dbeta.data_ptr() : nullptr, prev ? prev->accumulate : 0, rows, C,
              dtype_of(dy.scalar_type()), xt, dtype_of(dx.scalar_type()), pt, here.stream()),
          name());
    if (prev) {
      // its gradients are complete with this task: the scheduler stamps them with its event
      for (const auto &w : {prev->gw, prev->gb})
        if (const auto impl = w.lock()) completed().push_back(impl);
      prev->detach();
      prev->partials = at::Tensor{};
    }
    auto mine = std::make_shared<LnSums>();
    mine->partials = partials;
    mine->dgamma = dg;
    if (has_bias) mine->dbeta = db;
    mine->gw = output()[1].impl();
    if (has_bias) mine->gb = output()[2].impl();
    mine->C = C;
    mine->x_dtype = xt;
    mine->p_dtype = pt;
    mine->accumulate = kernel_accumulates ? 1 : 0;
    mine->stream = here;
    output()[1].impl()->deferred() = mine;
    if (has_bias) output()[2].impl()->deferred() = mine;
    LnSums::slot(here.device_index()) = mine;
    return true;
  }
  [[nodiscard]] const char *name() const override {
    return has_residual ? "cs::compute::LayerNorm::backward_with_residual" : "cs::compute::LayerNorm::backward";
  }
};
}  // namespace

namespace {
Tensor ln_backward(const Scheduler &scheduler, const std::shared_ptr<LayerNorm::State> &state,
                   const ReadOnlyTensor &grad_output, const ReadOnlyTensor *grad_residual) {
  Tensor grad_input;
  std::vector<Tensor> outs{grad_input, state->forward.grad_weight};
  if (state->args.bias) outs.push_back(state->forward.grad_bias);
  std::vector<ReadOnlyTensor> ins{grad_output, state->backward.input, state->backward.mean, state->backward.rstd,
                                  state->forward.weight};
  if (grad_residual != nullptr) ins.push_back(*grad_residual);
  scheduler.impl()->submit(Task{
      std::make_shared<LnBackwardBody>(std::move(outs), std::move(ins), state->args.bias, grad_residual != nullptr)});
  state->backward.input.reset();
  state->backward.mean.reset();
  state->backward.rstd.reset();
  return grad_input;
}
}  // namespace

Tensor LayerNorm::backward(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                           const ReadOnlyTensor &grad_output) {
  return ln_backward(scheduler, state, grad_output, nullptr);
}

Tensor LayerNorm::backward_with_residual(const Scheduler &scheduler, const std::shared_ptr<State> &state,
                                         const ReadOnlyTensor &grad_output, const ReadOnlyTensor &grad_residual) {
  return ln_backward(scheduler, state, grad_output, &grad_residual);
}
}  // namespace compute

namespace {
// Lays the descriptor table out in pinned host memory and copies it to the device on the
// current stream; libtorch keeps the pinned block alive until the copy has run.
//
// A training loop hands the same tensors to the optimizer step after step (the allocator gives
// each step's gradients the addresses of the last step's), so the table usually comes out byte
// for byte as it did before.  The last few tables are kept, with their device copies, per
// stream: a table that is found there is not copied again (the copy is 3 us, but it sits
// between two kernels of the stream and cost 17 us of idle time around it in a GPT-2-small
// step).  The copy that filled the device block ran earlier on the same stream, so stream order
// covers the reuse.
at::Tensor upload_table(const std::vector<cs_adamw_tensor> &descs, const int dtype, const at::TensorOptions &like,
                        int64_t *slots, const char *who) {
  struct Kept {
    std::vector<uint8_t> bytes;
    at::Tensor device;
    c10::StreamId stream;
    c10::DeviceIndex device_index;
    uint64_t used;
  };
  constexpr size_t kKept = 8;
  static auto *kept = new std::vector<Kept>;  // never destroyed: holds device memory
  static auto *mutex = new std::mutex;
  static uint64_t clock = 0;

  const size_t bytes = cs_adamw_multi_table_bytes(static_cast<int64_t>(descs.size()));
  at::Tensor host = at::empty({static_cast<int64_t>(bytes)}, at::TensorOptions().dtype(at::kByte).pinned_memory(true));
  check(cs_adamw_multi_build_table(descs.data(), static_cast<int64_t>(descs.size()), dtype, host.data_ptr(), bytes,
                                   slots),
        who);
  const auto here = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
  const auto *fresh = static_cast<const uint8_t *>(host.data_ptr());
  std::lock_guard<std::mutex> lock{*mutex};
  for (auto &k : *kept) {
    if (k.stream == here.id() && k.device_index == here.device_index() && k.bytes.size() == bytes &&
        std::memcmp(k.bytes.data(), fresh, bytes) == 0) {
      k.used = ++clock;
      return k.device;
    }
  }
  at::Tensor table = at::empty({static_cast<int64_t>(bytes)}, like.dtype(at::kByte));
  table.copy_(host, /*non_blocking=*/true);
  Kept entry{std::vector<uint8_t>(fresh, fresh + bytes), table, here.id(), here.device_index(), ++clock};
  if (kept->size() < kKept) {
    kept->push_back(std::move(entry));
  } else {
    auto oldest = kept->begin();
    for (auto it = kept->begin(); it != kept->end(); ++it)
      if (it->used < oldest->used) oldest = it;
    *oldest = std::move(entry);
  }
  return table;
}
}  // namespace

// =================================================================== Utils
namespace compute::Utils {
Tensor clip_grad_norm_(const Scheduler &scheduler, const std::vector<Tensor> &tensor, const double max_norm,
                       const double norm_type) {
  struct Body final : Task::Impl {
    double max_norm, norm_type;
    Body(std::vector<Tensor> out /* gradients..., total_norm */, std::vector<ReadOnlyTensor> in /* gradients */,
         const double max_norm, const double norm_type)
        : Task::Impl{std::move(out), std::move(in), kMain, kCompute}, max_norm{max_norm}, norm_type{norm_type} {}
    void operator()() const override {
      // the gradient table of the optimizer step, with the gradient standing in for the other pointers
      std::vector<cs_adamw_tensor> descs;
      int dtype = -1;
      at::TensorOptions like;
      for (const auto &in : input()) {
        const at::Tensor &g = T(in);
        if (!g.defined()) continue;
        TORCH_CHECK(g.is_contiguous(), "clip_grad_norm_ needs contiguous gradients");
        const int dt = dtype_of(g.scalar_type());
        CS_ASSERT_TRUE(dtype < 0 || dt == dtype, "clip_grad_norm_ needs one dtype");
        dtype = dt;
        like = g.options();
        descs.push_back({g.data_ptr(), g.data_ptr(), g.data_ptr(), g.data_ptr(), nullptr, g.numel()});
      }
      if (descs.empty()) return;
      int64_t slots = 0;
      at::Tensor table = upload_table(descs, dtype, like, &slots, name());
      const auto count = static_cast<int64_t>(descs.size());
      at::Tensor norm = at::empty({}, like.dtype(at::kFloat)), coef = at::empty({}, like.dtype(at::kFloat));
      const size_t ws_bytes = cs_grad_norm_multi_workspace_bytes(slots);
      at::Tensor ws = at::empty({static_cast<int64_t>(ws_bytes)}, like.dtype(at::kByte));
      check(cs_grad_norm_multi(table.data_ptr(), count, slots, dtype, norm_type, max_norm, ws.data_ptr(), ws_bytes,
                               norm.data_ptr<float>(), coef.data_ptr<float>(), current_stream()),
            name());
      check(cs_grad_scale_multi(table.data_ptr(), count, slots, dtype, coef.data_ptr<float>(), current_stream()), name());
      T(output().back()) = norm;
      intermediate().push_back(table);
      intermediate().push_back(ws);
      intermediate().push_back(coef);
    }
    [[nodiscard]] const char *name() const override { return "cs::compute::Utils::clip_grad_norm_"; }
  };
  Tensor total_norm;
  std::vector<Tensor> outs{tensor};
  outs.push_back(total_norm);
  scheduler.impl()->submit(Task{std::make_shared<Body>(
      std::move(outs), std::vector<ReadOnlyTensor>{tensor.begin(), tensor.end()}, max_norm, norm_type)});
  return total_norm;
}
}  // namespace compute::Utils

// =================================================================== AdamW
namespace optimizer {
namespace {
// The kernels take one element type and one count for the parameter, its gradient and its state
// (the reference's data_ptr<T>() throws on a mismatch, src/optimizer/adamw.cu:96-103).
void check_adamw_tensors(const at::Tensor &g, const at::Tensor &w, const at::Tensor &m, const at::Tensor &v,
                         const at::Tensor *v_max) {
  const auto same = [&](const at::Tensor &t) { return t.scalar_type() == g.scalar_type() && t.numel() == g.numel(); };
  TORCH_CHECK(same(w) && same(m) && same(v) && (v_max == nullptr || same(*v_max)),
              "AdamW: the parameter, its gradient and its state must share one dtype and element count (gradient ",
              g.scalar_type(), " x ", g.numel(), ", parameter ", w.scalar_type(), " x ", w.numel(), ")");
}
}  // namespace

AdamW::State::State(const Tensors &tensors, const Options &options) : tensors{tensors}, options{options} {}
void AdamW::State::set_lr(const double lr) const { options.lr = lr; }
double AdamW::State::get_lr() const { return options.lr; }

std::shared_ptr<AdamW::State> AdamW::init(const Scheduler &scheduler, const ReadOnlyTensor &parameter,
                                          const Options &options) {
  struct Body final : Task::Impl {
    Body(std::vector<Tensor> out /* m, v[, v_max] */, std::vector<ReadOnlyTensor> in /* parameter */)
        : Task::Impl{std::move(out), std::move(in), kAssist, kCompute} {}
    void operator()() const override {
      for (const auto &o : output()) T(o) = at::zeros_like(T(input()[0]));
    }
    [[nodiscard]] const char *name() const override { return "cs::optimizer::AdamW::init"; }
  };
  Tensor m, v, v_max;
  std::vector<Tensor> outs{m, v};
  if (options.amsgrad()) outs.push_back(v_max);
  scheduler.impl()->submit(Task{std::make_shared<Body>(std::move(outs), std::vector<ReadOnlyTensor>{parameter})});
  State::Tensors tensors{m, v};
  if (options.amsgrad()) tensors.v_max = v_max;
  return std::make_shared<State>(tensors, State::Options{options.lr(), options.beta1(), options.beta2(), options.eps(),
                                                         options.weight_decay(), options.amsgrad(), options.t()});
}

void AdamW::step(const Scheduler &scheduler, const std::shared_ptr<module::OptimizerState> &state, const Tensor &w,
                 const ReadOnlyTensor &dw) {
  struct Body final : Task::Impl {
    State::Options options;  // by value: lr and t are those of submit time
    Body(std::vector<Tensor> out /* w, m, v[, v_max] */, std::vector<ReadOnlyTensor> in /* dw */,
         const State::Options &o)
        : Task::Impl{std::move(out), std::move(in), kAssist, kCompute}, options{o} {}
    void operator()() const override {
      const at::Tensor &g = T(input()[0]);
      if (!g.defined()) {
        CS_WARN_TRUE(false, "got non-defined gradient, skip the update");
        return;
      }
      at::Tensor &w = T(output()[0]), &m = T(output()[1]), &v = T(output()[2]);
      TORCH_CHECK(w.is_contiguous() && m.is_contiguous() && v.is_contiguous(), "AdamW needs contiguous state");
      check_adamw_tensors(g, w, m, v, options.amsgrad ? &T(output()[3]) : nullptr);
      const at::Tensor gc = g.contiguous();
      check(cs_adamw_step(w.data_ptr(), gc.data_ptr(), m.data_ptr(), v.data_ptr(),
                          options.amsgrad ? T(output()[3]).data_ptr() : nullptr, gc.numel(),
                          dtype_of(gc.scalar_type()), options.lr, options.beta1, options.beta2, options.eps,
                          options.weight_decay, options.t, current_stream()),
            name());
      if (!gc.is_same(g)) intermediate().push_back(gc);
    }
    [[nodiscard]] const char *name() const override { return "cs::optimizer::AdamW::step"; }
  };
  const auto s = std::dynamic_pointer_cast<State>(state);
  CS_ASSERT_TRUE(s != nullptr, "AdamW::step needs an AdamW state");
  s->options.t++;
  std::vector<Tensor> outs{w, s->tensors.m, s->tensors.v};
  if (s->options.amsgrad) outs.push_back(s->tensors.v_max);
  scheduler.impl()->submit(Task{std::make_shared<Body>(std::move(outs), std::vector<ReadOnlyTensor>{dw}, s->options)});
}

void AdamW::step(const Scheduler &scheduler, const std::vector<std::shared_ptr<module::OptimizerState>> &states,
                 const std::vector<Tensor> &ws, const std::vector<ReadOnlyTensor> &dws) {
  (void)step(scheduler, states, ws, dws, c10::nullopt, 2.0);
}

Tensor AdamW::step(const Scheduler &scheduler, const std::vector<std::shared_ptr<module::OptimizerState>> &states,
                   const std::vector<Tensor> &ws, const std::vector<ReadOnlyTensor> &dws,
                   const c10::optional<double> max_grad_norm, const double norm_type) {
  CS_ASSERT_TRUE(states.size() == ws.size() && ws.size() == dws.size(), "one state and one gradient per parameter");
  Tensor total_norm;
  if (states.empty()) return total_norm;
  struct Body final : Task::Impl {
    State::Options options;
    size_t n;
    c10::optional<double> max_norm;
    double norm_type;
    Body(std::vector<Tensor> out /* n x (w, m, v, v_max), total_norm */, std::vector<ReadOnlyTensor> in /* n x dw */,
         const State::Options &o, const size_t count, const c10::optional<double> max_norm, const double norm_type)
        : Task::Impl{std::move(out), std::move(in), kAssist, kCompute},
          options{o},
          n{count},
          max_norm{max_norm},
          norm_type{norm_type} {}
    void operator()() const override {
      std::vector<cs_adamw_tensor> descs;
      descs.reserve(n);
      int dtype = -1;
      at::TensorOptions like;
      for (size_t i = 0; i < n; ++i) {
        const at::Tensor &g = T(input()[i]);
        if (!g.defined()) {
          CS_WARN_TRUE(false, "got non-defined gradient, skip the update");
          continue;
        }
        at::Tensor &w = T(output()[4 * i]), &m = T(output()[4 * i + 1]), &v = T(output()[4 * i + 2]);
        TORCH_CHECK(g.is_contiguous() && w.is_contiguous() && m.is_contiguous() && v.is_contiguous(),
                    "multi-tensor AdamW needs contiguous tensors");
        check_adamw_tensors(g, w, m, v, options.amsgrad ? &T(output()[4 * i + 3]) : nullptr);
        const int dt = dtype_of(g.scalar_type());
        CS_ASSERT_TRUE(dtype < 0 || dt == dtype, "multi-tensor AdamW needs one dtype");
        dtype = dt;
        like = g.options();
        descs.push_back({w.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(),
                         options.amsgrad ? T(output()[4 * i + 3]).data_ptr() : nullptr, g.numel()});
      }
      if (descs.empty()) return;
      int64_t slots = 0;
      at::Tensor table = upload_table(descs, dtype, like, &slots, name());
      const auto count = static_cast<int64_t>(descs.size());
      if (max_norm.has_value()) {
        // global norm first (two small launches), then the step scales each gradient as it reads it
        at::Tensor norm = at::empty({}, like.dtype(at::kFloat)), coef = at::empty({}, like.dtype(at::kFloat));
        const size_t ws_bytes = cs_grad_norm_multi_workspace_bytes(slots);
        at::Tensor ws = at::empty({static_cast<int64_t>(ws_bytes)}, like.dtype(at::kByte));
        check(cs_grad_norm_multi(table.data_ptr(), count, slots, dtype, norm_type, *max_norm, ws.data_ptr(), ws_bytes,
                                 norm.data_ptr<float>(), coef.data_ptr<float>(), current_stream()),
              name());
        check(cs_adamw_multi_step_clipped(table.data_ptr(), count, slots, dtype, options.amsgrad ? 1 : 0, options.lr,
                                          options.beta1, options.beta2, options.eps, options.weight_decay, options.t,
                                          coef.data_ptr<float>(), current_stream()),
              name());
        T(output().back()) = norm;
        intermediate().push_back(ws);
        intermediate().push_back(coef);
      } else {
        check(cs_adamw_multi_step(table.data_ptr(), count, slots, dtype, options.amsgrad ? 1 : 0, options.lr,
                                  options.beta1, options.beta2, options.eps, options.weight_decay, options.t,
                                  current_stream()),
              name());
      }
      intermediate().push_back(table);
    }
    [[nodiscard]] const char *name() const override { return "cs::optimizer::AdamW::step(all)"; }
  };
  std::vector<Tensor> outs;
  std::vector<ReadOnlyTensor> ins;
  std::optional<State::Options> first;  // the options have const members: no assignment
  for (size_t i = 0; i < states.size(); ++i) {
    const auto s = std::dynamic_pointer_cast<State>(states[i]);
    CS_ASSERT_TRUE(s != nullptr, "AdamW::step needs AdamW states");
    s->options.t++;
    if (!first.has_value()) {
      first.emplace(s->options);
    } else {
      CS_ASSERT_TRUE(s->options.t == first->t && s->options.lr == first->lr && s->options.beta1 == first->beta1 &&
                         s->options.beta2 == first->beta2 && s->options.eps == first->eps &&
                         s->options.weight_decay == first->weight_decay && s->options.amsgrad == first->amsgrad,
                     "multi-tensor AdamW needs the same hyper-parameters and step count for every parameter");
    }
    outs.push_back(ws[i]);
    outs.push_back(s->tensors.m);
    outs.push_back(s->tensors.v);
    outs.push_back(s->tensors.v_max);
    ins.push_back(dws[i]);
  }
  outs.push_back(total_norm);
  scheduler.impl()->submit(
      Task{std::make_shared<Body>(std::move(outs), std::move(ins), *first, states.size(), max_grad_norm, norm_type)});
  return total_norm;
}
}  // namespace optimizer

// ================================================================== memory
namespace memory {
at::Tensor to_torch(const Scheduler &scheduler, const ReadOnlyTensor &tensor) {
  tensor.wait();  // the producing task has run
  if (!T(tensor).defined()) return {};
  at::Tensor copy = T(tensor).clone();
  c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().synchronize();
  return copy;
}

Tensor from_torch(const Scheduler &scheduler, const at::Tensor &tensor) {
  Tensor handle;
  handle.impl()->tensor() = tensor;
  // whoever produced `tensor` did so on the caller's current stream: stamp the handle with an
  // event there and with a priority no scheduler stream has, so every consumer waits for it
  handle.impl()->priority() = Task::Impl::kNumPriority;
  if (tensor.defined() && tensor.is_cuda()) handle.impl()->event().record();
  return handle;
}
}  // namespace memory

// ================================================================ autocast
namespace autocast {
ContextGuard::ContextGuard(const Scheduler &scheduler, const at::ScalarType dtype)
    : previous_{at::autocast::is_autocast_enabled(at::kCUDA)},
      previous_dtype_{at::autocast::get_autocast_dtype(at::kCUDA)} {
  at::autocast::set_autocast_enabled(at::kCUDA, true);
  at::autocast::set_autocast_dtype(at::kCUDA, dtype);
}
ContextGuard::~ContextGuard() {
  at::autocast::set_autocast_enabled(at::kCUDA, previous_);
  at::autocast::set_autocast_dtype(at::kCUDA, previous_dtype_);
}
}  // namespace autocast
}  // namespace cs
