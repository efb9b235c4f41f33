// Module tree, optimizer module and the Embedding / LayerNorm / AdamW modules over the
// cs::compute and cs::optimizer ops.
#include <map>
#include <tuple>
#include <vector>

#include "logger.h"
#include "module/adamw.h"
#include "module/embedding.h"
#include "module/layer_norm.h"
#include "module/module.h"
#include "module/optimizer_module.h"
#include "tensor_impl.h"

namespace cs::module {
namespace {
std::string join(const std::string &prefix, const std::string &name) {
  return prefix.empty() ? name : prefix + "." + name;
}
}  // namespace

// ------------------------------------------------------------------ Module
void Module::apply_to_submodules(const NamedModulePointerApplyFunction &function, const std::string &name_prefix,
                                 const std::size_t depth) const {
  for (const auto &child : children_) {
    const std::string qualified = depth == 0 ? child.key() : join(name_prefix, child.key());
    function(qualified, child.value());
    child.value()->apply_to_submodules(function, qualified, depth + 1);
  }
}

void Module::apply(const ConstNamedModuleApplyFunction &function, const std::string &name_prefix) const {
  function(name_prefix, *this);
  apply_to_submodules(
      [&function](const std::string &name, const std::shared_ptr<Module> &module) { function(name, *module); },
      name_prefix);
}

void Module::register_state(std::shared_ptr<State> state) {
  CS_ASSERT_TRUE(state_ == nullptr, "one module can only register state once");
  state_ = std::move(state);
}

OrderedDict<std::string, std::shared_ptr<State>> Module::named_states() const {
  OrderedDict<std::string, std::shared_ptr<State>> result;
  apply([&result](const std::string &name, const Module &module) {
    if (module.state_ != nullptr) result.insert(name, module.state_);
  });
  return result;
}

OrderedDict<std::string, Tensor> Module::named_parameters(const bool) const {
  OrderedDict<std::string, Tensor> result;
  for (const auto &state : named_states())
    for (const auto &parameter : state.value()->parameters())
      result.insert(join(state.key(), parameter.key()), parameter.value());
  return result;
}

OrderedDict<std::string, Tensor> Module::named_gradients(const bool) const {
  OrderedDict<std::string, Tensor> result;
  for (const auto &state : named_states())
    for (const auto &gradient : state.value()->gradients())
      result.insert(join(state.key(), gradient.key()), gradient.value());
  return result;
}

OrderedDict<std::string, State::Increment> Module::named_increments(const bool) const {
  OrderedDict<std::string, State::Increment> result;
  for (const auto &state : named_states())
    for (const auto &increment : state.value()->increments())
      result.insert(join(state.key(), increment.key()), increment.value());
  return result;
}

void Module::zero_grad() const {
  for (const auto &state : named_states()) state.value()->zero_grad();
}

void Module::to(const TensorOptions options) const {
  for (const auto &parameter : named_parameters()) {
    parameter.value().wait();  // the init task has filled it
    auto &tensor = parameter.value().impl()->tensor();
    tensor = tensor.to(options);
  }
}

// --------------------------------------------------------- OptimizerModule
OrderedDict<std::string, std::shared_ptr<OptimizerState>> OptimizerModule::named_states() const { return states_; }

void OptimizerModule::set_lr(const double lr) const {
  for (const auto &state : states_) state.value()->set_lr(lr);
}

double OptimizerModule::get_lr() const {
  CS_ASSERT_TRUE(!states_.is_empty(), "Got empty state");
  return states_.begin()->value()->get_lr();
}

void OptimizerModule::zero_grad(const Scheduler &) const {
  const auto module = module_.lock();
  CS_ASSERT_TRUE(module != nullptr, "the module of this optimizer is gone");
  module->zero_grad();
}

// --------------------------------------------------------------- Embedding
EmbeddingImpl::EmbeddingImpl(const Scheduler &scheduler, const Options &options) {
  register_state(compute::Embedding::init(scheduler, options));
}
Tensor EmbeddingImpl::forward(const Scheduler &scheduler, const ReadOnlyTensor &input) const {
  return compute::Embedding::forward(scheduler, state(), input);
}
void EmbeddingImpl::backward(const Scheduler &scheduler, const ReadOnlyTensor &grad_output) const {
  compute::Embedding::backward(scheduler, state(), grad_output);
}
std::shared_ptr<compute::Embedding::State> EmbeddingImpl::state() const {
  return std::dynamic_pointer_cast<compute::Embedding::State>(state_);
}

// --------------------------------------------------------------- LayerNorm
LayerNormImpl::LayerNormImpl(const Scheduler &scheduler, const Options &options) {
  register_state(compute::LayerNorm::init(scheduler, options));
}
Tensor LayerNormImpl::forward(const Scheduler &scheduler, const ReadOnlyTensor &input) const {
  return compute::LayerNorm::forward(scheduler, state(), input);
}
Tensor LayerNormImpl::backward(const Scheduler &scheduler, const ReadOnlyTensor &grad_output) const {
  return compute::LayerNorm::backward(scheduler, state(), grad_output);
}
std::shared_ptr<compute::LayerNorm::State> LayerNormImpl::state() const {
  return std::dynamic_pointer_cast<compute::LayerNorm::State>(state_);
}

// ------------------------------------------------------------------- AdamW
AdamWImpl::AdamWImpl(const Scheduler &scheduler, const Module &module, const Options &options) {
  for (const auto &parameter : module.named_parameters())
    states_.insert(parameter.key(), optimizer::AdamW::init(scheduler, parameter.value(), options));
  module_ = module.weak_from_this();
  max_grad_norm_ = options.max_grad_norm();
}

void AdamWImpl::step(const Scheduler &scheduler) const {
  const auto module = module_.lock();
  CS_ASSERT_TRUE(module != nullptr, "the module of this optimizer is gone");
  auto increments = module->named_increments();
  // parameters that can share a launch: same element type, hyper-parameters and step count
  using Key = std::tuple<int, double, double, double, double, double, bool, long>;
  struct Group {
    std::vector<std::shared_ptr<OptimizerState>> states;
    std::vector<Tensor> parameters;
    std::vector<ReadOnlyTensor> gradients;
  };
  std::map<Key, Group> groups;
  std::vector<Key> order;  // first-seen order, so the task sequence does not depend on key values
  for (const auto &kv : states_) {
    const auto state = std::dynamic_pointer_cast<optimizer::AdamW::State>(kv.value());
    CS_ASSERT_TRUE(state != nullptr, "not an AdamW state: " + kv.key());
    const auto *increment = increments.find(kv.key());
    CS_ASSERT_TRUE(increment != nullptr, "parameter " + kv.key() + " is no longer in the module");
    // no host wait: the handle's at::Tensor exists since the task that made it was submitted
    // (tasks run inline on the submitting thread), and only its dtype is read here
    const auto &o = state->options;
    const Key key{static_cast<int>(increment->parameter.impl()->tensor().scalar_type()), o.lr, o.beta1, o.beta2,
                  o.eps, o.weight_decay, o.amsgrad, o.t};
    auto found = groups.find(key);
    if (found == groups.end()) {
      found = groups.emplace(key, Group{}).first;
      order.push_back(key);
    }
    found->second.states.push_back(kv.value());
    found->second.parameters.push_back(increment->parameter);
    found->second.gradients.push_back(increment->gradient);
  }
  CS_ASSERT_TRUE(!max_grad_norm_.has_value() || order.size() <= 1,
                 "gradient clipping needs one dtype and one set of hyper-parameters for all parameters");
  for (const auto &key : order) {
    const auto &group = groups.at(key);
    last_grad_norm_ = optimizer::AdamW::step(scheduler, group.states, group.parameters, group.gradients,
                                             max_grad_norm_, 2.0);
  }
}
}  // namespace cs::module
