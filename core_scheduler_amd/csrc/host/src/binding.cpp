// Python binding of the host API, so that the parity tests can drive cs::compute /
// cs::optimizer exactly as the reference's gtest suites do: build a DynamicScheduler, init an
// op state, call forward / backward, wait on the returned handles and compare.
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <memory>
#include <optional>
#include <sstream>
#include <string>
#include <vector>

#include "autocast.h"
#include "compute/cross_entropy.h"
#include "compute/embedding.h"
#include "compute/gelu.h"
#include "compute/layer_norm.h"
#include "compute/utils.h"
#include "memory/to_torch.h"
#include "module/adamw.h"
#include "module/embedding.h"
#include "module/layer_norm.h"
#include "module/module.h"
#include "optimizer/adamw.h"
#include "tensor_impl.h"
#include "threading/dynamic_scheduler.h"

namespace py = pybind11;
using namespace cs;

namespace {
at::ScalarType dtype_from(const std::string &name) {
  if (name == "float32") return at::kFloat;
  if (name == "float64") return at::kDouble;
  if (name == "float16") return at::kHalf;
  if (name == "bfloat16") return at::kBFloat16;
  throw std::invalid_argument("unknown dtype " + name);
}
Tensor as_tensor(const ReadOnlyTensor &t) {
  Tensor out;
  static_cast<ReadOnlyTensor &>(out) = t;
  return out;
}
c10::DeviceIndex device_of(const Scheduler &s) {
  return static_cast<c10::DeviceIndex>(s.impl() ? s.get_device_rank() : 0);
}
struct AutocastScope {
  std::unique_ptr<autocast::ContextGuard> guard;
};
// a module with no state of its own, to build trees from Python
struct Container final : module::Module {};
template <typename Value>
std::vector<std::pair<std::string, Value>> items(const OrderedDict<std::string, Value> &dict) {
  std::vector<std::pair<std::string, Value>> out;
  for (const auto &kv : dict) out.emplace_back(kv.key(), kv.value());
  return out;
}
}  // namespace

PYBIND11_MODULE(_cs_host, m) {
  m.doc() = "cs::compute / cs::optimizer host API over the gfx950 kernel library";

  // a bare Scheduler has no implementation behind it; it exists so that argument checks that
  // fail before any task is submitted can be exercised without a device
  py::class_<Scheduler>(m, "Scheduler").def(py::init<>()).def("get_device_rank", &Scheduler::get_device_rank);
  py::class_<DynamicScheduler, Scheduler>(m, "DynamicScheduler").def(py::init<int>(), py::arg("local_rank"));

  py::class_<ReadOnlyTensor>(m, "ReadOnlyTensor")
      .def("wait", &ReadOnlyTensor::wait)
      .def("numel", &ReadOnlyTensor::numel)
      .def("defined", [](const ReadOnlyTensor &t) { return t.impl()->tensor().defined(); })
      .def("sizes", [](const ReadOnlyTensor &t) { return t.sizes().vec(); })
      .def("priority", [](const ReadOnlyTensor &t) { return static_cast<int>(t.impl()->priority()); });
  py::class_<Tensor, ReadOnlyTensor>(m, "Tensor").def(py::init<>());

  // operator<< of a handle (include/tensor.h): waits, then at::print with 80 characters per line
  m.def("tensor_to_string", [](const ReadOnlyTensor &t) {
    std::ostringstream out;
    out << t;
    return out.str();
  }, py::arg("tensor"));
  m.def("to_torch", &memory::to_torch, py::arg("scheduler"), py::arg("tensor"));
  m.def("clip_grad_norm_", &compute::Utils::clip_grad_norm_, py::arg("scheduler"), py::arg("tensors"),
        py::arg("max_norm"), py::arg("norm_type") = 2.0);
  m.def("from_torch", &memory::from_torch, py::arg("scheduler"), py::arg("tensor"));
  // what cs::load does with each row of a checkpoint (src/module/module.cpp:216-218): the values,
  // converted to the parameter's dtype and device and viewed in its shape, are copied into it
  m.def("assign_", [](const Scheduler &s, const ReadOnlyTensor &parameter, const at::Tensor &values) {
    parameter.wait();
    auto &dst = parameter.impl()->tensor();
    TORCH_CHECK(dst.defined(), "assign_ needs a defined parameter");
    TORCH_CHECK(values.numel() == dst.numel(), "assign_: ", values.numel(), " values for a parameter of ", dst.numel());
    (void)dst.copy_(values.to(dst.options()).view(dst.sizes()));
    c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().synchronize();
  }, py::arg("scheduler"), py::arg("parameter"), py::arg("values"));

  py::class_<AutocastScope>(m, "autocast")
      .def(py::init([]() { return AutocastScope{}; }))
      .def("enter",
           [](AutocastScope &s, const Scheduler &sched, const std::string &dtype) {
             s.guard = std::make_unique<autocast::ContextGuard>(sched, dtype_from(dtype));
           })
      .def("exit", [](AutocastScope &s) { s.guard.reset(); });

  // ---- GeLU
  {
    using Op = compute::GeLU;
    py::class_<Op::State, std::shared_ptr<Op::State>>(m, "GeLUState");
    auto sub = m.def_submodule("GeLU");
    sub.def("init", [](const Scheduler &s, int approximate) {
      return approximate == 0 ? Op::init(s) : Op::init(s, Op::Options{}.approximate(approximate));
    }, py::arg("scheduler"), py::arg("approximate") = 0);
    sub.def("forward", &Op::forward);
    sub.def("backward", &Op::backward);
  }
  // ---- CrossEntropy
  {
    using Op = compute::CrossEntropy;
    py::class_<Op::State, std::shared_ptr<Op::State>>(m, "CrossEntropyState")
        .def("total_weight", [](const Op::State &s) { return as_tensor(s.backward.total_weight); })
        .def("set_weight", [](Op::State &s, const Tensor &t) { s.forward.weight = t; });
    auto sub = m.def_submodule("CrossEntropy");
    sub.def("init", [](const Scheduler &s, int reduction, int64_t ignore_index, double label_smoothing,
                       int64_t num_classes) {
      return Op::init(s, Op::Options{}
                             .reduction(static_cast<at::Reduction::Reduction>(reduction))
                             .ignore_index(ignore_index)
                             .label_smoothing(label_smoothing)
                             .num_classes(num_classes));
    }, py::arg("scheduler"), py::arg("reduction") = 1, py::arg("ignore_index") = -100,
            py::arg("label_smoothing") = 0.0, py::arg("num_classes") = -1);
    sub.def("forward", &Op::forward);
    sub.def("backward", &Op::backward);
  }
  // ---- LayerNorm
  {
    using Op = compute::LayerNorm;
    py::class_<Op::State, std::shared_ptr<Op::State>>(m, "LayerNormState")
        .def_property_readonly("weight", [](const Op::State &s) { return s.forward.weight; })
        .def_property_readonly("bias", [](const Op::State &s) { return s.forward.bias; })
        .def_property_readonly("grad_weight", [](const Op::State &s) { return s.forward.grad_weight; })
        .def_property_readonly("grad_bias", [](const Op::State &s) { return s.forward.grad_bias; })
        .def("set_weight", [](Op::State &s, const Tensor &t) { s.forward.weight = t; })
        .def("set_bias", [](Op::State &s, const Tensor &t) { s.forward.bias = t; })
        .def("parameter_names", [](const Op::State &s) { return s.parameters().keys(); })
        .def("zero_grad", &Op::State::zero_grad);
    auto sub = m.def_submodule("LayerNorm");
    sub.def("init", [](const Scheduler &s, std::vector<int64_t> shape, double eps, bool affine, bool bias,
                       const std::string &dtype) {
      return Op::init(s, Op::Options{shape}.eps(eps).elementwise_affine(affine).bias(bias)
                             .device(at::Device(at::kCUDA, device_of(s)))
                             .dtype(dtype_from(dtype)));
    }, py::arg("scheduler"), py::arg("normalized_shape"), py::arg("eps") = 1e-5,
            py::arg("elementwise_affine") = true, py::arg("bias") = true, py::arg("dtype") = "float32");
    sub.def("forward", &Op::forward);
    sub.def("backward", &Op::backward);
    sub.def("forward_with_residual", [](const Scheduler &s, const std::shared_ptr<Op::State> &state,
                                        const ReadOnlyTensor &x, const ReadOnlyTensor &residual) {
      const auto r = Op::forward_with_residual(s, state, x, residual);
      return std::make_pair(r.output, r.residual);
    });
    sub.def("backward_with_residual", &Op::backward_with_residual);
  }
  // ---- Embedding
  {
    using Op = compute::Embedding;
    py::class_<Op::State, std::shared_ptr<Op::State>>(m, "EmbeddingState")
        .def_property_readonly("weight", [](const Op::State &s) { return s.forward.weight; })
        .def_property_readonly("grad_weight", [](const Op::State &s) { return s.forward.grad_weight; })
        .def_property_readonly("padding_idx", [](const Op::State &s) { return s.args.padding_idx; })
        .def("set_weight", [](Op::State &s, const Tensor &t) { s.forward.weight = t; })
        .def("zero_grad", &Op::State::zero_grad);
    auto sub = m.def_submodule("Embedding");
    sub.def("init", [](const Scheduler &s, int64_t n, int64_t d, std::optional<int64_t> padding_idx,
                       std::optional<double> max_norm, const std::string &dtype, bool scale_grad_by_freq,
                       bool sparse) {
      auto o = Op::Options{n, d}
                   .device(at::Device(at::kCUDA, device_of(s)))
                   .dtype(dtype_from(dtype))
                   .scale_grad_by_freq(scale_grad_by_freq)
                   .sparse(sparse);
      if (padding_idx) o = o.padding_idx(*padding_idx);
      if (max_norm) o = o.max_norm(*max_norm);
      return Op::init(s, o);
    }, py::arg("scheduler"), py::arg("num_embeddings"), py::arg("embedding_dim"),
            py::arg("padding_idx") = py::none(), py::arg("max_norm") = py::none(), py::arg("dtype") = "float32",
            py::arg("scale_grad_by_freq") = false, py::arg("sparse") = false);
    sub.def("forward", &Op::forward);
    sub.def("backward", &Op::backward);
    sub.def("forward_with_positions", &Op::forward_with_positions);
    sub.def("backward_with_positions", &Op::backward_with_positions);
  }
  // ---- AdamW
  {
    using Op = optimizer::AdamW;
    py::class_<module::OptimizerState, std::shared_ptr<module::OptimizerState>>(m, "OptimizerState")
        .def("set_lr", &module::OptimizerState::set_lr)
        .def("get_lr", &module::OptimizerState::get_lr);
    py::class_<Op::State, module::OptimizerState, std::shared_ptr<Op::State>>(m, "AdamWState")
        .def_property_readonly("m", [](const Op::State &s) { return s.tensors.m; })
        .def_property_readonly("v", [](const Op::State &s) { return s.tensors.v; })
        .def_property_readonly("v_max", [](const Op::State &s) { return s.tensors.v_max; })
        .def_property_readonly("t", [](const Op::State &s) { return s.options.t; });
    auto sub = m.def_submodule("AdamW");
    sub.def("init", [](const Scheduler &s, const ReadOnlyTensor &p, double lr, double beta1, double beta2, double eps,
                       double weight_decay, bool amsgrad, long t) {
      return Op::init(s, p, Op::Options{}.lr(lr).beta1(beta1).beta2(beta2).eps(eps).weight_decay(weight_decay)
                                .amsgrad(amsgrad).t(t));
    }, py::arg("scheduler"), py::arg("parameter"), py::arg("lr") = 1e-3, py::arg("beta1") = 0.9,
            py::arg("beta2") = 0.999, py::arg("eps") = 1e-8, py::arg("weight_decay") = 1e-2,
            py::arg("amsgrad") = false, py::arg("t") = 0);
    sub.def("step", [](const Scheduler &s, const std::shared_ptr<Op::State> &state, const Tensor &w,
                       const ReadOnlyTensor &dw) { Op::step(s, state, w, dw); });
    sub.def("step_all", [](const Scheduler &s, const std::vector<std::shared_ptr<Op::State>> &states,
                           const std::vector<Tensor> &ws, const std::vector<Tensor> &dws) {
      std::vector<std::shared_ptr<module::OptimizerState>> base(states.begin(), states.end());
      std::vector<ReadOnlyTensor> grads(dws.begin(), dws.end());
      Op::step(s, base, ws, grads);
    });
  }
  // ---- checkpoints (cs::save / cs::load, include/module/module.h and optimizer_module.h)
  m.def("save_module", [](const std::shared_ptr<module::Module> &mod, const std::string &path) { cs::save(*mod, path); },
        py::arg("module"), py::arg("path"));
  m.def("load_module", [](const std::shared_ptr<module::Module> &mod, const std::string &path) { cs::load(*mod, path); },
        py::arg("module"), py::arg("path"));
  m.def("save_optimizer", [](const std::shared_ptr<module::AdamWImpl> &opt, const std::string &path) { cs::save(static_cast<const module::OptimizerModule &>(*opt), path); },
        py::arg("optimizer"), py::arg("path"));
  m.def("load_optimizer", [](const std::shared_ptr<module::AdamWImpl> &opt, const std::string &path) { cs::load(static_cast<const module::OptimizerModule &>(*opt), path); },
        py::arg("optimizer"), py::arg("path"));
  // ---- module layer
  {
    using module::Module;
    py::class_<Module, std::shared_ptr<Module>>(m, "Module")
        .def("named_parameters", [](const Module &mod) { return items(mod.named_parameters()); })
        .def("named_gradients", [](const Module &mod) { return items(mod.named_gradients()); })
        .def("named_states", [](const Module &mod) {
          std::vector<std::string> names;
          for (const auto &kv : mod.named_states()) names.push_back(kv.key());
          return names;
        })
        .def("named_increments", [](const Module &mod) {
          std::vector<std::tuple<std::string, Tensor, Tensor>> out;
          for (const auto &kv : mod.named_increments())
            out.emplace_back(kv.key(), kv.value().parameter, kv.value().gradient);
          return out;
        })
        .def("zero_grad", &Module::zero_grad)
        .def("to", [](const Module &mod, const std::string &dtype) { mod.to(at::TensorOptions().dtype(dtype_from(dtype))); });
    py::class_<Container, Module, std::shared_ptr<Container>>(m, "Container")
        .def(py::init([]() { return std::make_shared<Container>(); }))
        .def("register_module", [](Container &c, const std::string &name, const std::shared_ptr<Module> &child) {
          return c.register_module(name, child);
        });
    py::class_<module::EmbeddingImpl, Module, std::shared_ptr<module::EmbeddingImpl>>(m, "EmbeddingModule")
        .def(py::init([](const Scheduler &s, int64_t n, int64_t d, const std::string &dtype) {
               return std::make_shared<module::EmbeddingImpl>(
                   s, module::EmbeddingImpl::Options{n, d}.device(at::Device(at::kCUDA, device_of(s))).dtype(dtype_from(dtype)));
             }),
             py::arg("scheduler"), py::arg("num_embeddings"), py::arg("embedding_dim"), py::arg("dtype") = "float32")
        .def("forward", &module::EmbeddingImpl::forward)
        .def("backward", &module::EmbeddingImpl::backward)
        .def("state", &module::EmbeddingImpl::state);
    py::class_<module::LayerNormImpl, Module, std::shared_ptr<module::LayerNormImpl>>(m, "LayerNormModule")
        .def(py::init([](const Scheduler &s, std::vector<int64_t> shape, double eps, bool bias, const std::string &dtype) {
               return std::make_shared<module::LayerNormImpl>(
                   s, module::LayerNormImpl::Options{shape}.eps(eps).bias(bias)
                          .device(at::Device(at::kCUDA, device_of(s))).dtype(dtype_from(dtype)));
             }),
             py::arg("scheduler"), py::arg("normalized_shape"), py::arg("eps") = 1e-5, py::arg("bias") = true,
             py::arg("dtype") = "float32")
        .def("forward", &module::LayerNormImpl::forward)
        .def("backward", &module::LayerNormImpl::backward)
        .def("state", &module::LayerNormImpl::state);
    py::class_<module::AdamWImpl, std::shared_ptr<module::AdamWImpl>>(m, "AdamWModule")
        .def(py::init([](const Scheduler &s, const std::shared_ptr<Module> &mod, double lr, double beta1, double beta2,
                         double eps, double weight_decay, bool amsgrad, long t, std::optional<double> max_grad_norm) {
               auto o = module::AdamWImpl::Options{}.lr(lr).beta1(beta1).beta2(beta2).eps(eps)
                            .weight_decay(weight_decay).amsgrad(amsgrad).t(t);
               if (max_grad_norm) o = o.max_grad_norm(*max_grad_norm);
               return std::make_shared<module::AdamWImpl>(s, *mod, o);
             }),
             py::arg("scheduler"), py::arg("module"), py::arg("lr") = 1e-3, py::arg("beta1") = 0.9,
             py::arg("beta2") = 0.999, py::arg("eps") = 1e-8, py::arg("weight_decay") = 1e-2,
             py::arg("amsgrad") = false, py::arg("t") = 0, py::arg("max_grad_norm") = py::none())
        .def("step", &module::AdamWImpl::step)
        .def("last_grad_norm", &module::AdamWImpl::last_grad_norm)
        .def("zero_grad", &module::AdamWImpl::zero_grad)
        .def("set_lr", &module::AdamWImpl::set_lr)
        .def("get_lr", &module::AdamWImpl::get_lr)
        .def("named_states", [](const module::AdamWImpl &o) {
          std::vector<std::pair<std::string, std::shared_ptr<optimizer::AdamW::State>>> out;
          for (const auto &kv : o.named_states())
            out.emplace_back(kv.key(), std::dynamic_pointer_cast<optimizer::AdamW::State>(kv.value()));
          return out;
        });
  }
}
