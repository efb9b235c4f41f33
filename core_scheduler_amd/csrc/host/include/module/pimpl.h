// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Holder classes for modules (the reference's include/module/pimpl.h:21-30): `Name` is a
// shared-pointer holder of `NameImpl`, built on libtorch's ModuleHolder.
#pragma once
#include <torch/csrc/api/include/torch/nn/pimpl.h>

#define CS_MODULE_IMPL(Name, ImplType)                                 \
  class Name : public torch::nn::ModuleHolder<ImplType> { /* NOLINT */ \
   public:                                                             \
    using torch::nn::ModuleHolder<ImplType>::ModuleHolder;             \
    using Impl = ImplType;                                             \
    using Options = typename Impl::Options;                            \
  }

#define CS_MODULE(Name) CS_MODULE_IMPL(Name, Name##Impl)
