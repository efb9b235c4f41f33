// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Builder-style option members, as the reference's CS_ARG (include/arg.h:20):
//   struct Options { CS_ARG(double, lr) = 1e-3; };   Options{}.lr(3e-4).lr()
#pragma once
#define CS_ARG(T, name)                                   \
 public:                                                  \
  inline auto name(const T &new_##name) -> decltype(*this) { \
    this->name##_ = new_##name;                           \
    return *this;                                         \
  }                                                       \
  inline const T &name() const noexcept { return this->name##_; } \
                                                          \
 private:                                                 \
  T name##_
