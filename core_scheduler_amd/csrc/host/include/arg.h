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
