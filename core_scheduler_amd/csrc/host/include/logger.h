// The declarations in this header restate the public interface of CoreScheduler
// (Copyright (c) 2024 The Core team, licensed under the Apache License, Version 2.0,
// http://www.apache.org/licenses/LICENSE-2.0) so that code written against it compiles
// unchanged; the comments and everything behind the declarations are this project's.
//
// Error convention of the reference (include/logger.h:26-34): a failed
// CS_ASSERT_TRUE logs at critical level and aborts; CS_WARN_TRUE only logs.
// spdlog is not a dependency here: the message goes to stderr.
#pragma once
#include <cstdio>
#include <cstdlib>
#include <string>

namespace cs::detail {
inline void log_line(const char *level, const std::string &msg, const char *file, int line) {
  std::fprintf(stderr, "[CS] [%s] %s (%s:%d)\n", level, msg.c_str(), file, line);
  std::fflush(stderr);
}
}  // namespace cs::detail

#define CS_ASSERT_TRUE(statement, ...)                                                   \
  do {                                                                                   \
    if (!(statement)) {                                                                  \
      ::cs::detail::log_line("critical", std::string(__VA_ARGS__), __FILE__, __LINE__); \
      std::abort();                                                                      \
    }                                                                                    \
  } while (false)

#define CS_WARN_TRUE(statement, ...)                                                     \
  do {                                                                                   \
    if (!(statement)) {                                                                  \
      ::cs::detail::log_line("warning", std::string(__VA_ARGS__), __FILE__, __LINE__);  \
    }                                                                                    \
  } while (false)
