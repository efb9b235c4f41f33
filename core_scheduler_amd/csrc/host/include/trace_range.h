// Named ranges in profiler traces (the reference's include/nvtx_helper.h:21-41, which pushes
// NVTX ranges; here they are ROCTx ranges, which rocprofv3 --marker-trace records).  The
// scheduler opens one around every task body with the task's name
// (src/threading/dynamic_scheduler.cpp:135,148 in the reference); CS_TRACE_RANGE_FN opens one
// for the rest of the enclosing scope.  Without a profiler attached a range costs a call into
// the ROCTx library and nothing else.
#pragma once
#include <rocprofiler-sdk-roctx/roctx.h>

#include <string>

namespace cs {
struct TraceRange {
  explicit TraceRange(const char *name) { roctxRangePushA(name); }
  explicit TraceRange(const std::string &name) { roctxRangePushA(name.c_str()); }
  TraceRange(const TraceRange &) = delete;
  TraceRange &operator=(const TraceRange &) = delete;
  ~TraceRange() { roctxRangePop(); }
};
}  // namespace cs

#define CS_TRACE_CONCAT_(a, b) a##b
#define CS_TRACE_CONCAT(a, b) CS_TRACE_CONCAT_(a, b)
#define CS_TRACE_RANGE_FN(NAME) ::cs::TraceRange CS_TRACE_CONCAT(cs_trace_range_, __LINE__)(NAME)
