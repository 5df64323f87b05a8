/*
 * Named ranges around the stages of the search for ROCm's marker tracing (rocprofv3
 * --marker-trace), in the role of the NVTX ranges of the reference
 * (cpp/src/core/nvtx.hpp:12-21; cpp/src/neighbors/ivf_pq/ivf_pq_search.cuh:74-79,436-441,894-899,
 * 974-975).  The marker library is not linked: its entry points are looked up once among the
 * objects already loaded into the process (the profiler preloads it; an application that links it
 * counts too).  Without it a range costs one predictable branch and formats nothing.
 */
#pragma once

#include <cstdarg>
#include <cstdio>

namespace cuvs::tracing {

/** The marker library's push / pop are reachable in this process. */
bool enabled();
void push(const char* name);
void pop();

/** Scope guard: `range r("ivf_pq::search(n_queries = %u)", n);` */
class range {
 public:
  explicit range(const char* fmt, ...) __attribute__((format(printf, 2, 3))) : on_(enabled())
  {
    if (!on_) { return; }
    char buf[256];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    push(buf);
  }
  ~range()
  {
    if (on_) { pop(); }
  }
  range(const range&)            = delete;
  range& operator=(const range&) = delete;

 private:
  bool on_;
};

}  // namespace cuvs::tracing
