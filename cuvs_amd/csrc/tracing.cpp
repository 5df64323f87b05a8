/* Lookup of the ROCm marker library's range calls (see tracing.hpp). */
#include "tracing.hpp"

#include <dlfcn.h>

namespace cuvs::tracing {

namespace {

struct marker_api {
  int (*push)(const char*) = nullptr;
  int (*pop)()             = nullptr;
  marker_api()
  {
    // whatever is loaded already: the profiler's preloaded library, or one the application links
    push = reinterpret_cast<int (*)(const char*)>(dlsym(RTLD_DEFAULT, "roctxRangePushA"));
    pop  = reinterpret_cast<int (*)()>(dlsym(RTLD_DEFAULT, "roctxRangePop"));
    if (push == nullptr || pop == nullptr) {
      push = nullptr;
      pop  = nullptr;
    }
  }
};

const marker_api& api()
{
  static const marker_api a;
  return a;
}

}  // namespace

bool enabled() { return api().push != nullptr; }
void push(const char* name) { (void)api().push(name); }
void pop() { (void)api().pop(); }

}  // namespace cuvs::tracing
