/*
 * Core C ABI: resources, stream control, error text, device allocation.
 * Replaces the cuVS entry points of the same names (c/src/core/c_api.cpp); exceptions are turned
 * into CUVS_ERROR plus a thread-local message exactly as c/src/core/exceptions.hpp:17-33 does.
 */
#include "c_common.hpp"

namespace {
thread_local std::string last_error_text;
cuvsLogLevel_t g_log_level = CUVS_LOG_LEVEL_INFO;
}  // namespace

namespace cuvs::core {
void set_error_text(const std::string& s) { last_error_text = s; }
}  // namespace cuvs::core

extern "C" {

const char* cuvsGetLastErrorText(void)
{
  return last_error_text.empty() ? nullptr : last_error_text.c_str();
}

void cuvsSetLastErrorText(const char* error) { last_error_text = error ? error : ""; }

cuvsLogLevel_t cuvsGetLogLevel(void) { return g_log_level; }
void cuvsSetLogLevel(cuvsLogLevel_t level) { g_log_level = level; }

cuvsError_t cuvsResourcesCreate(cuvsResources_t* res)
{
  return cuvs::core::translate_exceptions([=] {
    CUVS_EXPECTS(res != nullptr, "res must not be null");
    auto* r = new cuvs::resources();
    *res    = reinterpret_cast<uintptr_t>(r);
  });
}

cuvsError_t cuvsResourcesDestroy(cuvsResources_t res)
{
  return cuvs::core::translate_exceptions([=] { delete reinterpret_cast<cuvs::resources*>(res); });
}

cuvsError_t cuvsStreamSet(cuvsResources_t res, cudaStream_t stream)
{
  return cuvs::core::translate_exceptions([=] { cuvs::core::res_of(res)->set_stream(stream); });
}

cuvsError_t cuvsStreamGet(cuvsResources_t res, cudaStream_t* stream)
{
  return cuvs::core::translate_exceptions([=] {
    CUVS_EXPECTS(stream != nullptr, "stream must not be null");
    *stream = cuvs::core::res_of(res)->stream();
  });
}

cuvsError_t cuvsStreamSync(cuvsResources_t res)
{
  return cuvs::core::translate_exceptions([=] { cuvs::core::res_of(res)->sync(); });
}

cuvsError_t cuvsDeviceIdGet(cuvsResources_t res, int* device_id)
{
  return cuvs::core::translate_exceptions([=] {
    CUVS_EXPECTS(device_id != nullptr, "device_id must not be null");
    *device_id = cuvs::core::res_of(res)->device_id();
  });
}

cuvsError_t cuvsResourcesSetWorkspacePool(cuvsResources_t res, int percent_of_free_memory)
{
  return cuvs::core::translate_exceptions([=] {
    CUVS_EXPECTS(percent_of_free_memory > 0 && percent_of_free_memory <= 100,
                 "percent_of_free_memory must be within (0, 100]");
    size_t free_b = 0, total_b = 0;
    CUVS_HIP_TRY(hipMemGetInfo(&free_b, &total_b));
    cuvs::core::res_of(res)->set_workspace_limit(free_b / 100 * size_t(percent_of_free_memory));
  });
}

cuvsError_t cuvsRMMAlloc(cuvsResources_t res, void** ptr, size_t bytes)
{
  return cuvs::core::translate_exceptions([=] {
    (void)cuvs::core::res_of(res);
    CUVS_EXPECTS(ptr != nullptr, "ptr must not be null");
    CUVS_HIP_TRY(hipMalloc(ptr, bytes));
  });
}

cuvsError_t cuvsRMMFree(cuvsResources_t res, void* ptr, size_t)
{
  return cuvs::core::translate_exceptions([=] {
    (void)cuvs::core::res_of(res);
    CUVS_HIP_TRY(hipFree(ptr));
  });
}

cuvsError_t cuvsVersionGet(uint16_t* major, uint16_t* minor, uint16_t* patch)
{
  return cuvs::core::translate_exceptions([=] {
    CUVS_EXPECTS(major && minor && patch, "output pointers must not be null");
    *major = 26;  // API level of the cuVS release whose search entry points are mirrored
    *minor = 10;
    *patch = 0;
  });
}

}  // extern "C"
