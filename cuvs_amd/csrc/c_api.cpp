/*
 * Core C ABI: resources, stream control, error text, device allocation.
 * Replaces the cuVS entry points of the same names (c/src/core/c_api.cpp); exceptions are turned
 * into CUVS_ERROR plus a thread-local message exactly as c/src/core/exceptions.hpp:17-33 does.
 */
#include "c_common.hpp"

#include <cuvs/version_config.h>

#include <memory>

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

cuvsError_t cuvsResourcesCreateWithMemoryTracking(cuvsResources_t* res, const char* csv_path,
                                                  int64_t sample_interval_ms)
{
  return cuvs::core::translate_exceptions([=] {
    CUVS_EXPECTS(res != nullptr, "res must not be null");
    CUVS_EXPECTS(csv_path != nullptr && csv_path[0] != '\0', "csv_path must be a non-empty string");
    CUVS_EXPECTS(sample_interval_ms >= 0, "sample_interval_ms must be >= 0");
    auto r = std::make_unique<cuvs::resources>();
    r->track_memory(csv_path, sample_interval_ms);
    *res = reinterpret_cast<uintptr_t>(r.release());
  });
}

namespace {
[[noreturn]] void no_multi_gpu()
{
  cuvs::fail("multi-GPU resources are not part of this library: it drives one GPU per process");
}
}  // namespace

cuvsError_t cuvsMultiGpuResourcesCreate(cuvsResources_t*)
{
  return cuvs::core::translate_exceptions([] { no_multi_gpu(); });
}

cuvsError_t cuvsMultiGpuResourcesCreateWithDeviceIds(cuvsResources_t*, DLManagedTensor*)
{
  return cuvs::core::translate_exceptions([] { no_multi_gpu(); });
}

cuvsError_t cuvsMultiGpuResourcesDestroy(cuvsResources_t)
{
  return cuvs::core::translate_exceptions([] { no_multi_gpu(); });
}

cuvsError_t cuvsMultiGpuResourcesSetMemoryPool(cuvsResources_t, int)
{
  return cuvs::core::translate_exceptions([] { no_multi_gpu(); });
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

cuvsError_t cuvsResourcesSetWorkspacePool(cuvsResources_t res, size_t initial_size_bytes)
{
  return cuvs::core::translate_exceptions(
    [=] { cuvs::core::res_of(res)->set_workspace_pool(initial_size_bytes); });
}

cuvsError_t cuvsRMMAlloc(cuvsResources_t res, void** ptr, size_t bytes)
{
  return cuvs::core::translate_exceptions([=] {
    auto* r = cuvs::core::res_of(res);
    CUVS_EXPECTS(ptr != nullptr, "ptr must not be null");
    if (auto* own = r->workspace_pool()) {
      *ptr = cuvs::memory::pool_allocate(*own, bytes, r->stream(), true);
    } else {
      *ptr = cuvs::memory::allocate_on_stream(bytes, r->stream());
    }
  });
}

cuvsError_t cuvsRMMFree(cuvsResources_t res, void* ptr, size_t)
{
  return cuvs::core::translate_exceptions([=] {
    auto* r   = cuvs::core::res_of(res);
    auto* own = r->workspace_pool();
    if (ptr == nullptr || (own && cuvs::memory::pool_deallocate(*own, ptr, r->stream(), true))) { return; }
    cuvs::memory::deallocate_on_stream(ptr, r->stream());
  });
}

cuvsError_t cuvsRMMPoolMemoryResourceEnable(int initial_pool_size_percent, int max_pool_size_percent,
                                            bool managed)
{
  return cuvs::core::translate_exceptions(
    [=] { cuvs::memory::enable_pool(initial_pool_size_percent, max_pool_size_percent, managed); });
}

cuvsError_t cuvsRMMAsyncMemoryResourceEnable(void)
{
  return cuvs::core::translate_exceptions([] { cuvs::memory::enable_async(); });
}

cuvsError_t cuvsRMMMemoryResourceReset(void)
{
  return cuvs::core::translate_exceptions([] { cuvs::memory::reset(); });
}

cuvsError_t cuvsRMMHostAlloc(void** ptr, size_t bytes)
{
  return cuvs::core::translate_exceptions([=] {
    CUVS_EXPECTS(ptr != nullptr, "ptr must not be null");
    *ptr = cuvs::memory::host_allocate(bytes);
  });
}

cuvsError_t cuvsRMMHostFree(void* ptr, size_t)
{
  return cuvs::core::translate_exceptions([=] {
    cuvs::memory::host_deallocate(ptr);
  });
}

cuvsError_t cuvsVersionGet(uint16_t* major, uint16_t* minor, uint16_t* patch)
{
  return cuvs::core::translate_exceptions([=] {
    CUVS_EXPECTS(major && minor && patch, "output pointers must not be null");
    *major = CUVS_VERSION_MAJOR;  // API level of the cuVS release whose entry points are mirrored
    *minor = CUVS_VERSION_MINOR;
    *patch = CUVS_VERSION_PATCH;
  });
}

cuvsError_t cuvsMatrixCopy(cuvsResources_t res, DLManagedTensor* src_managed,
                           DLManagedTensor* dst_managed)
{
  return cuvs::core::translate_exceptions([=] {
    auto* r = cuvs::core::res_of(res);
    CUVS_EXPECTS(src_managed != nullptr && dst_managed != nullptr, "src and dst must not be null");
    const DLTensor& src = src_managed->dl_tensor;
    const DLTensor& dst = dst_managed->dl_tensor;
    CUVS_EXPECTS(src.ndim == dst.ndim, "src and dst tensors should have the same dimensions");
    for (int i = 0; i < src.ndim; ++i) {
      CUVS_EXPECTS(src.shape[i] == dst.shape[i], "shape mismatch between src and dst tensors");
    }
    CUVS_EXPECTS(src.dtype.code == dst.dtype.code, "dtype mismatch between src and dst tensors");
    CUVS_EXPECTS(src.dtype.bits == dst.dtype.bits,
                 "dtype bits width mismatch between src and dst tensors");
    const int bits       = src.dtype.bits;
    const bool supported = (src.dtype.code == kDLFloat && (bits == 16 || bits == 32 || bits == 64)) ||
                           ((src.dtype.code == kDLInt || src.dtype.code == kDLUInt) &&
                            (bits == 8 || bits == 16 || bits == 32 || bits == 64));
    CUVS_EXPECTS(supported && src.dtype.lanes == 1, "Unsupported dtype: %d and bits: %d",
                 int(src.dtype.code), bits);
    const size_t elt = size_t(bits) / 8;
    if (src.ndim == 2) {
      // rows may be further apart than their length on either side
      CUVS_EXPECTS((src.strides == nullptr || src.strides[1] == 1 || src.shape[1] <= 1) &&
                     (dst.strides == nullptr || dst.strides[1] == 1 || dst.shape[1] <= 1),
                   "cuvsMatrixCopy needs unit stride along the rows");
      const int64_t src_row = src.strides == nullptr ? src.shape[1] : src.strides[0];
      const int64_t dst_row = dst.strides == nullptr ? dst.shape[1] : dst.strides[0];
      CUVS_EXPECTS(src_row >= src.shape[1] && dst_row >= dst.shape[1], "row strides shorter than the rows");
      if (src.shape[0] == 0 || src.shape[1] == 0) { return; }
      CUVS_HIP_TRY(hipMemcpy2DAsync(cuvs::core::tensor_data(dst_managed), size_t(dst_row) * elt,
                                    cuvs::core::tensor_data(src_managed), size_t(src_row) * elt,
                                    size_t(src.shape[1]) * elt, size_t(src.shape[0]), hipMemcpyDefault,
                                    r->stream()));
    } else {
      CUVS_EXPECTS(src.strides == nullptr && dst.strides == nullptr,
                   "cuvsCopyMatrix only supports strides with 2D inputs");
      size_t elements = 1;
      for (int i = 0; i < src.ndim; ++i) { elements *= size_t(src.shape[i]); }
      if (elements == 0) { return; }
      CUVS_HIP_TRY(hipMemcpyAsync(cuvs::core::tensor_data(dst_managed), cuvs::core::tensor_data(src_managed),
                                  elements * elt, hipMemcpyDefault, r->stream()));
    }
  });
}

/** Deleter of the views cuvsMatrixSliceRows makes: they own their shape and stride arrays only. */
static void release_matrix_view(DLManagedTensor* tensor)
{
  delete[] tensor->dl_tensor.shape;
  tensor->dl_tensor.shape = nullptr;
  delete[] tensor->dl_tensor.strides;
  tensor->dl_tensor.strides = nullptr;
}

cuvsError_t cuvsMatrixSliceRows(cuvsResources_t res, DLManagedTensor* src_managed, int64_t start,
                                int64_t end, DLManagedTensor* dst_managed)
{
  return cuvs::core::translate_exceptions([=] {
    (void)cuvs::core::res_of(res);
    CUVS_EXPECTS(src_managed != nullptr && dst_managed != nullptr, "src and dst must not be null");
    CUVS_EXPECTS(end >= start, "end index must be greater than start index");
    const DLTensor& src = src_managed->dl_tensor;
    DLTensor& dst       = dst_managed->dl_tensor;
    CUVS_EXPECTS(src.ndim == 1 || src.ndim == 2, "src should be a 1 or 2 dimensional tensor");
    CUVS_EXPECTS(src.shape != nullptr, "shape should be initialized in the src tensor");
    CUVS_EXPECTS(start >= 0 && end <= src.shape[0], "rows [%lld, %lld) are outside the %lld rows of src",
                 static_cast<long long>(start), static_cast<long long>(end),
                 static_cast<long long>(src.shape[0]));
    dst.dtype       = src.dtype;
    dst.device      = src.device;
    dst.ndim        = src.ndim;
    dst.byte_offset = src.byte_offset;
    dst.strides     = nullptr;
    dst.shape       = new int64_t[dst.ndim];
    dst.shape[0]    = end - start;
    int64_t row_stride = 1;
    if (dst.ndim == 2) {
      dst.shape[1] = src.shape[1];
      row_stride   = src.shape[1];
      if (src.strides != nullptr) {
        dst.strides    = new int64_t[2];
        dst.strides[0] = src.strides[0];
        dst.strides[1] = src.strides[1];
        row_stride     = src.strides[0];
      }
    }
    dst.data = static_cast<char*>(src.data) + start * row_stride * int64_t(dst.dtype.bits / 8);
    dst_managed->deleter     = release_matrix_view;
  });
}

}  // extern "C"
