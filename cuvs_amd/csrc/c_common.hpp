/*
 * Helpers shared by the extern "C" translation units: exception translation
 * (cuVS c/src/core/exceptions.hpp:17-33) and DLPack tensor checks
 * (cuVS c/src/core/detail/interop.hpp:49-139).
 */
#pragma once

#include "detail.hpp"

#include <cuvs/core/c_api.h>
#include <cuvs/neighbors/ivf_pq.h>
#include <dlpack/dlpack.h>

#include <exception>
#include <string>

namespace cuvs::core {

void set_error_text(const std::string& s);

template <typename Fn>
cuvsError_t translate_exceptions(Fn func)
{
  cuvsError_t status;
  try {
    func();
    status = CUVS_SUCCESS;
    set_error_text("");
  } catch (const std::exception& e) {
    set_error_text(e.what());
    status = CUVS_ERROR;
  } catch (...) {
    set_error_text("unknown exception");
    status = CUVS_ERROR;
  }
  return status;
}

inline cuvs::resources* res_of(cuvsResources_t res)
{
  CUVS_EXPECTS(res != 0, "cuvsResources_t handle must not be null");
  return reinterpret_cast<cuvs::resources*>(res);
}

/** kDLCUDA* are accepted alongside kDLROCM* so that callers written against the CUDA build of
 *  the API keep working unchanged; both denote device-accessible memory here. */
inline bool is_dlpack_device_compatible(const DLTensor& t)
{
  return t.device.device_type == kDLCUDAManaged || t.device.device_type == kDLCUDAHost ||
         t.device.device_type == kDLCUDA || t.device.device_type == kDLROCM ||
         t.device.device_type == kDLROCMHost;
}

inline bool is_dlpack_host_compatible(const DLTensor& t)
{
  return t.device.device_type == kDLCUDAManaged || t.device.device_type == kDLCUDAHost ||
         t.device.device_type == kDLROCMHost || t.device.device_type == kDLCPU;
}

inline bool is_c_contiguous(const DLTensor& t)
{
  if (t.strides == nullptr) { return true; }
  int64_t expected = 1;
  for (int64_t i = t.ndim - 1; i >= 0; --i) {
    if (t.strides[i] != expected) { return false; }
    expected *= t.shape[i];
  }
  return true;
}

/** Checks that mirror from_dlpack<device_matrix_view<T, ..., row_major>>. */
inline void expect_tensor(const DLManagedTensor* mt, const char* name, int ndim, uint8_t code,
                          uint8_t bits)
{
  CUVS_EXPECTS(mt != nullptr, "%s must not be null", name);
  const DLTensor& t = mt->dl_tensor;
  CUVS_EXPECTS(is_c_contiguous(t), "Expected a row-major matrix");
  CUVS_EXPECTS(t.dtype.code == code, "code mismatch between return mdspan (%i) and DLTensor (%i)",
               int(code), int(t.dtype.code));
  CUVS_EXPECTS(t.dtype.bits == bits, "bits mismatch between return mdspan (%i) and DLTensor (%i)",
               int(bits), int(t.dtype.bits));
  CUVS_EXPECTS(t.dtype.lanes == 1, "More than 1 DLTensor lanes not supported");
  CUVS_EXPECTS(t.ndim == ndim, "ndim mismatch between return mdspan and DLTensor");
  for (int i = 0; i < t.ndim; i++) {
    CUVS_EXPECTS(t.shape[i] >= 0, "%s has a negative extent", name);
  }
}

/** Body of cuvsIvfPqSearch / cuvsAmdIvfPqSearchWithBitset on a given handle: tensor checks, then
 *  the C++ search (ivf_pq_c.cpp). */
void ivf_pq_search_tensors(cuvs::resources& res, cuvsIvfPqSearchParams_t params,
                           cuvsIvfPqIndex_t index, DLManagedTensor* queries,
                           DLManagedTensor* neighbors, DLManagedTensor* distances,
                           DLManagedTensor* bitset, int64_t n_bits);

inline void* tensor_data(const DLManagedTensor* mt)
{
  return static_cast<char*>(mt->dl_tensor.data) + mt->dl_tensor.byte_offset;
}

}  // namespace cuvs::core
