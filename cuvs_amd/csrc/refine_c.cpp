/*
 * C ABI of the refinement step (cuVS c/src/neighbors/refine.cpp:62-135).
 */
#include "c_common.hpp"
#include "detail.hpp"

#include <cuvs/neighbors/refine.h>
#include <cuvs/neighbors/refine.hpp>

namespace {

using cuvs::neighbors::ivf_pq::elem_type;
using namespace cuvs::core;

bool refine_elem_type(const DLDataType& dt, elem_type* out)
{
  if (dt.code == kDLFloat && dt.bits == 32) { *out = elem_type::f32; return true; }
  if (dt.code == kDLFloat && dt.bits == 16) { *out = elem_type::f16; return true; }
  if (dt.code == kDLInt && dt.bits == 8) { *out = elem_type::i8; return true; }
  if (dt.code == kDLUInt && dt.bits == 8) { *out = elem_type::u8; return true; }
  return false;
}

}  // namespace

extern "C" cuvsError_t cuvsRefine(cuvsResources_t res,
                                  DLManagedTensor* dataset_t,
                                  DLManagedTensor* queries_t,
                                  DLManagedTensor* candidates_t,
                                  cuvsDistanceType metric,
                                  DLManagedTensor* indices_t,
                                  DLManagedTensor* distances_t)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(dataset_t && queries_t && candidates_t && indices_t && distances_t,
                 "tensors must not be null");
    const auto& dataset    = dataset_t->dl_tensor;
    const auto& queries    = queries_t->dl_tensor;
    const auto& candidates = candidates_t->dl_tensor;
    const auto& indices    = indices_t->dl_tensor;
    const auto& distances  = distances_t->dl_tensor;
    // all matrices on the device (or reachable from it: pinned, managed), or all in plain host
    // memory; the latter are staged through the device, a batch of queries at a time
    const bool on_device = is_dlpack_device_compatible(dataset);
    CUVS_EXPECTS(on_device == is_dlpack_device_compatible(queries) &&
                   on_device == is_dlpack_device_compatible(candidates) &&
                   on_device == is_dlpack_device_compatible(indices) &&
                   on_device == is_dlpack_device_compatible(distances),
                 "Tensors must either all be on device memory, or all on host memory");
    CUVS_EXPECTS(candidates.dtype.code == kDLInt && candidates.dtype.bits == 64,
                 "candidates should be of type int64_t");
    CUVS_EXPECTS(indices.dtype.code == kDLInt && indices.dtype.bits == 64,
                 "indices should be of type int64_t");
    CUVS_EXPECTS(distances.dtype.code == kDLFloat && distances.dtype.bits == 32,
                 "distances should be of type float32");
    CUVS_EXPECTS(queries.dtype.code == dataset.dtype.code && queries.dtype.bits == dataset.dtype.bits,
                 "type mismatch between dataset and queries");
    elem_type t;
    CUVS_EXPECTS(refine_elem_type(queries.dtype, &t), "Unsupported queries DLtensor dtype: %d and bits: %d",
                 int(queries.dtype.code), int(queries.dtype.bits));
    expect_tensor(dataset_t, "dataset", 2, dataset.dtype.code, dataset.dtype.bits);
    expect_tensor(queries_t, "queries", 2, queries.dtype.code, queries.dtype.bits);
    expect_tensor(candidates_t, "candidates", 2, kDLInt, 64);
    expect_tensor(indices_t, "indices", 2, kDLInt, 64);
    expect_tensor(distances_t, "distances", 2, kDLFloat, 32);
    // refine_check_input (cpp/src/neighbors/refine/refine_common.hpp:16-46)
    const int64_t n_queries = queries.shape[0];
    CUVS_EXPECTS(indices.shape[0] == n_queries && distances.shape[0] == n_queries &&
                   candidates.shape[0] == n_queries,
                 "Number of rows in output indices, distances and candidates matrices must be equal "
                 "with the number of rows in search matrix.");
    CUVS_EXPECTS(indices.shape[1] == distances.shape[1],
                 "Number of columns in output indices and distances matrices must be equal to k");
    CUVS_EXPECTS(queries.shape[1] == dataset.shape[1],
                 "Number of columns must be equal for dataset and queries");
    const auto type_of_metric = cuvs::distance::DistanceType(int(metric));
    const auto* cand          = static_cast<const int64_t*>(tensor_data(candidates_t));
    auto* out_idx             = static_cast<int64_t*>(tensor_data(indices_t));
    auto* out_dist            = static_cast<float*>(tensor_data(distances_t));
    if (on_device) {
      cuvs::neighbors::refine(*res_of(res), tensor_data(dataset_t), tensor_data(queries_t), t, dataset.shape[0],
                              n_queries, dataset.shape[1], cand, candidates.shape[1], out_idx, out_dist,
                              indices.shape[1], type_of_metric);
    } else {
      cuvs::neighbors::refine_host(*res_of(res), tensor_data(dataset_t), tensor_data(queries_t), t,
                                   dataset.shape[0], n_queries, dataset.shape[1], cand, candidates.shape[1],
                                   out_idx, out_dist, indices.shape[1], type_of_metric);
    }
  });
}
