/*
 * Host side of knn_merge_parts (cuVS cpp/src/neighbors/knn_merge_parts.cu) and its C entry point.
 */
#include "c_common.hpp"
#include "detail.hpp"

#include <cuvs/neighbors/knn_merge_parts.h>
#include <cuvs/neighbors/knn_merge_parts.hpp>

namespace cuvs::neighbors {

namespace detail {
template <typename IdT>
void launch_merge_parts(const float* in_keys, const IdT* in_ids, float* out_keys, IdT* out_ids,
                        uint64_t n_samples, uint32_t n_parts, uint32_t k, const IdT* translations,
                        hipStream_t stream);
}

template <typename IdT>
void knn_merge_parts(cuvs::resources const& res,
                     device_matrix_view<const float> in_keys,
                     device_matrix_view<const IdT> in_ids,
                     device_matrix_view<float> out_keys,
                     device_matrix_view<IdT> out_ids,
                     const IdT* translations,
                     int64_t n_parts)
{
  // knn_merge_parts.cu: extents of the four matrices must agree
  CUVS_EXPECTS(n_parts > 0, "n_parts must be positive");
  CUVS_EXPECTS(in_keys.extent(1) == in_ids.extent(1) && in_keys.extent(0) == in_ids.extent(0),
               "in_keys and in_ids must have the same shape");
  CUVS_EXPECTS(out_keys.extent(0) == out_ids.extent(0) && out_keys.extent(1) == out_ids.extent(1),
               "out_keys and out_ids must have the same shape");
  CUVS_EXPECTS(out_keys.extent(1) == in_keys.extent(1), "input and output must have the same k");
  CUVS_EXPECTS(in_keys.extent(0) == out_keys.extent(0) * n_parts,
               "the input must hold n_parts blocks of as many rows as the output");
  CUVS_EXPECTS(translations != nullptr, "translations must not be null");
  detail::launch_merge_parts<IdT>(in_keys.data_handle(), in_ids.data_handle(), out_keys.data_handle(),
                                  out_ids.data_handle(), uint64_t(out_keys.extent(0)), uint32_t(n_parts),
                                  uint32_t(out_keys.extent(1)), translations, res.stream());
}

template void knn_merge_parts<int64_t>(cuvs::resources const&, device_matrix_view<const float>,
                                       device_matrix_view<const int64_t>, device_matrix_view<float>,
                                       device_matrix_view<int64_t>, const int64_t*, int64_t);
template void knn_merge_parts<int32_t>(cuvs::resources const&, device_matrix_view<const float>,
                                       device_matrix_view<const int32_t>, device_matrix_view<float>,
                                       device_matrix_view<int32_t>, const int32_t*, int64_t);
template void knn_merge_parts<uint32_t>(cuvs::resources const&, device_matrix_view<const float>,
                                        device_matrix_view<const uint32_t>, device_matrix_view<float>,
                                        device_matrix_view<uint32_t>, const uint32_t*, int64_t);

}  // namespace cuvs::neighbors

using namespace cuvs::core;

extern "C" cuvsError_t cuvsAmdKnnMergeParts(cuvsResources_t res,
                                            DLManagedTensor* in_keys_t,
                                            DLManagedTensor* in_ids_t,
                                            DLManagedTensor* translations_t,
                                            DLManagedTensor* out_keys_t,
                                            DLManagedTensor* out_ids_t)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(in_keys_t && in_ids_t && translations_t && out_keys_t && out_ids_t,
                 "tensors must not be null");
    for (auto* t : {in_keys_t, in_ids_t, translations_t, out_keys_t, out_ids_t}) {
      CUVS_EXPECTS(is_dlpack_device_compatible(t->dl_tensor), "Tensors must all be accessible from the device");
    }
    expect_tensor(in_keys_t, "in_keys", 2, kDLFloat, 32);
    expect_tensor(in_ids_t, "in_ids", 2, kDLInt, 64);
    expect_tensor(out_keys_t, "out_keys", 2, kDLFloat, 32);
    expect_tensor(out_ids_t, "out_ids", 2, kDLInt, 64);
    expect_tensor(translations_t, "translations", 1, kDLInt, 64);
    const int64_t n_parts = translations_t->dl_tensor.shape[0];
    const auto& ik        = in_keys_t->dl_tensor;
    const auto& ok        = out_keys_t->dl_tensor;
    using cuvs::device_matrix_view;
    cuvs::neighbors::knn_merge_parts<int64_t>(
      *res_of(res),
      device_matrix_view<const float>{static_cast<const float*>(tensor_data(in_keys_t)), ik.shape[0], ik.shape[1]},
      device_matrix_view<const int64_t>{static_cast<const int64_t*>(tensor_data(in_ids_t)),
                                        in_ids_t->dl_tensor.shape[0], in_ids_t->dl_tensor.shape[1]},
      device_matrix_view<float>{static_cast<float*>(tensor_data(out_keys_t)), ok.shape[0], ok.shape[1]},
      device_matrix_view<int64_t>{static_cast<int64_t*>(tensor_data(out_ids_t)), out_ids_t->dl_tensor.shape[0],
                                  out_ids_t->dl_tensor.shape[1]},
      static_cast<const int64_t*>(tensor_data(translations_t)), n_parts);
  });
}
