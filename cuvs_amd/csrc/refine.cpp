/*
 * Host side of the refinement step: argument checks of cuVS refine_check_input
 * (cpp/src/neighbors/refine/refine_common.hpp:16-46) and the metric mapping of the IVF-Flat scan
 * the reference runs underneath (squared L2, its root, or the inner product as a similarity).
 */
#include "detail.hpp"

#include <cuvs/neighbors/refine.hpp>

namespace cuvs::neighbors {

void refine(cuvs::resources const& res, const void* dataset, const void* queries,
            ivf_pq::elem_type type, int64_t n_rows, int64_t n_queries, int64_t dim,
            const int64_t* candidates, int64_t n_candidates, int64_t* indices, float* distances,
            int64_t k, cuvs::distance::DistanceType metric)
{
  using cuvs::distance::DistanceType;
  CUVS_EXPECTS(n_rows >= 0 && n_queries >= 0 && dim > 0, "refine: invalid matrix extents");
  CUVS_EXPECTS(k > 0, "refine: k must be positive");
  CUVS_EXPECTS(n_candidates >= k,
               "Number of neighbor candidates must not be smaller than k (%lld vs %lld)",
               static_cast<long long>(n_candidates), static_cast<long long>(k));
  CUVS_EXPECTS(dataset != nullptr && queries != nullptr && candidates != nullptr &&
                 indices != nullptr && distances != nullptr,
               "refine: all tensors must be given");
  bool ip = false, sqrt_out = false;
  switch (metric) {
    case DistanceType::L2Expanded:
    case DistanceType::L2Unexpanded: break;
    case DistanceType::L2SqrtExpanded:
    case DistanceType::L2SqrtUnexpanded: sqrt_out = true; break;
    case DistanceType::InnerProduct: ip = true; break;
    default: fail("refine: unsupported distance type %d (L2, sqrt-L2 and inner product are supported)", int(metric));
  }
  CUVS_EXPECTS(n_queries <= 0x7fffffff && dim <= 16384 && n_candidates <= 0x7fffffff,
               "refine: extents out of range");
  ivf_pq::detail::launch_refine(dataset, queries, type, candidates, n_rows, uint32_t(n_queries),
                                uint32_t(dim), uint32_t(n_candidates), uint32_t(k), ip, sqrt_out,
                                indices, distances, res.stream());
}

template <typename T>
struct refine_elem;
template <>
struct refine_elem<float> {
  static constexpr ivf_pq::elem_type value = ivf_pq::elem_type::f32;
};
template <>
struct refine_elem<_Float16> {
  static constexpr ivf_pq::elem_type value = ivf_pq::elem_type::f16;
};
template <>
struct refine_elem<int8_t> {
  static constexpr ivf_pq::elem_type value = ivf_pq::elem_type::i8;
};
template <>
struct refine_elem<uint8_t> {
  static constexpr ivf_pq::elem_type value = ivf_pq::elem_type::u8;
};

template <typename T>
void refine(cuvs::resources const& res,
            device_matrix_view<const T> dataset,
            device_matrix_view<const T> queries,
            device_matrix_view<const int64_t> neighbor_candidates,
            device_matrix_view<int64_t> indices,
            device_matrix_view<float> distances,
            cuvs::distance::DistanceType metric)
{
  // refine_check_input
  const int64_t n_queries = queries.extent(0);
  CUVS_EXPECTS(indices.extent(0) == n_queries && distances.extent(0) == n_queries &&
                 neighbor_candidates.extent(0) == n_queries,
               "Number of rows in output indices, distances and candidates matrices must be equal "
               "with the number of rows in search matrix. Expected %lld, got %lld, %lld, and %lld",
               static_cast<long long>(n_queries), static_cast<long long>(indices.extent(0)),
               static_cast<long long>(distances.extent(0)),
               static_cast<long long>(neighbor_candidates.extent(0)));
  CUVS_EXPECTS(indices.extent(1) == distances.extent(1),
               "Number of columns in output indices and distances matrices must be equal to k");
  CUVS_EXPECTS(queries.extent(1) == dataset.extent(1),
               "Number of columns must be equal for dataset and queries");
  refine(res, dataset.data_handle(), queries.data_handle(), refine_elem<T>::value, dataset.extent(0),
         n_queries, dataset.extent(1), neighbor_candidates.data_handle(),
         neighbor_candidates.extent(1), indices.data_handle(), distances.data_handle(),
         indices.extent(1), metric);
}

#define INSTANTIATE_REFINE(T)                                                                  \
  template void refine<T>(cuvs::resources const&, device_matrix_view<const T>,                \
                          device_matrix_view<const T>, device_matrix_view<const int64_t>,     \
                          device_matrix_view<int64_t>, device_matrix_view<float>,             \
                          cuvs::distance::DistanceType);
INSTANTIATE_REFINE(float)
INSTANTIATE_REFINE(_Float16)
INSTANTIATE_REFINE(int8_t)
INSTANTIATE_REFINE(uint8_t)

}  // namespace cuvs::neighbors
