/*
 * Host side of the refinement step: argument checks of cuVS refine_check_input
 * (cpp/src/neighbors/refine/refine_common.hpp:16-46) and the metric mapping of the IVF-Flat scan
 * the reference runs underneath (squared L2, its root, or the inner product as a similarity).
 */
#include "detail.hpp"

#include <cuvs/neighbors/refine.hpp>

#include <algorithm>
#include <cstring>
#include <thread>
#include <vector>

namespace cuvs::neighbors {

namespace {

struct refine_metric {
  bool ip       = false;
  bool sqrt_out = false;
};

/** Argument checks shared by the device and the host entry; the metric as the kernel takes it. */
refine_metric check_refine(const void* dataset, const void* queries, int64_t n_rows, int64_t n_queries,
                           int64_t dim, const int64_t* candidates, int64_t n_candidates,
                           const int64_t* indices, const float* distances, int64_t k,
                           cuvs::distance::DistanceType metric)
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
  return refine_metric{ip, sqrt_out};
}

struct pinned_buffer {
  void* ptr = nullptr;
  explicit pinned_buffer(size_t bytes) : ptr(cuvs::memory::host_allocate(bytes)) {}
  ~pinned_buffer() { cuvs::memory::host_deallocate(ptr); }
  pinned_buffer(const pinned_buffer&)            = delete;
  pinned_buffer& operator=(const pinned_buffer&) = delete;
  template <typename T>
  T* as() const
  {
    return static_cast<T*>(ptr);
  }
};

size_t refine_elem_bytes(ivf_pq::elem_type type)
{
  switch (type) {
    case ivf_pq::elem_type::f32: return 4;
    case ivf_pq::elem_type::f16: return 2;
    default: return 1;
  }
}

/** fn(first, last) over [0, n) on up to eight host threads (one when the range is small). */
template <typename F>
void for_ranges(int64_t n, int64_t min_per_thread, F&& fn)
{
  const int64_t hw        = int64_t(std::max(1u, std::thread::hardware_concurrency()));
  const int64_t n_threads = std::max<int64_t>(1, std::min<int64_t>({8, hw, n / std::max<int64_t>(1, min_per_thread)}));
  if (n_threads == 1) {
    fn(int64_t(0), n);
    return;
  }
  std::vector<std::thread> workers;
  const int64_t per = (n + n_threads - 1) / n_threads;
  for (int64_t t = 0; t < n_threads; t++) {
    const int64_t first = t * per, last = std::min(n, first + per);
    if (first < last) { workers.emplace_back([&fn, first, last] { fn(first, last); }); }
  }
  for (auto& w : workers) { w.join(); }
}

}  // namespace

void refine(cuvs::resources const& res, const void* dataset, const void* queries,
            ivf_pq::elem_type type, int64_t n_rows, int64_t n_queries, int64_t dim,
            const int64_t* candidates, int64_t n_candidates, int64_t* indices, float* distances,
            int64_t k, cuvs::distance::DistanceType metric)
{
  const refine_metric m = check_refine(dataset, queries, n_rows, n_queries, dim, candidates, n_candidates,
                                       indices, distances, k, metric);
  ivf_pq::detail::launch_refine(dataset, queries, type, candidates, n_rows, uint32_t(n_queries),
                                uint32_t(dim), uint32_t(n_candidates), uint32_t(k), m.ip, m.sqrt_out,
                                indices, distances, res.stream());
}

/*
 * Host matrices (the reference's refine_host, cpp/src/neighbors/refine/refine_host-inl.hpp, runs
 * on the CPU).  Only the candidate rows matter, so the dataset itself never crosses the bus: for a
 * batch of queries the host copies each candidate's row to slot (query, position) of a pinned
 * buffer, the device kernel ranks the slots (a candidate outside the dataset becomes slot -1, which
 * the kernel skips as it skips such an id), and the winning slots are turned back into the ids the
 * caller gave.  Ties are broken by position in the candidate list in both overloads, so the two
 * return the same rows.
 */
void refine_host(cuvs::resources const& res, const void* dataset, const void* queries,
                 ivf_pq::elem_type type, int64_t n_rows, int64_t n_queries, int64_t dim,
                 const int64_t* candidates, int64_t n_candidates, int64_t* indices, float* distances,
                 int64_t k, cuvs::distance::DistanceType metric)
{
  const refine_metric m = check_refine(dataset, queries, n_rows, n_queries, dim, candidates, n_candidates,
                                       indices, distances, k, metric);
  if (n_queries == 0) { return; }
  const size_t row_bytes  = size_t(dim) * refine_elem_bytes(type);
  const size_t per_query  = size_t(n_candidates) * row_bytes;
  constexpr size_t kBatchBytes = size_t(256) << 20;  // candidate rows in flight
  const int64_t batch = std::max<int64_t>(1, std::min<int64_t>(n_queries, int64_t(kBatchBytes / per_query)));
  CUVS_EXPECTS(uint64_t(batch) * uint64_t(n_candidates) <= 0x7fffffffull, "refine: extents out of range");

  const size_t n_slots = size_t(batch) * size_t(n_candidates);
  pinned_buffer rows_h(n_slots * row_bytes), slots_h(n_slots * 8), out_idx_h(size_t(batch) * k * 8),
    out_dist_h(size_t(batch) * k * 4);
  cuvs::device_buffer rows_d(n_slots * row_bytes), slots_d(n_slots * 8),
    queries_d(size_t(batch) * row_bytes), out_idx_d(size_t(batch) * k * 8), out_dist_d(size_t(batch) * k * 4);
  hipStream_t stream = res.stream();
  const auto* data   = static_cast<const uint8_t*>(dataset);

  for (int64_t q0 = 0; q0 < n_queries; q0 += batch) {
    const int64_t nq = std::min(batch, n_queries - q0);
    const int64_t n  = nq * n_candidates;
    for_ranges(n, 4096, [&](int64_t first, int64_t last) {
      for (int64_t s = first; s < last; s++) {
        const int64_t id = candidates[q0 * n_candidates + s];
        int64_t slot     = -1;
        if (id >= 0 && id < n_rows) {
          std::memcpy(rows_h.as<uint8_t>() + size_t(s) * row_bytes, data + size_t(id) * row_bytes, row_bytes);
          slot = s;
        }
        slots_h.as<int64_t>()[s] = slot;
      }
    });
    CUVS_HIP_TRY(hipMemcpyAsync(rows_d.ptr, rows_h.ptr, size_t(n) * row_bytes, hipMemcpyHostToDevice, stream));
    CUVS_HIP_TRY(hipMemcpyAsync(slots_d.ptr, slots_h.ptr, size_t(n) * 8, hipMemcpyHostToDevice, stream));
    CUVS_HIP_TRY(hipMemcpyAsync(queries_d.ptr, static_cast<const uint8_t*>(queries) + size_t(q0) * row_bytes,
                                size_t(nq) * row_bytes, hipMemcpyHostToDevice, stream));
    ivf_pq::detail::launch_refine(rows_d.ptr, queries_d.ptr, type, slots_d.as<int64_t>(), n, uint32_t(nq),
                                  uint32_t(dim), uint32_t(n_candidates), uint32_t(k), m.ip, m.sqrt_out,
                                  out_idx_d.as<int64_t>(), out_dist_d.as<float>(), stream);
    CUVS_HIP_TRY(hipMemcpyAsync(out_idx_h.ptr, out_idx_d.ptr, size_t(nq) * k * 8, hipMemcpyDeviceToHost, stream));
    CUVS_HIP_TRY(hipMemcpyAsync(out_dist_h.ptr, out_dist_d.ptr, size_t(nq) * k * 4, hipMemcpyDeviceToHost, stream));
    CUVS_HIP_TRY(hipStreamSynchronize(stream));
    for (int64_t i = 0; i < nq * k; i++) {
      const int64_t slot       = out_idx_h.as<int64_t>()[i];
      indices[q0 * k + i]      = slot < 0 ? slot : candidates[q0 * n_candidates + slot];
      distances[q0 * k + i]    = out_dist_h.as<float>()[i];
    }
  }
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

template <typename T>
void refine(cuvs::resources const& res,
            host_matrix_view<const T> dataset,
            host_matrix_view<const T> queries,
            host_matrix_view<const int64_t> neighbor_candidates,
            host_matrix_view<int64_t> indices,
            host_matrix_view<float> distances,
            cuvs::distance::DistanceType metric)
{
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
  refine_host(res, dataset.data_handle(), queries.data_handle(), refine_elem<T>::value, dataset.extent(0),
              n_queries, dataset.extent(1), neighbor_candidates.data_handle(),
              neighbor_candidates.extent(1), indices.data_handle(), distances.data_handle(),
              indices.extent(1), metric);
}

namespace {
template <typename View32, typename ViewOut32>
void check_u32_views(int64_t n_queries, const View32& cand, const ViewOut32& indices, int64_t dist_rows,
                     int64_t dist_cols, int64_t q_cols, int64_t d_cols)
{
  CUVS_EXPECTS(indices.extent(0) == n_queries && dist_rows == n_queries && cand.extent(0) == n_queries,
               "Number of rows in output indices, distances and candidates matrices must be equal "
               "with the number of rows in search matrix.");
  CUVS_EXPECTS(indices.extent(1) == dist_cols,
               "Number of columns in output indices and distances matrices must be equal to k");
  CUVS_EXPECTS(q_cols == d_cols, "Number of columns must be equal for dataset and queries");
}
}  // namespace

void refine(cuvs::resources const& res,
            device_matrix_view<const float> dataset,
            device_matrix_view<const float> queries,
            device_matrix_view<const uint32_t> neighbor_candidates,
            device_matrix_view<uint32_t> indices,
            device_matrix_view<float> distances,
            cuvs::distance::DistanceType metric)
{
  const int64_t nq = queries.extent(0), nc = neighbor_candidates.extent(1), k = indices.extent(1);
  check_u32_views(nq, neighbor_candidates, indices, distances.extent(0), distances.extent(1), queries.extent(1),
                  dataset.extent(1));
  CUVS_EXPECTS(nq >= 0 && nc >= 0 && k >= 0, "refine: invalid matrix extents");
  cuvs::device_buffer wide_cand(size_t(nq) * nc * 8 + 8), wide_idx(size_t(nq) * k * 8 + 8);
  hipStream_t s = res.stream();
  ivf_pq::detail::launch_widen_ids(neighbor_candidates.data_handle(), wide_cand.as<int64_t>(), uint64_t(nq) * nc, s);
  refine(res, dataset.data_handle(), queries.data_handle(), ivf_pq::elem_type::f32, dataset.extent(0), nq,
         dataset.extent(1), wide_cand.as<int64_t>(), nc, wide_idx.as<int64_t>(), distances.data_handle(), k, metric);
  ivf_pq::detail::launch_narrow_ids(wide_idx.as<int64_t>(), indices.data_handle(), uint64_t(nq) * k, s);
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // the wide copies go out of scope
}

void refine(cuvs::resources const& res,
            host_matrix_view<const float> dataset,
            host_matrix_view<const float> queries,
            host_matrix_view<const uint32_t> neighbor_candidates,
            host_matrix_view<uint32_t> indices,
            host_matrix_view<float> distances,
            cuvs::distance::DistanceType metric)
{
  const int64_t nq = queries.extent(0), nc = neighbor_candidates.extent(1), k = indices.extent(1);
  check_u32_views(nq, neighbor_candidates, indices, distances.extent(0), distances.extent(1), queries.extent(1),
                  dataset.extent(1));
  CUVS_EXPECTS(nq >= 0 && nc >= 0 && k >= 0, "refine: invalid matrix extents");
  std::vector<int64_t> wide_cand(size_t(nq) * nc + 1), wide_idx(size_t(nq) * k + 1);
  for (size_t i = 0; i < size_t(nq) * nc; i++) { wide_cand[i] = int64_t(neighbor_candidates.data_handle()[i]); }
  refine_host(res, dataset.data_handle(), queries.data_handle(), ivf_pq::elem_type::f32, dataset.extent(0), nq,
              dataset.extent(1), wide_cand.data(), nc, wide_idx.data(), distances.data_handle(), k, metric);
  for (size_t i = 0; i < size_t(nq) * k; i++) { indices.data_handle()[i] = uint32_t(wide_idx[i]); }
}

#define INSTANTIATE_REFINE(T)                                                                  \
  template void refine<T>(cuvs::resources const&, device_matrix_view<const T>,                \
                          device_matrix_view<const T>, device_matrix_view<const int64_t>,     \
                          device_matrix_view<int64_t>, device_matrix_view<float>,             \
                          cuvs::distance::DistanceType);                                      \
  template void refine<T>(cuvs::resources const&, host_matrix_view<const T>,                  \
                          host_matrix_view<const T>, host_matrix_view<const int64_t>,         \
                          host_matrix_view<int64_t>, host_matrix_view<float>,                 \
                          cuvs::distance::DistanceType);
INSTANTIATE_REFINE(float)
INSTANTIATE_REFINE(_Float16)
INSTANTIATE_REFINE(int8_t)
INSTANTIATE_REFINE(uint8_t)

}  // namespace cuvs::neighbors
