/*
 * Index training: coarse centres, rotation matrix and PQ codebooks from a dataset.
 * Role of cuVS ivf_pq::build (cpp/src/neighbors/ivf_pq/ivf_pq_build.cuh:1240-1410): subsample a
 * training set, cluster it into n_lists balanced clusters, label the training rows, make the
 * rotation matrix, train the codebooks on the rotated residuals, and (add_data_on_build) encode
 * the whole dataset.
 *
 * The reference clusters hierarchically (mesoclusters, then fine clusters inside each) to keep the
 * assignment step affordable; here the assignment step is the search path's coarse stage (fp32
 * matrix-core scores + selection of the best centre), fast enough that the clustering is flat:
 * every iteration assigns every training row against all n_lists centres.  The balancing rule is
 * the reference's (size-sorted pairs of under- and overfull clusters, kmeans_balanced.cuh:616-720).
 */
#include "detail.hpp"

#include <algorithm>
#include <cmath>
#include <numeric>
#include <random>
#include <vector>

namespace cuvs::neighbors::ivf_pq {

namespace {

using detail::DistanceType;
using detail::index_impl;

size_t elem_size(elem_type t) { return t == elem_type::f32 ? 4 : (t == elem_type::f16 ? 2 : 1); }

bool on_device(const void* p)
{
  hipPointerAttribute_t attr;
  const hipError_t st = hipPointerGetAttributes(&attr, p);
  if (st != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged ||
         attr.type == hipMemoryTypeHost;
}

constexpr uint32_t kTrainSeed = 137;  // the reference's RngState seed (ivf_pq_build.cuh:1284)

/** Training rows as float [n_train, dim] on the device: row i is a pseudo-random row of the i-th
 *  stretch of `ratio` dataset rows. */
void gather_trainset(const cuvs::resources& res, const void* dataset, elem_type type, uint64_t ratio,
                     uint64_t n_train, uint32_t dim, bool normalize, float* out)
{
  hipStream_t s            = res.stream();
  const uint64_t row_bytes = uint64_t(dim) * elem_size(type);
  device_buffer raw(n_train * row_bytes);
  if (on_device(dataset)) {
    detail::launch_gather_rows(dataset, row_bytes, n_train, ratio, kTrainSeed, raw.ptr, s);
  } else {
    // host dataset: pick the same rows on the host (same hash as the kernel), one upload
    std::vector<uint8_t> host(n_train * row_bytes);
    auto mix = [](uint32_t x) {
      x ^= x >> 16;
      x *= 0x7feb352du;
      x ^= x >> 15;
      x *= 0x846ca68bu;
      x ^= x >> 16;
      return x;
    };
    for (uint64_t i = 0; i < n_train; i++) {
      const uint64_t row = i * ratio + (ratio > 1 ? mix(uint32_t(i) ^ kTrainSeed) % ratio : 0);
      std::copy_n(static_cast<const uint8_t*>(dataset) + row * row_bytes, row_bytes,
                  host.data() + i * row_bytes);
    }
    CUVS_HIP_TRY(hipMemcpyAsync(raw.ptr, host.data(), host.size(), hipMemcpyHostToDevice, s));
    CUVS_HIP_TRY(hipStreamSynchronize(s));
  }
  detail::launch_map_queries(raw.ptr, type, n_train * dim, out, s);
  if (normalize) { detail::launch_normalize_rows(out, n_train, dim, s); }
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // `raw` goes out of scope
}

/** Size-sorted pairs of clusters to rebalance: the i-th smallest receives from the i-th largest
 *  while the small one is underfull or the large one overfull (kmeans_balanced.cuh:650-670). */
uint32_t balance_pairs(const std::vector<uint32_t>& sizes, uint64_t n_rows, std::vector<uint32_t>& receivers,
                       std::vector<uint32_t>& donors)
{
  const uint32_t n = uint32_t(sizes.size());
  const float average = float(n_rows) / float(n);
  const float lower = 0.25f * average, upper = 4.0f * average;
  std::vector<std::pair<uint32_t, uint32_t>> sorted(n);
  for (uint32_t c = 0; c < n; c++) { sorted[c] = {sizes[c], c}; }
  std::sort(sorted.begin(), sorted.end());
  receivers.clear();
  donors.clear();
  for (uint32_t p = 0; p < n / 2; p++) {
    const auto [small_size, small_cluster] = sorted[p];
    const auto [large_size, large_cluster] = sorted[n - 1 - p];
    if (small_cluster == large_cluster || large_size == 0) { break; }
    if (float(small_size) >= lower && float(large_size) <= upper) { break; }
    receivers.push_back(small_cluster);
    donors.push_back(large_cluster);
  }
  return uint32_t(receivers.size());
}

}  // namespace

namespace detail {

/** rotation [rot_dim, dim]: the identity (zero-padded) unless a random one is asked for or needed
 *  (make_rotation_matrix, ivf_pq_build_common.cu:235-261): then `dim` orthonormal columns. */
std::vector<float> make_rotation(uint32_t rot_dim, uint32_t dim, bool force_random)
{
  std::vector<float> r(size_t(rot_dim) * dim, 0.0f);
  if (!force_random && rot_dim == dim) {
    for (uint32_t d = 0; d < dim; d++) { r[size_t(d) * dim + d] = 1.0f; }
    return r;
  }
  // Gram-Schmidt (two passes) of `dim` Gaussian vectors of length rot_dim
  std::mt19937_64 gen(7);
  std::normal_distribution<double> normal(0.0, 1.0);
  std::vector<std::vector<double>> cols(dim, std::vector<double>(rot_dim));
  for (uint32_t d = 0; d < dim; d++) {
    auto& v = cols[d];
    for (auto& e : v) { e = normal(gen); }
    for (int pass = 0; pass < 2; pass++) {
      for (uint32_t p = 0; p < d; p++) {
        double dot = 0.0;
        for (uint32_t i = 0; i < rot_dim; i++) { dot += v[i] * cols[p][i]; }
        for (uint32_t i = 0; i < rot_dim; i++) { v[i] -= dot * cols[p][i]; }
      }
    }
    double nrm = 0.0;
    for (double e : v) { nrm += e * e; }
    nrm = std::sqrt(nrm);
    for (auto& e : v) { e /= nrm; }
  }
  for (uint32_t o = 0; o < rot_dim; o++) {
    for (uint32_t d = 0; d < dim; d++) { r[size_t(o) * dim + d] = float(cols[d][o]); }
  }
  return r;
}


}  // namespace detail

index<int64_t> build(cuvs::resources const& res_c,
                     const index_params& params,
                     const void* dataset,
                     elem_type type,
                     int64_t n_rows_signed,
                     uint32_t dim)
{
  auto& res = const_cast<cuvs::resources&>(res_c);
  CUVS_EXPECTS(dataset != nullptr && n_rows_signed > 0, "the dataset must not be empty");
  const uint64_t n_rows = uint64_t(n_rows_signed);
  CUVS_EXPECTS(n_rows >= params.n_lists, "number of rows can't be less than n_lists");
  CUVS_EXPECTS(params.kmeans_trainset_fraction > 0.0 && params.kmeans_trainset_fraction <= 1.0,
               "kmeans_trainset_fraction must be in (0, 1]");
  CUVS_EXPECTS(params.codes_layout == list_layout::INTERLEAVED,
               "only the INTERLEAVED codes layout is supported");
  hipStream_t s = res.stream();

  // a scratch index that holds only the coarse centres: the expectation step runs the search
  // path's coarse stage on it
  index<int64_t> coarse;
  auto& cx = *coarse.impl();
  detail::init_index(cx, params, dim);
  const uint32_t L = cx.n_lists;
  CUVS_EXPECTS(cx.pq_len <= detail::train_codebook_max_pq_len(),
               "codebook training supports pq_len up to %u (dim %u / pq_dim %u gives %u)",
               detail::train_codebook_max_pq_len(), dim, cx.pq_dim, cx.pq_len);
  const bool cosine = cx.metric == DistanceType::CosineExpanded;
  // clustering metric: L2 also for inner product (coarse_clustering_metric, ivf_pq_build.cuh:70-76)
  if (cx.metric == DistanceType::InnerProduct || cx.metric == DistanceType::L2SqrtExpanded) {
    cx.metric = DistanceType::L2Expanded;
  }

  /* 1. training set (ivf_pq_build.cuh:1285-1345) */
  const uint64_t want   = std::max<uint64_t>(uint64_t(params.kmeans_trainset_fraction * double(n_rows)), L);
  const uint64_t ratio  = std::max<uint64_t>(1, n_rows / want);
  const uint64_t n_train = n_rows / ratio;
  CUVS_EXPECTS(n_train <= 0xFFFFFFFFull, "training set too large; lower kmeans_trainset_fraction");
  device_buffer trainset(n_train * dim * sizeof(float));
  gather_trainset(res, dataset, type, ratio, n_train, dim, cosine, trainset.as<float>());

  /* 2. balanced k-means of the coarse centres */
  device_buffer flat(size_t(L) * dim * sizeof(float));
  device_buffer sums(size_t(L) * dim * sizeof(float));
  device_buffer counts(size_t(L) * sizeof(uint32_t)), member(size_t(L) * sizeof(uint32_t));
  device_buffer labels(n_train * sizeof(uint32_t));
  device_buffer d_recv(size_t(L) * sizeof(uint32_t)), d_donor(size_t(L) * sizeof(uint32_t));
  cx.centers.allocate(size_t(L) * cx.dim_ext * sizeof(float));
  // initial centres: training rows spread evenly over the set
  detail::launch_gather_rows(trainset.ptr, uint64_t(dim) * 4, L, n_train / L, kTrainSeed + 1, flat.ptr, s);

  search_params sp;
  sp.n_probes = 1;
  auto assign = [&]() {
    detail::launch_set_centers(flat.as<float>(), L, dim, cx.dim_ext, cx.centers.as<float>(), s);
    cx.refresh_coarse(s);
    select_clusters(res, sp, coarse, trainset.ptr, elem_type::f32, int64_t(n_train), labels.as<uint32_t>());
  };
  std::vector<uint32_t> h_counts(L), receivers, donors;
  uint32_t n_iters           = std::max<uint32_t>(params.kmeans_n_iters, 1);
  const uint32_t iters_cap   = 2 * n_iters + 2;
  const uint32_t pullback    = 2;  // balancing_pullback (kmeans_balanced.cuh:752-820)
  uint32_t balancing_counter = pullback;
  for (uint32_t iter = 0; iter < n_iters; iter++) {
    if (iter > 0) {
      CUVS_HIP_TRY(hipMemcpyAsync(h_counts.data(), counts.ptr, counts.bytes, hipMemcpyDeviceToHost, s));
      CUVS_HIP_TRY(hipStreamSynchronize(s));
      const uint32_t n_pairs = balance_pairs(h_counts, n_train, receivers, donors);
      if (n_pairs > 0) {
        CUVS_HIP_TRY(hipMemcpyAsync(d_recv.ptr, receivers.data(), n_pairs * 4, hipMemcpyHostToDevice, s));
        CUVS_HIP_TRY(hipMemcpyAsync(d_donor.ptr, donors.data(), n_pairs * 4, hipMemcpyHostToDevice, s));
        detail::launch_adjust_centers(d_recv.as<uint32_t>(), d_donor.as<uint32_t>(), n_pairs,
                                      trainset.as<float>(), member.as<uint32_t>(), dim, 0.05f,
                                      flat.as<float>(), s);
        CUVS_HIP_TRY(hipStreamSynchronize(s));  // the host vectors are reused next iteration
        if (balancing_counter++ >= pullback) {
          balancing_counter -= pullback;
          if (n_iters < iters_cap) { n_iters++; }
        }
      }
    }
    assign();
    CUVS_HIP_TRY(hipMemsetAsync(sums.ptr, 0, sums.bytes, s));
    CUVS_HIP_TRY(hipMemsetAsync(counts.ptr, 0, counts.bytes, s));
    detail::launch_accumulate(trainset.as<float>(), labels.as<uint32_t>(), n_train, dim,
                              sums.as<float>(), counts.as<uint32_t>(), member.as<uint32_t>(), s);
    detail::launch_finish_centers(sums.as<float>(), counts.as<uint32_t>(), L, dim, cosine, flat.as<float>(), s);
  }
  assign();  // labels of the training rows under the final centres (ivf_pq_build.cuh:1361-1369)

  /* 3. rotation and rotated centres */
  const std::vector<float> rot = detail::make_rotation(cx.rot_dim, dim, params.force_random_rotation);
  std::vector<float> rot_t(rot.size());
  bool identity = cx.rot_dim == dim;
  for (uint32_t o = 0; o < cx.rot_dim; o++) {
    for (uint32_t d = 0; d < dim; d++) {
      const float v                 = rot[size_t(o) * dim + d];
      rot_t[size_t(d) * cx.rot_dim + o] = v;
      if (v != (o == d ? 1.0f : 0.0f)) { identity = false; }
    }
  }
  device_buffer d_rot(rot.size() * sizeof(float)), d_rot_t(rot.size() * sizeof(float));
  CUVS_HIP_TRY(hipMemcpyAsync(d_rot.ptr, rot.data(), d_rot.bytes, hipMemcpyHostToDevice, s));
  CUVS_HIP_TRY(hipMemcpyAsync(d_rot_t.ptr, rot_t.data(), d_rot_t.bytes, hipMemcpyHostToDevice, s));
  device_buffer centers_rot(size_t(L) * cx.rot_dim * sizeof(float));
  detail::launch_rotate(flat.as<float>(), d_rot_t.as<float>(), L, dim, cx.rot_dim, identity, false,
                        CUDA_R_32F, centers_rot.as<float>(), s);

  /* 4. codebooks on the rotated residuals of the training rows */
  const bool per_cluster = cx.codebook_kind == codebook_gen::PER_CLUSTER;
  const uint32_t book    = cx.book_size;
  // rows used: max_train_points_per_pq_code per entry (ivf_pq_build.cuh:340-343, :475-481)
  const uint64_t n_pq = per_cluster ? n_train
                                    : std::min<uint64_t>(n_train, uint64_t(params.max_train_points_per_pq_code) * book);
  device_buffer diff(n_pq * dim * sizeof(float));
  device_buffer resid(n_pq * cx.rot_dim * sizeof(float));
  detail::launch_residuals(trainset.as<float>(), labels.as<uint32_t>(), cx.centers.as<float>(), n_pq, dim,
                           cx.dim_ext, diff.as<float>(), s);
  for (uint64_t r0 = 0; r0 < n_pq; r0 += (1u << 20)) {
    const uint32_t n = uint32_t(std::min<uint64_t>(1u << 20, n_pq - r0));
    detail::launch_rotate(diff.as<float>() + r0 * dim, d_rot_t.as<float>(), n, dim, cx.rot_dim, identity,
                          false, CUDA_R_32F, resid.as<float>() + r0 * cx.rot_dim, s);
  }
  const uint32_t n_groups = per_cluster ? L : cx.pq_dim;
  device_buffer pq_centers(size_t(n_groups) * cx.pq_len * book * sizeof(float));
  device_buffer d_rows, d_offsets;
  uint32_t max_samples = uint32_t(std::min<uint64_t>(n_pq, 0xFFFFFFFFull));
  if (per_cluster) {
    // training rows grouped by list
    std::vector<uint32_t> h_labels(n_train);
    CUVS_HIP_TRY(hipMemcpyAsync(h_labels.data(), labels.ptr, labels.bytes, hipMemcpyDeviceToHost, s));
    CUVS_HIP_TRY(hipStreamSynchronize(s));
    std::vector<uint32_t> offsets(size_t(L) + 1, 0), rows(n_train);
    for (uint32_t l : h_labels) { offsets[l + 1]++; }
    std::partial_sum(offsets.begin(), offsets.end(), offsets.begin());
    std::vector<uint32_t> cursor(offsets.begin(), offsets.end() - 1);
    for (uint64_t i = 0; i < n_train; i++) { rows[cursor[h_labels[i]]++] = uint32_t(i); }
    d_rows.allocate(rows.size() * 4);
    d_offsets.allocate(offsets.size() * 4);
    CUVS_HIP_TRY(hipMemcpyAsync(d_rows.ptr, rows.data(), d_rows.bytes, hipMemcpyHostToDevice, s));
    CUVS_HIP_TRY(hipMemcpyAsync(d_offsets.ptr, offsets.data(), d_offsets.bytes, hipMemcpyHostToDevice, s));
    CUVS_HIP_TRY(hipStreamSynchronize(s));
    max_samples = uint32_t(std::min<uint64_t>(
      uint64_t(params.max_train_points_per_pq_code) * std::max<uint32_t>(book, cx.pq_dim), 0xFFFFFFFFull));
  }
  detail::launch_train_codebooks(resid.as<float>(), cx.rot_dim, cx.pq_dim, cx.pq_len, book, per_cluster,
                                 n_groups, uint32_t(n_pq), d_rows.as<uint32_t>(), d_offsets.as<uint32_t>(),
                                 max_samples, std::max<uint32_t>(params.kmeans_n_iters, 1), kTrainSeed,
                                 pq_centers.as<float>(), s);

  /* 5. the index, and the data */
  detail::launch_set_centers(flat.as<float>(), L, dim, cx.dim_ext, cx.centers.as<float>(), s);
  index<int64_t> idx = build(res, params, dim, pq_centers.as<float>(), cx.centers.as<float>(),
                             centers_rot.as<float>(), d_rot.as<float>());
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // training buffers go out of scope
  trainset.release();
  resid.release();
  diff.release();
  if (params.add_data_on_build) { extend(res, dataset, type, n_rows_signed, nullptr, &idx); }
  return idx;
}

template <typename T>
index<int64_t> build(cuvs::resources const& res, const index_params& params,
                     device_matrix_view<const T> dataset)
{
  elem_type t = elem_type::f32;
  if (std::is_same<T, _Float16>::value) { t = elem_type::f16; }
  if (std::is_same<T, int8_t>::value) { t = elem_type::i8; }
  if (std::is_same<T, uint8_t>::value) { t = elem_type::u8; }
  return build(res, params, dataset.data_handle(), t, dataset.extent(0), uint32_t(dataset.extent(1)));
}
template index<int64_t> build<float>(cuvs::resources const&, const index_params&, device_matrix_view<const float>);
template index<int64_t> build<_Float16>(cuvs::resources const&, const index_params&, device_matrix_view<const _Float16>);
template index<int64_t> build<int8_t>(cuvs::resources const&, const index_params&, device_matrix_view<const int8_t>);
template index<int64_t> build<uint8_t>(cuvs::resources const&, const index_params&, device_matrix_view<const uint8_t>);

template <typename T>
void build(cuvs::resources const& res, const index_params& params, device_matrix_view<const T> dataset,
           index<int64_t>* idx)
{
  CUVS_EXPECTS(idx != nullptr, "index must not be null");
  *idx = build<T>(res, params, dataset);
}
template void build<float>(cuvs::resources const&, const index_params&, device_matrix_view<const float>, index<int64_t>*);
template void build<_Float16>(cuvs::resources const&, const index_params&, device_matrix_view<const _Float16>, index<int64_t>*);
template void build<int8_t>(cuvs::resources const&, const index_params&, device_matrix_view<const int8_t>, index<int64_t>*);
template void build<uint8_t>(cuvs::resources const&, const index_params&, device_matrix_view<const uint8_t>, index<int64_t>*);

}  // namespace cuvs::neighbors::ivf_pq
