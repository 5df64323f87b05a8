/*
 * Appending rows to an index and encoding rows without storing them.
 * Role of cuVS ivf_pq::extend / transform (cpp/src/neighbors/ivf_pq/ivf_pq_build.cuh:998-1230,
 * :819-843 and ivf_pq_transform.cuh): predict the list of every row with the coarse quantiser,
 * compute the rotated residual, pick the nearest codebook entry per subspace, and write the codes
 * in the interleaved list layout.  Lists are kept in two arenas that are re-laid-out on every
 * call, so a list is always one contiguous, 32-row-aligned range.
 */
#include "detail.hpp"

#include <algorithm>

namespace cuvs::neighbors::ivf_pq {

namespace {

using detail::index_impl;

size_t elem_size(elem_type t) { return t == elem_type::f32 ? 4 : (t == elem_type::f16 ? 2 : 1); }

bool is_device_pointer(const void* p)
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

/** Rows processed per pass: bounds the [chunk, n_lists] score matrix to about 1 GiB. */
uint64_t chunk_rows_for(const index_impl& ix, uint64_t n_rows)
{
  uint64_t c = (uint64_t(1) << 28) / std::max<uint32_t>(ix.n_lists, 1);
  c          = std::max<uint64_t>(c, 1024);
  c          = std::min<uint64_t>(c, uint64_t(1) << 18);
  return std::min<uint64_t>(c, n_rows);
}

/** Rows encoded per pass: enough to fill the GPU, bounded by about 1 GiB for the float copy of the
 *  rows plus the rotated residuals. */
uint64_t encode_chunk_rows_for(const index_impl& ix, uint64_t n_rows)
{
  // per-cluster codebooks: larger passes, so that a pass holds many rows of each list (the rows of
  // a pass are encoded grouped by list)
  const bool per_cluster = ix.codebook_kind == codebook_gen::PER_CLUSTER;
  uint64_t c = (uint64_t(1) << (per_cluster ? 30 : 28)) / std::max<uint32_t>(ix.dim + ix.rot_dim, 1);
  c          = std::max<uint64_t>(c, 1024);
  c          = std::min<uint64_t>(c, uint64_t(1) << (per_cluster ? 22 : 20));
  return std::min<uint64_t>(c, n_rows);
}

/** Stages one chunk of rows on the device (when the input is host memory) and maps it to float. */
struct row_stager {
  const void* src;
  elem_type type;
  uint32_t dim;
  bool on_device;
  device_buffer staging;
  device_buffer xf;
  row_stager(const void* src_, elem_type t, uint32_t dim_, uint64_t chunk)
    : src(src_), type(t), dim(dim_), on_device(is_device_pointer(src_))
  {
    if (!on_device) { staging.allocate(chunk * dim * elem_size(t)); }
    xf.allocate(chunk * dim * sizeof(float));
  }
  float* load(uint64_t r0, uint64_t n, bool normalize, hipStream_t s)
  {
    const char* p = static_cast<const char*>(src) + r0 * dim * elem_size(type);
    const void* d = p;
    if (!on_device) {
      CUVS_HIP_TRY(hipMemcpyAsync(staging.ptr, p, n * dim * elem_size(type), hipMemcpyHostToDevice, s));
      d = staging.ptr;
    }
    detail::launch_map_queries(d, type, n * dim, xf.as<float>(), s);
    if (normalize) { detail::launch_normalize_rows(xf.as<float>(), n, dim, s); }
    return xf.as<float>();
  }
};

void predict_labels(const cuvs::resources& res, const index_impl& ix, const float* xf, uint64_t n,
                    float* scores, uint32_t* labels)
{
  // Rows join the list the coarse clustering would give them: nearest centre by L2 also for an
  // inner-product index, by inner product of the normalised row for cosine
  // (coarse_clustering_metric, cpp/src/neighbors/ivf_pq/ivf_pq_build.cuh:70-76, used by extend
  // :1141 and transform, ivf_pq_transform.cuh:58).
  const bool ip = ix.metric == detail::DistanceType::CosineExpanded;
  detail::launch_coarse_scores(xf, ix.centers.as<float>(), uint32_t(n), ix.n_lists, ix.dim,
                               ix.dim_ext, ip, false, scores, res.stream());
  detail::launch_select_probes(scores, uint32_t(n), ix.n_lists, 1, labels, res.stream());
}

detail::encode_args base_encode_args(const index_impl& ix)
{
  detail::encode_args a{};
  a.dim               = ix.dim;
  a.dim_ext           = ix.dim_ext;
  a.rot_dim           = ix.rot_dim;
  a.pq_dim            = ix.pq_dim;
  a.pq_len            = ix.pq_len;
  a.pq_bits           = ix.pq_bits;
  a.n_chunks          = ix.n_chunks;
  a.per_cluster       = ix.codebook_kind == codebook_gen::PER_CLUSTER;
  a.centers           = ix.centers.as<float>();
  a.rotation_t        = ix.rotation_t.as<float>();
  a.identity_rotation = ix.rotation_is_identity;
  a.pq_centers        = ix.pq_centers.as<float>();
  return a;
}

}  // namespace

namespace detail {

void relayout_lists(const cuvs::resources& res, index_impl& ix, const std::vector<uint32_t>& new_sizes)
{
  hipStream_t s = res.stream();
  CUVS_EXPECTS(new_sizes.size() == ix.n_lists, "one size per list is needed");
  std::vector<uint64_t> new_offsets(ix.n_lists + 1, 0);
  for (uint32_t l = 0; l < ix.n_lists; l++) {
    CUVS_EXPECTS(new_sizes[l] >= ix.h_list_sizes[l], "list %u cannot shrink while it is moved", l);
    new_offsets[l + 1] = new_offsets[l] + round_up_u64(new_sizes[l], kIndexGroupSize);
  }
  const uint64_t total_rows = new_offsets[ix.n_lists];
  // two groups of slack: the scan kernels read whole 64-row tiles past a list's last group
  device_buffer new_codes((total_rows / kIndexGroupSize + 2) * ix.group_bytes());
  device_buffer new_ids(total_rows * sizeof(int64_t));
  if (new_codes.bytes > 0) { CUVS_HIP_TRY(hipMemsetAsync(new_codes.ptr, 0, new_codes.bytes, s)); }
  if (new_ids.bytes > 0) { CUVS_HIP_TRY(hipMemsetAsync(new_ids.ptr, 0xFF, new_ids.bytes, s)); }

  device_buffer d_old_off(sizeof(uint64_t) * (ix.n_lists + 1));
  device_buffer d_new_off(sizeof(uint64_t) * (ix.n_lists + 1));
  CUVS_HIP_TRY(hipMemcpyAsync(d_old_off.ptr, ix.h_row_offsets.data(), d_old_off.bytes,
                              hipMemcpyHostToDevice, s));
  CUVS_HIP_TRY(hipMemcpyAsync(d_new_off.ptr, new_offsets.data(), d_new_off.bytes,
                              hipMemcpyHostToDevice, s));
  if (ix.size > 0) {
    launch_relocate_lists(ix.codes_arena.as<uint8_t>(), ix.ids_arena.as<int64_t>(),
                          new_codes.as<uint8_t>(), new_ids.as<int64_t>(), d_old_off.as<uint64_t>(),
                          d_new_off.as<uint64_t>(), ix.list_sizes.as<uint32_t>(), ix.n_lists,
                          ix.n_chunks, s);
  }
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // old arenas are released below
  ix.codes_arena   = std::move(new_codes);
  ix.ids_arena     = std::move(new_ids);
  ix.h_list_sizes  = new_sizes;
  ix.h_row_offsets = new_offsets;
  ix.recompute_internal_state(s);
}

}  // namespace detail

void extend(cuvs::resources const& res,
            const void* new_vectors,
            elem_type type,
            int64_t n_rows_signed,
            const int64_t* new_indices,
            index<int64_t>* idx,
            const uint32_t* labels_in)
{
  CUVS_EXPECTS(idx != nullptr && idx->impl() != nullptr, "index must not be null");
  auto& ix = *idx->impl();
  CUVS_EXPECTS(ix.centers.ptr != nullptr, "the index has no trained model");
  CUVS_EXPECTS(n_rows_signed >= 0, "number of rows must not be negative");
  if (n_rows_signed == 0) { return; }
  CUVS_EXPECTS(new_vectors != nullptr, "new_vectors must not be null");
  const uint64_t n_rows = uint64_t(n_rows_signed);
  CUVS_EXPECTS(uint64_t(ix.size) + n_rows < (uint64_t(1) << 40), "index too large");
  hipStream_t s        = res.stream();
  const bool cosine    = ix.metric == detail::DistanceType::CosineExpanded;
  device_buffer labels(n_rows * sizeof(uint32_t));

  /* 1. list labels */
  if (labels_in != nullptr) {
    CUVS_HIP_TRY(hipMemcpyAsync(labels.ptr, labels_in, n_rows * sizeof(uint32_t),
                                hipMemcpyDefault, s));
  } else if ((ix.metric == detail::DistanceType::L2Expanded || ix.metric == detail::DistanceType::L2SqrtExpanded) &&
             is_device_pointer(new_vectors)) {
    // the nearest list under the index's own metric is the search path's coarse stage with one probe
    search_params sp;
    sp.n_probes = 1;
    select_clusters(res, sp, *idx, new_vectors, type, n_rows_signed, labels.as<uint32_t>());
    CUVS_HIP_TRY(hipStreamSynchronize(s));
  } else if (cosine) {
    // cosine: the same stage on the normalised rows.  (On the rows as they are the largest product
    // is the same centre in exact arithmetic, but not always in fp32: the labels must be the ones
    // the normalised rows get, as in the reference's predict step.)
    const uint64_t label_chunk = chunk_rows_for(ix, n_rows);
    row_stager label_stager(new_vectors, type, ix.dim, label_chunk);
    search_params sp;
    sp.n_probes = 1;
    for (uint64_t r0 = 0; r0 < n_rows; r0 += label_chunk) {
      const uint64_t n = std::min(label_chunk, n_rows - r0);
      const float* xf  = label_stager.load(r0, n, true, s);
      select_clusters(res, sp, *idx, xf, elem_type::f32, int64_t(n), labels.as<uint32_t>() + r0);
    }
    CUVS_HIP_TRY(hipStreamSynchronize(s));  // the stager goes out of scope
  } else {
    const uint64_t label_chunk = chunk_rows_for(ix, n_rows);
    row_stager label_stager(new_vectors, type, ix.dim, label_chunk);
    device_buffer scores(label_chunk * ix.n_lists * sizeof(float) + detail::kSelectSlackBytes);
    for (uint64_t r0 = 0; r0 < n_rows; r0 += label_chunk) {
      const uint64_t n = std::min(label_chunk, n_rows - r0);
      float* xf        = label_stager.load(r0, n, cosine, s);
      predict_labels(res, ix, xf, n, scores.as<float>(), labels.as<uint32_t>() + r0);
    }
    CUVS_HIP_TRY(hipStreamSynchronize(s));  // the stager and the scores go out of scope
  }
  const uint64_t chunk = encode_chunk_rows_for(ix, n_rows);
  row_stager stager(new_vectors, type, ix.dim, chunk);

  /* 2. new list sizes */
  device_buffer counts(sizeof(uint32_t) * ix.n_lists);
  detail::launch_fill_u32(counts.as<uint32_t>(), 0, ix.n_lists, s);
  detail::launch_histogram(labels.as<uint32_t>(), n_rows, ix.n_lists, counts.as<uint32_t>(), s);
  std::vector<uint32_t> h_counts(ix.n_lists);
  CUVS_HIP_TRY(hipMemcpyAsync(h_counts.data(), counts.ptr, sizeof(uint32_t) * ix.n_lists,
                              hipMemcpyDeviceToHost, s));
  CUVS_HIP_TRY(hipStreamSynchronize(s));
  if (labels_in != nullptr) {
    uint64_t total = 0;
    for (uint32_t c : h_counts) { total += c; }
    // labels >= n_lists were left out of the histogram (nothing has been written to the index yet)
    CUVS_EXPECTS(total == n_rows, "labels must be smaller than n_lists (%u): %llu of %llu are not",
                 ix.n_lists, static_cast<unsigned long long>(n_rows - total),
                 static_cast<unsigned long long>(n_rows));
  }

  /* 3. new arena layout: every list owns round_up(size, 32) rows */
  std::vector<uint32_t> new_sizes(ix.n_lists);
  for (uint32_t l = 0; l < ix.n_lists; l++) {
    const uint64_t ns = uint64_t(ix.h_list_sizes[l]) + h_counts[l];
    CUVS_EXPECTS(ns <= 0xFFFFFFFFull, "list %u would exceed 2^32 rows", l);
    new_sizes[l] = uint32_t(ns);
  }
  // cursors start at the old sizes (the device copy of list_sizes still holds them)
  device_buffer cursors(sizeof(uint32_t) * ix.n_lists);
  CUVS_HIP_TRY(hipMemcpyAsync(cursors.ptr, ix.list_sizes.ptr, cursors.bytes,
                              hipMemcpyDeviceToDevice, s));
  const int64_t first_id = ix.size;
  detail::relayout_lists(res, ix, new_sizes);

  /* 4. encode and append */
  device_buffer scratch(chunk * ix.rot_dim * sizeof(float));
  device_buffer ids_stage;
  const bool group_rows = ix.codebook_kind == codebook_gen::PER_CLUSTER;
  device_buffer perm, perm_counters;
  if (group_rows) {
    perm.allocate(chunk * sizeof(uint32_t));
    perm_counters.allocate(size_t(2) * ix.n_lists * sizeof(uint32_t));
  }
  const bool ids_on_device = new_indices == nullptr || is_device_pointer(new_indices);
  if (!ids_on_device) { ids_stage.allocate(chunk * sizeof(int64_t)); }
  for (uint64_t r0 = 0; r0 < n_rows; r0 += chunk) {
    const uint64_t n = std::min(chunk, n_rows - r0);
    float* xf        = stager.load(r0, n, cosine, s);
    auto a           = base_encode_args(ix);
    a.xf             = xf;
    a.n_rows         = n;
    a.labels         = labels.as<uint32_t>() + r0;
    a.cursors        = cursors.as<uint32_t>();
    a.data_ptrs      = ix.data_ptrs.as<uint8_t*>();
    a.inds_ptrs      = ix.inds_ptrs.as<int64_t*>();
    a.first_id       = first_id + int64_t(r0);
    a.ids            = nullptr;
    if (new_indices != nullptr) {
      if (ids_on_device) {
        a.ids = new_indices + r0;
      } else {
        CUVS_HIP_TRY(hipMemcpyAsync(ids_stage.ptr, new_indices + r0, n * sizeof(int64_t),
                                    hipMemcpyHostToDevice, s));
        a.ids = ids_stage.as<int64_t>();
      }
    }
    a.flat_codes = nullptr;
    a.scratch    = scratch.as<float>();
    if (group_rows) {
      detail::launch_rows_by_label(a.labels, n, ix.n_lists, perm_counters.as<uint32_t>(),
                                   perm.as<uint32_t>(), s);
      a.perm = perm.as<uint32_t>();
    }
    detail::launch_encode(a, s);
  }
  ix.rebuild_lead_plane(s);
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // temporaries go out of scope
}

template <typename T>
void extend(cuvs::resources const& res,
            device_matrix_view<const T> new_vectors,
            const int64_t* new_indices,
            index<int64_t>* idx)
{
  CUVS_EXPECTS(idx != nullptr, "index must not be null");
  CUVS_EXPECTS(new_vectors.extent(1) == int64_t(idx->dim()),
               "new_vectors should have the same dimension as the index");
  elem_type t = elem_type::f32;
  if (std::is_same<T, _Float16>::value) { t = elem_type::f16; }
  if (std::is_same<T, int8_t>::value) { t = elem_type::i8; }
  if (std::is_same<T, uint8_t>::value) { t = elem_type::u8; }
  extend(res, new_vectors.data_handle(), t, new_vectors.extent(0), new_indices, idx, nullptr);
}
template void extend<float>(cuvs::resources const&, device_matrix_view<const float>, const int64_t*, index<int64_t>*);
template void extend<_Float16>(cuvs::resources const&, device_matrix_view<const _Float16>, const int64_t*, index<int64_t>*);
template void extend<int8_t>(cuvs::resources const&, device_matrix_view<const int8_t>, const int64_t*, index<int64_t>*);
template void extend<uint8_t>(cuvs::resources const&, device_matrix_view<const uint8_t>, const int64_t*, index<int64_t>*);

template <typename T>
index<int64_t> extend(cuvs::resources const& res,
                      device_matrix_view<const T> new_vectors,
                      const int64_t* new_indices,
                      const index<int64_t>& orig)
{
  index<int64_t> out = clone(res, orig);
  extend<T>(res, new_vectors, new_indices, &out);
  return out;
}
template index<int64_t> extend<float>(cuvs::resources const&, device_matrix_view<const float>, const int64_t*, const index<int64_t>&);
template index<int64_t> extend<_Float16>(cuvs::resources const&, device_matrix_view<const _Float16>, const int64_t*, const index<int64_t>&);
template index<int64_t> extend<int8_t>(cuvs::resources const&, device_matrix_view<const int8_t>, const int64_t*, const index<int64_t>&);
template index<int64_t> extend<uint8_t>(cuvs::resources const&, device_matrix_view<const uint8_t>, const int64_t*, const index<int64_t>&);

void transform(cuvs::resources const& res,
               const index<int64_t>& idx,
               const void* vectors,
               elem_type type,
               int64_t n_rows_signed,
               uint32_t* labels_out,
               uint8_t* codes_out)
{
  const auto& ix = *idx.impl();
  CUVS_EXPECTS(ix.centers.ptr != nullptr, "the index has no trained model");
  if (n_rows_signed <= 0) { return; }
  CUVS_EXPECTS(is_device_pointer(labels_out) && is_device_pointer(codes_out),
               "output tensors must be accessible from the device");
  const uint64_t n_rows    = uint64_t(n_rows_signed);
  hipStream_t s            = res.stream();
  const bool cosine        = ix.metric == detail::DistanceType::CosineExpanded;
  const uint64_t chunk     = chunk_rows_for(ix, n_rows);
  const uint32_t row_bytes = (ix.pq_dim * ix.pq_bits + 7) / 8;
  row_stager stager(vectors, type, ix.dim, chunk);
  device_buffer scores(chunk * ix.n_lists * sizeof(float) + detail::kSelectSlackBytes);
  device_buffer scratch(chunk * ix.rot_dim * sizeof(float));
  for (uint64_t r0 = 0; r0 < n_rows; r0 += chunk) {
    const uint64_t n = std::min(chunk, n_rows - r0);
    float* xf        = stager.load(r0, n, cosine, s);
    predict_labels(res, ix, xf, n, scores.as<float>(), labels_out + r0);
    auto a       = base_encode_args(ix);
    a.xf         = xf;
    a.n_rows     = n;
    a.labels     = labels_out + r0;
    a.flat_codes = codes_out + r0 * row_bytes;
    a.scratch    = scratch.as<float>();
    detail::launch_encode(a, s);
  }
  CUVS_HIP_TRY(hipStreamSynchronize(s));
}

/** Bit-contiguous codes of rows encoded against list `label` (no nearest-centre search): what
 *  cuVS' encode_list_data computes for helpers::codepacker::extend_list (ivf_pq_build.cuh:931-944). */
void encode_for_list(cuvs::resources const& res,
                     const index<int64_t>& idx,
                     const void* vectors,
                     elem_type type,
                     int64_t n_rows_signed,
                     uint32_t label,
                     uint8_t* codes_out)
{
  const auto& ix = *idx.impl();
  CUVS_EXPECTS(ix.centers.ptr != nullptr, "the index has no trained model");
  if (n_rows_signed <= 0) { return; }
  const uint64_t n_rows    = uint64_t(n_rows_signed);
  hipStream_t s            = res.stream();
  const bool cosine        = ix.metric == detail::DistanceType::CosineExpanded;
  const uint64_t chunk     = encode_chunk_rows_for(ix, n_rows);
  const uint32_t row_bytes = (ix.pq_dim * ix.pq_bits + 7) / 8;
  row_stager stager(vectors, type, ix.dim, chunk);
  device_buffer labels(chunk * sizeof(uint32_t));
  device_buffer scratch(chunk * ix.rot_dim * sizeof(float));
  detail::launch_fill_u32(labels.as<uint32_t>(), label, chunk, s);
  for (uint64_t r0 = 0; r0 < n_rows; r0 += chunk) {
    const uint64_t n = std::min(chunk, n_rows - r0);
    auto a           = base_encode_args(ix);
    a.xf             = stager.load(r0, n, cosine, s);
    a.n_rows         = n;
    a.labels         = labels.as<uint32_t>();
    a.flat_codes     = codes_out + r0 * row_bytes;
    a.scratch        = scratch.as<float>();
    detail::launch_encode(a, s);
  }
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // the temporaries go out of scope
}

}  // namespace cuvs::neighbors::ivf_pq
