/*
 * IVF-PQ index object: derived dimensions, model storage, list arenas and the dependent state
 * (pointer tables, sorted size prefix sums).  Contents and derived quantities follow cuVS
 * cpp/src/neighbors/ivf_pq_index.cu:78-111,223-235,599-622 and
 * cpp/include/cuvs/neighbors/ivf_pq.hpp:222-296.
 */
#include "detail.hpp"

#include <algorithm>
#include <cmath>
#include <functional>

namespace cuvs::neighbors::ivf_pq {

namespace detail {

/* Every live index, so that a write through a bare list pointer finds the index it belongs to. */
namespace {
std::mutex& registry_mutex()
{
  static std::mutex m;
  return m;
}
std::vector<index_impl*>& registry()
{
  static std::vector<index_impl*> all;
  return all;
}
}  // namespace

index_impl::index_impl()
{
  std::lock_guard<std::mutex> guard(registry_mutex());
  registry().push_back(this);
}

index_impl::~index_impl()
{
  std::lock_guard<std::mutex> guard(registry_mutex());
  auto& all = registry();
  all.erase(std::remove(all.begin(), all.end(), this), all.end());
}

void mark_lists_written(const void* list_data)
{
  const auto p = reinterpret_cast<uintptr_t>(list_data);
  std::lock_guard<std::mutex> guard(registry_mutex());
  for (index_impl* ix : registry()) {
    const auto begin = reinterpret_cast<uintptr_t>(ix->codes_arena.ptr);
    if (begin != 0 && p >= begin && p < begin + ix->codes_arena.bytes) { ix->derived_stale.store(true); }
  }
}

void screen_feedback::create()
{
  if (host != nullptr) { return; }
  CUVS_HIP_TRY(hipHostMalloc(reinterpret_cast<void**>(&host), 64, hipHostMallocDefault));
  host[0] = 0;
  CUVS_HIP_TRY(hipEventCreateWithFlags(&landed, hipEventDisableTiming));
}

void screen_feedback::collect()
{
  if (!pending || hipEventQuery(landed) != hipSuccess) { return; }
  pending = false;
  if (pending_pairs == 0) { return; }
  verdict* v = find(pending_probes, pending_k);
  if (v == nullptr) {
    // a new parameter set takes the place of the one used longest ago
    for (int i = kVerdicts - 1; i > 0; i--) { verdicts[i] = verdicts[i - 1]; }
    v         = &verdicts[0];
    v->probes = pending_probes;
    v->k      = pending_k;
    v->screened_searches = 0;
    v->screen_off        = false;
  }
  v->off            = double(host[0]) > kKeepLimit * double(pending_pairs);
  v->plain_searches = 0;
  // host[1]: pairs dropped on their lists' distance alone; what the screening kernel was given is the rest
  const double given = double(pending_pairs) - double(host[1]);
  v->screen_off          = !v->off && pending_far && double(host[0]) > kKeepLimit * given;
  v->unscreened_searches = 0;
}

screen_feedback::verdict* screen_feedback::find(uint32_t probes, uint32_t k)
{
  for (int i = 0; i < kVerdicts; i++) {
    if (verdicts[i].probes == probes && verdicts[i].k == k && probes != 0) {
      const verdict hit = verdicts[i];
      for (int j = i; j > 0; j--) { verdicts[j] = verdicts[j - 1]; }
      verdicts[0] = hit;
      return &verdicts[0];
    }
  }
  return nullptr;
}

screen_feedback::~screen_feedback()
{
  if (landed != nullptr) {
    (void)hipEventSynchronize(landed);  // a copy into `host` may still be on its way
    (void)hipEventDestroy(landed);
  }
  if (host != nullptr) { (void)hipHostFree(host); }
}

void init_index(index_impl& ix, const index_params& params, uint32_t dim)
{
  CUVS_EXPECTS(params.pq_bits >= 4 && params.pq_bits <= 8,
               "pq_bits must be within [4, 8], got %u", params.pq_bits);
  CUVS_EXPECTS(dim > 0, "dim must be positive");
  CUVS_EXPECTS(params.n_lists > 0, "n_lists must be positive");
  uint32_t pq_dim = params.pq_dim;
  if (pq_dim == 0) {
    // calculate_pq_dim (ivf_pq_index.cu:612-622): half the dimension from 128 up, rounded down
    // to a multiple of 32, or to a power of two below 32
    uint32_t d = dim >= 128 ? dim / 2 : dim;
    pq_dim     = (d / 32) * 32;
    if (pq_dim == 0) {
      pq_dim = 1;
      while ((pq_dim << 1) <= d) { pq_dim <<= 1; }
    }
  }
  CUVS_EXPECTS((params.pq_bits * pq_dim) % 8 == 0,
               "pq_bits * pq_dim must be a multiple of 8 (pq_bits = %u, pq_dim = %u)",
               params.pq_bits, pq_dim);
  switch (params.metric) {
    case DistanceType::L2Expanded:
    case DistanceType::L2SqrtExpanded:
    case DistanceType::InnerProduct:
    case DistanceType::CosineExpanded: break;
    default: fail("Unsupported distance type %d.", int(params.metric));
  }
  ix.metric                         = params.metric;
  ix.codebook_kind                  = params.codebook_kind;
  ix.conservative_memory_allocation = params.conservative_memory_allocation;
  ix.n_lists                        = params.n_lists;
  ix.dim                            = dim;
  ix.pq_bits                        = params.pq_bits;
  ix.pq_dim                         = pq_dim;
  ix.dim_ext                        = round_up_u32(dim + 1, 8);
  ix.pq_len                         = (dim + pq_dim - 1) / pq_dim;
  ix.rot_dim                        = ix.pq_len * pq_dim;
  ix.book_size                      = 1u << params.pq_bits;
  const uint32_t cpc                = (kIndexGroupVecLen * 8u) / params.pq_bits;
  ix.n_chunks                       = (pq_dim + cpc - 1) / cpc;
  ix.h_list_sizes.assign(ix.n_lists, 0);
  ix.h_row_offsets.assign(ix.n_lists + 1, 0);
  ix.accum_sorted_sizes.assign(ix.n_lists + 1, 0);
  ix.list_sizes.allocate(sizeof(uint32_t) * ix.n_lists);
  ix.data_ptrs.allocate(sizeof(void*) * ix.n_lists);
  ix.inds_ptrs.allocate(sizeof(void*) * ix.n_lists);
  ix.size = 0;
  ix.feedback.create();
}

void index_impl::recompute_internal_state(hipStream_t stream)
{
  std::vector<uint8_t*> dptr(n_lists);
  std::vector<int64_t*> iptr(n_lists);
  const uint64_t gb = group_bytes();
  for (uint32_t l = 0; l < n_lists; l++) {
    dptr[l] = codes_arena.as<uint8_t>() + (h_row_offsets[l] / kIndexGroupSize) * gb;
    iptr[l] = ids_arena.as<int64_t>() + h_row_offsets[l];
  }
  CUVS_HIP_TRY(hipMemcpyAsync(data_ptrs.ptr, dptr.data(), sizeof(void*) * n_lists,
                              hipMemcpyHostToDevice, stream));
  CUVS_HIP_TRY(hipMemcpyAsync(inds_ptrs.ptr, iptr.data(), sizeof(void*) * n_lists,
                              hipMemcpyHostToDevice, stream));
  CUVS_HIP_TRY(hipMemcpyAsync(list_sizes.ptr, h_list_sizes.data(), sizeof(uint32_t) * n_lists,
                              hipMemcpyHostToDevice, stream));
  std::vector<uint32_t> by_size(n_lists), rank(n_lists);
  for (uint32_t l = 0; l < n_lists; l++) { by_size[l] = l; }
  std::stable_sort(by_size.begin(), by_size.end(),
                   [&](uint32_t a, uint32_t b) { return h_list_sizes[a] > h_list_sizes[b]; });
  for (uint32_t i = 0; i < n_lists; i++) { rank[by_size[i]] = i; }
  if (list_rank.bytes != sizeof(uint32_t) * n_lists) { list_rank.allocate(sizeof(uint32_t) * n_lists); }
  CUVS_HIP_TRY(hipMemcpyAsync(list_rank.ptr, rank.data(), sizeof(uint32_t) * n_lists,
                              hipMemcpyHostToDevice, stream));
  CUVS_HIP_TRY(hipStreamSynchronize(stream));  // the host vectors above go out of scope
  std::vector<uint32_t> sorted(h_list_sizes);
  std::sort(sorted.begin(), sorted.end(), std::greater<uint32_t>());
  accum_sorted_sizes.assign(n_lists + 1, 0);
  for (uint32_t l = 0; l < n_lists; l++) {
    accum_sorted_sizes[l + 1] = accum_sorted_sizes[l] + sorted[l];
  }
  size = accum_sorted_sizes[n_lists];
}

void index_impl::refresh_coarse(hipStream_t stream)
{
  const uint32_t l_pad = coarse_pad(n_lists);
  if (centers_t.bytes == 0) { centers_t.allocate(size_t(dim_ext) * l_pad * sizeof(float)); }
  launch_transpose_centers(centers.as<float>(), n_lists, dim_ext, centers_t.as<float>(), stream);
  const uint32_t k_pad = coarse_fast_k_pad(dim);
  if (centers_h.bytes == 0) {
    centers_h.allocate(size_t(l_pad) * k_pad * sizeof(_Float16));
    center_norms.allocate(size_t(l_pad) * sizeof(float));
  }
  if (centers_i8.bytes == 0) { centers_i8.allocate(size_t(coarse_i8_words(dim)) * l_pad * sizeof(uint32_t)); }
  launch_pack_centers_i8(centers.as<float>(), n_lists, dim, dim_ext, centers_i8.as<uint32_t>(), stream);
  device_buffer stats(16);
  launch_pack_centers_f16(centers.as<float>(), n_lists, dim, dim_ext, centers_h.as<_Float16>(),
                          center_norms.as<float>(), stats.as<uint32_t>(), stream);
  float h[4] = {0, 0, 0, 0};
  CUVS_HIP_TRY(hipMemcpyAsync(h, stats.ptr, 16, hipMemcpyDeviceToHost, stream));
  CUVS_HIP_TRY(hipStreamSynchronize(stream));
  n_max          = h[1];
  c_max          = h[2];
  coarse_fast_ok = std::isfinite(h[0]) && h[0] < 60000.0f && std::isfinite(h[1]) && std::isfinite(h[2]);
}

void index_impl::rebuild_lead_plane(hipStream_t stream)
{
  derived_stale.store(false);  // whatever was written so far is seen by the kernels below
  const uint64_t n_slots = h_row_offsets.empty() ? 0 : h_row_offsets[n_lists];
  // Buffers of the right size are written in place; others are released before their successors
  // are allocated (the copies never exist twice).  Work that still reads them ends first.
  CUVS_HIP_TRY(hipStreamSynchronize(stream));
  auto sized = [](device_buffer& b, size_t bytes) {
    if (b.bytes != bytes) {
      b = device_buffer();
      b.allocate(bytes);
    }
  };
  // how far a row of each list can lie from the list's centre
  sized(list_radius, sizeof(float) * n_lists);
  if (n_slots != 0) {
    launch_list_radius(data_ptrs.as<const uint8_t*>(), list_sizes.as<uint32_t>(), 0, n_lists, pq_dim, pq_bits, pq_len,
                       pq_centers.as<float>(), codebook_kind == codebook_gen::PER_SUBSPACE, list_radius.as<float>(),
                       stream);
  } else {
    CUVS_HIP_TRY(hipMemsetAsync(list_radius.ptr, 0, list_radius.bytes, stream));
  }
  sized(center_terms, sizeof(float4) * n_lists);
  launch_center_terms(centers.as<float>(), centers_rot.as<float>(), rotation.as<float>(), n_lists, dim, dim_ext,
                      rot_dim, rotation_is_identity && rot_dim == dim, center_terms.as<float4>(), stream);
  // narrower codes, a byte each
  const bool widen = pq_bits >= 5 && pq_bits < 8 && n_slots != 0 && !conservative_memory_allocation;
  if (widen) {
    n_chunks8                = (pq_dim + 15u) / 16u;
    const uint64_t gb8       = uint64_t(n_chunks8) * kIndexGroupSize * kIndexGroupVecLen;
    const uint64_t n_groups  = n_slots / kIndexGroupSize;
    // two groups of slack: the scan kernels read whole 64-row tiles past a list's last group
    sized(codes8_arena, (n_groups + 2) * gb8);
    CUVS_HIP_TRY(hipMemsetAsync(codes8_arena.ptr, 0, codes8_arena.bytes, stream));
    launch_widen_codes(codes_arena.as<uint8_t>(), codes8_arena.as<uint8_t>(), n_slots, pq_dim, pq_bits, n_chunks,
                       n_chunks8, stream);
    std::vector<uint8_t*> dptr(n_lists);
    for (uint32_t l = 0; l < n_lists; l++) {
      dptr[l] = codes8_arena.as<uint8_t>() + (h_row_offsets[l] / kIndexGroupSize) * gb8;
    }
    sized(data_ptrs8, sizeof(void*) * n_lists);
    CUVS_HIP_TRY(hipMemcpyAsync(data_ptrs8.ptr, dptr.data(), data_ptrs8.bytes, hipMemcpyHostToDevice, stream));
    const uint64_t book_rows = pq_centers.bytes / (sizeof(float) * book_size);
    sized(pq_centers8, book_rows * 256 * sizeof(float));
    launch_pad_codebooks(pq_centers.as<float>(), pq_centers8.as<float>(), book_rows, book_size, stream);
    CUVS_HIP_TRY(hipStreamSynchronize(stream));  // `dptr` goes out of scope
  } else {
    codes8_arena = device_buffer();
    data_ptrs8   = device_buffer();
    pq_centers8  = device_buffer();
    n_chunks8    = 0;
  }
  derived_offsets = h_row_offsets;
  // byte codes (as stored or widened), and nibble codes unless memory is to be spared: the plane
  // is what lets an L2 search of either width screen pairs without scanning them
  const bool plane_codes = pq_bits == 8 || widen || (pq_bits == 4 && !conservative_memory_allocation);
  if (!plane_codes || n_slots == 0 || n_slots + kLeadPlaneSlack > 0xFFFFFFFFull) {
    lead_plane = device_buffer();
    return;
  }
  sized(lead_plane, (n_slots + kLeadPlaneSlack) * sizeof(uint64_t));
  CUVS_HIP_TRY(hipMemsetAsync(lead_plane.ptr, 0, lead_plane.bytes, stream));
  launch_build_lead_plane(widen ? codes8_arena.as<uint8_t>() : codes_arena.as<uint8_t>(), lead_plane.as<uint64_t>(), n_slots,
                          widen ? n_chunks8 : n_chunks, stream);
}

void index_impl::refresh_derived_rows(uint32_t label, hipStream_t stream)
{
  // The copies follow the lists where they are now only if no list has moved since they were made
  // (an edit that outgrows a list's padding moves the arenas); and a write through a bare pointer
  // may have touched any list.
  if (derived_stale.load() || derived_offsets != h_row_offsets) {
    rebuild_lead_plane(stream);
    return;
  }
  const uint64_t begin = h_row_offsets[label], end = h_row_offsets[label + 1];  // whole groups of 32 rows
  launch_list_radius(data_ptrs.as<const uint8_t*>(), list_sizes.as<uint32_t>(), label, 1, pq_dim, pq_bits, pq_len,
                     pq_centers.as<float>(), codebook_kind == codebook_gen::PER_SUBSPACE, list_radius.as<float>(),
                     stream);
  if (begin == end) { return; }
  const bool widen       = codes8_arena.bytes != 0;
  const uint64_t gb      = uint64_t(n_chunks) * kIndexGroupSize * kIndexGroupVecLen;
  const uint64_t gb8     = uint64_t(n_chunks8) * kIndexGroupSize * kIndexGroupVecLen;
  const uint64_t group   = begin / kIndexGroupSize;
  const uint8_t* packed  = codes_arena.as<uint8_t>() + group * gb;
  if (widen) {
    launch_widen_codes(packed, codes8_arena.as<uint8_t>() + group * gb8, end - begin, pq_dim, pq_bits, n_chunks, n_chunks8,
                       stream);
  }
  if (lead_plane.bytes != 0) {
    launch_build_lead_plane(widen ? codes8_arena.as<uint8_t>() + group * gb8 : packed, lead_plane.as<uint64_t>() + begin,
                            end - begin, widen ? n_chunks8 : n_chunks, stream);
  }
}

}  // namespace detail

template <typename IdxT>
index<IdxT>::index() : impl_(new detail::index_impl())
{
}
template <typename IdxT>
index<IdxT>::~index() = default;
template <typename IdxT>
index<IdxT>::index(index&&) noexcept = default;
template <typename IdxT>
index<IdxT>& index<IdxT>::operator=(index&&) noexcept = default;

#define IMPL_GETTER(type, name, expr)    \
  template <typename IdxT>               \
  type index<IdxT>::name() const         \
  {                                      \
    return expr;                         \
  }

IMPL_GETTER(int64_t, size, impl_->size)
IMPL_GETTER(uint32_t, dim, impl_->dim)
IMPL_GETTER(uint32_t, dim_ext, impl_->dim_ext)
IMPL_GETTER(uint32_t, rot_dim, impl_->rot_dim)
IMPL_GETTER(uint32_t, pq_bits, impl_->pq_bits)
IMPL_GETTER(uint32_t, pq_dim, impl_->pq_dim)
IMPL_GETTER(uint32_t, pq_len, impl_->pq_len)
IMPL_GETTER(uint32_t, pq_book_size, impl_->book_size)
IMPL_GETTER(uint32_t, n_lists, impl_->n_lists)
IMPL_GETTER(cuvs::distance::DistanceType, metric, impl_->metric)
IMPL_GETTER(codebook_gen, codebook_kind, impl_->codebook_kind)
IMPL_GETTER(list_layout, codes_layout, list_layout::INTERLEAVED)
IMPL_GETTER(bool, conservative_memory_allocation, impl_->conservative_memory_allocation)
IMPL_GETTER(const float*, centers, impl_->centers.template as<float>())
IMPL_GETTER(const float*, centers_rot, impl_->centers_rot.template as<float>())
IMPL_GETTER(const float*, rotation_matrix, impl_->rotation.template as<float>())
IMPL_GETTER(const float*, pq_centers, impl_->pq_centers.template as<float>())
IMPL_GETTER(const uint32_t*, list_sizes, impl_->list_sizes.template as<uint32_t>())
IMPL_GETTER(const uint8_t* const*, data_ptrs, impl_->data_ptrs.template as<const uint8_t*>())
IMPL_GETTER(const IdxT* const*, inds_ptrs, impl_->inds_ptrs.template as<const IdxT*>())
IMPL_GETTER(const int64_t*, accum_sorted_sizes, impl_->accum_sorted_sizes.data())

template class index<int64_t>;

index<int64_t> build(cuvs::resources const& res,
                     const index_params& params,
                     uint32_t dim,
                     const float* pq_centers,
                     const float* centers,
                     const float* centers_rot,
                     const float* rotation_matrix)
{
  CUVS_EXPECTS(params.codes_layout == list_layout::INTERLEAVED,
               "only the INTERLEAVED codes layout is supported");
  CUVS_EXPECTS(pq_centers != nullptr && centers != nullptr && centers_rot != nullptr &&
                 rotation_matrix != nullptr,
               "model tensors must not be null");
  index<int64_t> idx;
  auto& ix = *idx.impl();
  detail::init_index(ix, params, dim);
  hipStream_t stream = res.stream();
  const size_t n_books =
    ix.codebook_kind == codebook_gen::PER_SUBSPACE ? ix.pq_dim : ix.n_lists;
  auto copy_in = [&](device_buffer& dst, const float* src, size_t n) {
    dst.allocate(n * sizeof(float));
    CUVS_HIP_TRY(hipMemcpyAsync(dst.ptr, src, n * sizeof(float), hipMemcpyDefault, stream));
  };
  copy_in(ix.pq_centers, pq_centers, n_books * ix.pq_len * ix.book_size);
  copy_in(ix.centers, centers, size_t(ix.n_lists) * ix.dim_ext);
  copy_in(ix.centers_rot, centers_rot, size_t(ix.n_lists) * ix.rot_dim);
  ix.refresh_coarse(stream);
  copy_in(ix.rotation, rotation_matrix, size_t(ix.rot_dim) * ix.dim);

  // transposed copy [dim, rot_dim] for coalesced reads, and the identity check
  std::vector<float> rot(size_t(ix.rot_dim) * ix.dim), rot_t(size_t(ix.rot_dim) * ix.dim);
  CUVS_HIP_TRY(hipMemcpyAsync(rot.data(), rotation_matrix, rot.size() * sizeof(float),
                              hipMemcpyDefault, stream));
  CUVS_HIP_TRY(hipStreamSynchronize(stream));
  bool identity = ix.rot_dim == ix.dim;
  for (uint32_t r = 0; r < ix.rot_dim; r++) {
    for (uint32_t d = 0; d < ix.dim; d++) {
      const float v               = rot[size_t(r) * ix.dim + d];
      rot_t[size_t(d) * ix.rot_dim + r] = v;
      if (v != (r == d ? 1.0f : 0.0f)) { identity = false; }
    }
  }
  ix.rotation_is_identity = identity;
  {
    double longest = 0.0;
    for (uint32_t r = 0; r < ix.rot_dim; r++) {
      double n2 = 0.0;
      for (uint32_t d = 0; d < ix.dim; d++) { n2 += double(rot[size_t(r) * ix.dim + d]) * rot[size_t(r) * ix.dim + d]; }
      longest = std::max(longest, n2);
    }
    ix.rotation_bounded = longest <= 4.0;  // false for a NaN as well
  }
  ix.rotation_t.allocate(rot_t.size() * sizeof(float));
  CUVS_HIP_TRY(hipMemcpyAsync(ix.rotation_t.ptr, rot_t.data(), rot_t.size() * sizeof(float),
                              hipMemcpyHostToDevice, stream));
  ix.recompute_internal_state(stream);
  return idx;
}

index<int64_t> clone(cuvs::resources const& res, const index<int64_t>& source)
{
  CUVS_EXPECTS(source.impl() != nullptr, "index must not be null");
  const auto& src = *source.impl();
  index<int64_t> out;
  auto& dst          = *out.impl();
  hipStream_t stream = res.stream();
  auto copy          = [&](device_buffer& to, const device_buffer& from) {
    to.allocate(from.bytes);
    if (from.bytes > 0) {
      CUVS_HIP_TRY(hipMemcpyAsync(to.ptr, from.ptr, from.bytes, hipMemcpyDeviceToDevice, stream));
    }
  };
  dst.metric                         = src.metric;
  dst.codebook_kind                  = src.codebook_kind;
  dst.conservative_memory_allocation = src.conservative_memory_allocation;
  dst.n_lists                        = src.n_lists;
  dst.dim                            = src.dim;
  dst.pq_bits                        = src.pq_bits;
  dst.pq_dim                         = src.pq_dim;
  dst.dim_ext                        = src.dim_ext;
  dst.pq_len                         = src.pq_len;
  dst.rot_dim                        = src.rot_dim;
  dst.book_size                      = src.book_size;
  dst.n_chunks                       = src.n_chunks;
  dst.c_max                          = src.c_max;
  dst.n_max                          = src.n_max;
  dst.coarse_fast_ok                 = src.coarse_fast_ok;
  dst.rotation_is_identity           = src.rotation_is_identity;
  dst.rotation_bounded               = src.rotation_bounded;
  dst.feedback.create();
  copy(dst.centers, src.centers);
  copy(dst.centers_rot, src.centers_rot);
  copy(dst.rotation, src.rotation);
  copy(dst.rotation_t, src.rotation_t);
  copy(dst.pq_centers, src.pq_centers);
  copy(dst.centers_t, src.centers_t);
  copy(dst.centers_h, src.centers_h);
  copy(dst.center_norms, src.center_norms);
  copy(dst.centers_i8, src.centers_i8);
  copy(dst.codes_arena, src.codes_arena);
  copy(dst.ids_arena, src.ids_arena);
  dst.h_list_sizes  = src.h_list_sizes;
  dst.h_row_offsets = src.h_row_offsets;
  dst.list_sizes.allocate(sizeof(uint32_t) * dst.n_lists);
  dst.data_ptrs.allocate(sizeof(void*) * dst.n_lists);
  dst.inds_ptrs.allocate(sizeof(void*) * dst.n_lists);
  dst.recompute_internal_state(stream);  // the tables point into the copy's own arenas; synchronises
  dst.rebuild_lead_plane(stream);
  return out;
}

void unpack_contiguous_list_data(cuvs::resources const& res,
                                 const index<int64_t>& idx,
                                 uint8_t* out_codes,
                                 uint32_t n_rows,
                                 uint32_t label,
                                 uint32_t offset)
{
  const auto& ix = *idx.impl();
  CUVS_EXPECTS(label < ix.n_lists, "label (%u) must be smaller than n_lists (%u)", label, ix.n_lists);
  CUVS_EXPECTS(uint64_t(offset) + n_rows <= ix.h_list_sizes[label],
               "offset + n_rows (%u + %u) must not exceed the list size (%u)", offset, n_rows,
               ix.h_list_sizes[label]);
  const uint8_t* data = ix.codes_arena.as<uint8_t>() +
                        (ix.h_row_offsets[label] / kIndexGroupSize) * ix.group_bytes();
  detail::launch_unpack_contiguous(data, n_rows, offset, ix.pq_dim, ix.pq_bits, out_codes,
                                   res.stream());
}

}  // namespace cuvs::neighbors::ivf_pq
