/*
 * Reading and editing single lists of an index: the helpers of cuVS' ivf_pq::helpers namespace
 * (cpp/src/neighbors/ivf_pq/ivf_pq_build_common.cu:20-232, ivf_pq_build.cuh:594-690,852-960,
 * 1668-1687).  The lists of an index live back to back in two arenas, so a list that outgrows the
 * padding of its last 32-row group moves every list behind it: appending to single lists costs a
 * copy of the arenas, which is what keeps the search's address stream dense.
 */
#include "detail.hpp"

#include <type_traits>

namespace cuvs::neighbors::ivf_pq {

void encode_for_list(cuvs::resources const& res, const index<int64_t>& idx, const void* vectors,
                     elem_type type, int64_t n_rows, uint32_t label, uint8_t* codes_out);

namespace helpers {

namespace {

using detail::index_impl;

index_impl& checked(index<int64_t>* idx, uint32_t label)
{
  CUVS_EXPECTS(idx != nullptr && idx->impl() != nullptr, "index must not be null");
  index_impl& ix = *idx->impl();
  CUVS_EXPECTS(label < ix.n_lists, "label (%u) must be smaller than n_lists (%u)", label, ix.n_lists);
  return ix;
}

const index_impl& checked(const index<int64_t>& idx, uint32_t label)
{
  CUVS_EXPECTS(idx.impl() != nullptr, "index must not be null");
  const index_impl& ix = *idx.impl();
  CUVS_EXPECTS(label < ix.n_lists, "label (%u) must be smaller than n_lists (%u)", label, ix.n_lists);
  return ix;
}

uint8_t* list_codes(const index_impl& ix, uint32_t label)
{
  return ix.codes_arena.as<uint8_t>() + (ix.h_row_offsets[label] / kIndexGroupSize) * ix.group_bytes();
}

void expect_range(const index_impl& ix, uint32_t label, uint32_t offset, int64_t n_rows)
{
  CUVS_EXPECTS(n_rows >= 0 && uint64_t(offset) + uint64_t(n_rows) <= ix.h_list_sizes[label],
               "offset + number of rows (%u + %lld) must not exceed the list size (%u)", offset,
               static_cast<long long>(n_rows), ix.h_list_sizes[label]);
}

template <typename T>
elem_type elem_of()
{
  if (std::is_same<T, _Float16>::value) { return elem_type::f16; }
  if (std::is_same<T, int8_t>::value) { return elem_type::i8; }
  if (std::is_same<T, uint8_t>::value) { return elem_type::u8; }
  return elem_type::f32;
}

void reconstruct(cuvs::resources const& res, const index_impl& ix, void* out, elem_type type,
                 int64_t n_rows, int64_t out_dim, uint32_t label, uint32_t offset, const uint32_t* rows)
{
  if (n_rows == 0) { return; }
  CUVS_EXPECTS(out != nullptr, "out_vectors must not be null");
  CUVS_EXPECTS(out_dim == int64_t(ix.dim), "out_vectors must have the index's dimension (%u)", ix.dim);
  CUVS_EXPECTS(n_rows <= int64_t(ix.h_list_sizes[label]), "more rows asked for than the list holds");
  hipStream_t s = res.stream();
  const bool per_subspace = ix.codebook_kind == codebook_gen::PER_SUBSPACE;
  const float* book = ix.pq_centers.as<float>() +
                      (per_subspace ? 0 : uint64_t(label) * ix.pq_len * ix.book_size);
  device_buffer rot(uint64_t(n_rows) * ix.rot_dim * sizeof(float));
  detail::launch_reconstruct_rot(list_codes(ix, label), uint32_t(n_rows), offset, rows, ix.pq_dim,
                                 ix.pq_bits, ix.pq_len, book, per_subspace,
                                 ix.centers_rot.as<float>() + uint64_t(label) * ix.rot_dim,
                                 rot.as<float>(), s);
  // back to the original space: x = R^T y.  The rotation kernel computes out[c] = sum_r M[r][c] in[r]
  // for M stored [in, out]; the rotation matrix itself ([rot_dim, dim]) is that M here.
  device_buffer flat;
  float* xf = static_cast<float*>(out);
  if (type != elem_type::f32) {
    flat.allocate(uint64_t(n_rows) * ix.dim * sizeof(float));
    xf = flat.as<float>();
  }
  detail::launch_rotate(rot.as<float>(), ix.rotation.as<float>(), uint32_t(n_rows), ix.rot_dim, ix.dim,
                        false, false, CUDA_R_32F, xf, s);
  if (type != elem_type::f32) { detail::launch_unmap_rows(xf, uint64_t(n_rows) * ix.dim, type, out, s); }
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // the temporaries go out of scope
}

/** Makes room for `n_rows` more rows in list `label`, writes their source indices, and returns the
 *  position of the first (cuVS extend_list_prepare, ivf_pq_build.cuh:852-886). */
uint32_t extend_list_prepare(cuvs::resources const& res, index_impl& ix, const int64_t* new_indices,
                             int64_t n_rows, uint32_t label)
{
  hipStream_t s         = res.stream();
  const uint32_t offset = ix.h_list_sizes[label];
  const uint64_t grown  = uint64_t(offset) + uint64_t(n_rows);
  CUVS_EXPECTS(grown <= 0xFFFFFFFFull, "list %u would exceed 2^32 rows", label);
  const uint64_t room = ix.h_row_offsets[label + 1] - ix.h_row_offsets[label];
  if (grown <= room && ix.codes_arena.ptr != nullptr) {
    // the padding of the list's last group takes the rows: nothing moves
    ix.h_list_sizes[label] = uint32_t(grown);
    ix.recompute_internal_state(s);
  } else {
    std::vector<uint32_t> sizes(ix.h_list_sizes);
    sizes[label] = uint32_t(grown);
    detail::relayout_lists(res, ix, sizes);
  }
  CUVS_HIP_TRY(hipMemcpyAsync(ix.ids_arena.as<int64_t>() + ix.h_row_offsets[label] + offset, new_indices,
                              uint64_t(n_rows) * sizeof(int64_t), hipMemcpyDefault, s));
  return offset;
}

constexpr uint32_t kAllLists = 0xFFFFFFFFu;
/** The index's derived copies of the list codes follow an edit: of one list, or of everything. */
void finish_edit(cuvs::resources const& res, index_impl& ix, uint32_t label = kAllLists)
{
  if (label == kAllLists) {
    ix.rebuild_lead_plane(res.stream());
  } else {
    ix.refresh_derived_rows(label, res.stream());
  }
  CUVS_HIP_TRY(hipStreamSynchronize(res.stream()));
}

}  // namespace

namespace codepacker {

void unpack(cuvs::resources const& res, const uint8_t* list_data, uint32_t pq_bits, uint32_t offset,
            device_matrix_view<uint8_t> codes)
{
  CUVS_EXPECTS(pq_bits >= 4 && pq_bits <= 8, "pq_bits must be within [4, 8], got %u", pq_bits);
  CUVS_EXPECTS(list_data != nullptr || codes.extent(0) == 0, "list_data is null");
  if (codes.extent(0) == 0) { return; }
  detail::launch_unpack_codes(list_data, uint32_t(codes.extent(0)), offset, nullptr, uint32_t(codes.extent(1)),
                              pq_bits, codes.data_handle(), res.stream());
}

void pack(cuvs::resources const& res, device_matrix_view<const uint8_t> codes, uint32_t pq_bits,
          uint32_t offset, uint8_t* list_data)
{
  CUVS_EXPECTS(pq_bits >= 4 && pq_bits <= 8, "pq_bits must be within [4, 8], got %u", pq_bits);
  CUVS_EXPECTS(list_data != nullptr || codes.extent(0) == 0, "list_data is null");
  if (codes.extent(0) == 0) { return; }
  detail::launch_pack_codes(list_data, codes.data_handle(), false, uint32_t(codes.extent(0)), offset,
                            uint32_t(codes.extent(1)), pq_bits, res.stream());
  detail::mark_lists_written(list_data);
}

void unpack_contiguous(cuvs::resources const& res, const uint8_t* list_data, uint32_t pq_bits, uint32_t offset,
                       uint32_t n_rows, uint32_t pq_dim, uint8_t* codes)
{
  CUVS_EXPECTS(pq_bits >= 4 && pq_bits <= 8, "pq_bits must be within [4, 8], got %u", pq_bits);
  CUVS_EXPECTS(pq_dim > 0, "pq_dim must be positive");
  if (n_rows == 0) { return; }
  CUVS_EXPECTS(list_data != nullptr && codes != nullptr, "list_data and codes must not be null");
  detail::launch_unpack_contiguous(list_data, n_rows, offset, pq_dim, pq_bits, codes, res.stream());
}

void pack_contiguous(cuvs::resources const& res, const uint8_t* codes, uint32_t n_rows, uint32_t pq_dim,
                     uint32_t pq_bits, uint32_t offset, uint8_t* list_data)
{
  CUVS_EXPECTS(pq_bits >= 4 && pq_bits <= 8, "pq_bits must be within [4, 8], got %u", pq_bits);
  CUVS_EXPECTS(pq_dim > 0, "pq_dim must be positive");
  if (n_rows == 0) { return; }
  CUVS_EXPECTS(list_data != nullptr && codes != nullptr, "list_data and codes must not be null");
  detail::launch_pack_codes(list_data, codes, true, n_rows, offset, pq_dim, pq_bits, res.stream());
  detail::mark_lists_written(list_data);
}

void unpack_list_data(cuvs::resources const& res, const index<int64_t>& idx,
                      device_matrix_view<uint8_t> out_codes, uint32_t label, uint32_t offset)
{
  const index_impl& ix = checked(idx, label);
  if (out_codes.extent(0) == 0) { return; }
  CUVS_EXPECTS(out_codes.extent(1) == int64_t(ix.pq_dim), "out_codes must have pq_dim (%u) columns", ix.pq_dim);
  expect_range(ix, label, offset, out_codes.extent(0));
  detail::launch_unpack_codes(list_codes(ix, label), uint32_t(out_codes.extent(0)), offset, nullptr,
                              ix.pq_dim, ix.pq_bits, out_codes.data_handle(), res.stream());
}

void unpack_list_data(cuvs::resources const& res, const index<int64_t>& idx,
                      device_vector_view<const uint32_t> in_cluster_indices,
                      device_matrix_view<uint8_t> out_codes, uint32_t label)
{
  const index_impl& ix = checked(idx, label);
  if (out_codes.extent(0) == 0) { return; }
  CUVS_EXPECTS(out_codes.extent(1) == int64_t(ix.pq_dim), "out_codes must have pq_dim (%u) columns", ix.pq_dim);
  CUVS_EXPECTS(in_cluster_indices.extent(0) == out_codes.extent(0),
               "one position per output row is needed");
  detail::launch_unpack_codes(list_codes(ix, label), uint32_t(out_codes.extent(0)), 0,
                              in_cluster_indices.data_handle(), ix.pq_dim, ix.pq_bits,
                              out_codes.data_handle(), res.stream());
}

void unpack_contiguous_list_data(cuvs::resources const& res, const index<int64_t>& idx, uint8_t* out_codes,
                                 uint32_t n_rows, uint32_t label, uint32_t offset)
{
  cuvs::neighbors::ivf_pq::unpack_contiguous_list_data(res, idx, out_codes, n_rows, label, offset);
}

void pack_list_data(cuvs::resources const& res, index<int64_t>* idx,
                    device_matrix_view<const uint8_t> new_codes, uint32_t label, uint32_t offset)
{
  index_impl& ix = checked(idx, label);
  if (new_codes.extent(0) == 0) { return; }
  CUVS_EXPECTS(new_codes.extent(1) == int64_t(ix.pq_dim), "new_codes must have pq_dim (%u) columns", ix.pq_dim);
  expect_range(ix, label, offset, new_codes.extent(0));
  detail::launch_pack_codes(list_codes(ix, label), new_codes.data_handle(), false,
                            uint32_t(new_codes.extent(0)), offset, ix.pq_dim, ix.pq_bits, res.stream());
  finish_edit(res, ix, label);
}

void pack_contiguous_list_data(cuvs::resources const& res, index<int64_t>* idx, const uint8_t* new_codes,
                               uint32_t n_rows, uint32_t label, uint32_t offset)
{
  index_impl& ix = checked(idx, label);
  if (n_rows == 0) { return; }
  CUVS_EXPECTS(new_codes != nullptr, "new_codes must not be null");
  expect_range(ix, label, offset, n_rows);
  detail::launch_pack_codes(list_codes(ix, label), new_codes, true, n_rows, offset, ix.pq_dim, ix.pq_bits,
                            res.stream());
  finish_edit(res, ix, label);
}

template <typename T>
void reconstruct_list_data(cuvs::resources const& res, const index<int64_t>& idx,
                           device_matrix_view<T> out_vectors, uint32_t label, uint32_t offset)
{
  const index_impl& ix = checked(idx, label);
  expect_range(ix, label, offset, out_vectors.extent(0));
  reconstruct(res, ix, out_vectors.data_handle(), elem_of<T>(), out_vectors.extent(0),
              out_vectors.extent(1), label, offset, nullptr);
}

template <typename T>
void reconstruct_list_data(cuvs::resources const& res, const index<int64_t>& idx,
                           device_vector_view<const uint32_t> in_cluster_indices,
                           device_matrix_view<T> out_vectors, uint32_t label)
{
  const index_impl& ix = checked(idx, label);
  CUVS_EXPECTS(in_cluster_indices.extent(0) == out_vectors.extent(0),
               "one position per output row is needed");
  reconstruct(res, ix, out_vectors.data_handle(), elem_of<T>(), out_vectors.extent(0),
              out_vectors.extent(1), label, 0, in_cluster_indices.data_handle());
}

#define CUVS_INSTANTIATE_RECONSTRUCT(T)                                                              \
  template void reconstruct_list_data<T>(cuvs::resources const&, const index<int64_t>&,              \
                                         device_matrix_view<T>, uint32_t, uint32_t);                 \
  template void reconstruct_list_data<T>(cuvs::resources const&, const index<int64_t>&,              \
                                         device_vector_view<const uint32_t>, device_matrix_view<T>,  \
                                         uint32_t);
CUVS_INSTANTIATE_RECONSTRUCT(float)
CUVS_INSTANTIATE_RECONSTRUCT(_Float16)
CUVS_INSTANTIATE_RECONSTRUCT(int8_t)
CUVS_INSTANTIATE_RECONSTRUCT(uint8_t)
#undef CUVS_INSTANTIATE_RECONSTRUCT

void extend_list_with_codes(cuvs::resources const& res, index<int64_t>* idx,
                            device_matrix_view<const uint8_t> new_codes,
                            device_vector_view<const int64_t> new_indices, uint32_t label)
{
  index_impl& ix = checked(idx, label);
  CUVS_EXPECTS(new_codes.extent(0) == new_indices.extent(0), "one source index per row is needed");
  if (new_codes.extent(0) == 0) { return; }
  CUVS_EXPECTS(new_codes.extent(1) == int64_t(ix.pq_dim), "new_codes must have pq_dim (%u) columns", ix.pq_dim);
  const uint32_t offset = extend_list_prepare(res, ix, new_indices.data_handle(), new_codes.extent(0), label);
  detail::launch_pack_codes(list_codes(ix, label), new_codes.data_handle(), false,
                            uint32_t(new_codes.extent(0)), offset, ix.pq_dim, ix.pq_bits, res.stream());
  finish_edit(res, ix, label);
}

void extend_list_with_contiguous_codes(cuvs::resources const& res, index<int64_t>* idx,
                                       device_matrix_view<const uint8_t> new_codes,
                                       device_vector_view<const int64_t> new_indices, uint32_t label)
{
  index_impl& ix = checked(idx, label);
  CUVS_EXPECTS(new_codes.extent(0) == new_indices.extent(0), "one source index per row is needed");
  if (new_codes.extent(0) == 0) { return; }
  const uint32_t row_bytes = (ix.pq_dim * ix.pq_bits + 7) / 8;
  CUVS_EXPECTS(new_codes.extent(1) == int64_t(row_bytes), "new_codes must have %u bytes per row", row_bytes);
  const uint32_t offset = extend_list_prepare(res, ix, new_indices.data_handle(), new_codes.extent(0), label);
  detail::launch_pack_codes(list_codes(ix, label), new_codes.data_handle(), true,
                            uint32_t(new_codes.extent(0)), offset, ix.pq_dim, ix.pq_bits, res.stream());
  finish_edit(res, ix, label);
}

template <typename T>
void extend_list(cuvs::resources const& res, index<int64_t>* idx, device_matrix_view<const T> new_vectors,
                 device_vector_view<const int64_t> new_indices, uint32_t label)
{
  index_impl& ix = checked(idx, label);
  CUVS_EXPECTS(new_vectors.extent(0) == new_indices.extent(0), "one source index per row is needed");
  if (new_vectors.extent(0) == 0) { return; }
  CUVS_EXPECTS(new_vectors.extent(1) == int64_t(ix.dim), "new_vectors must have the index's dimension (%u)", ix.dim);
  const int64_t n          = new_vectors.extent(0);
  const uint32_t row_bytes = (ix.pq_dim * ix.pq_bits + 7) / 8;
  device_buffer codes(uint64_t(n) * row_bytes);
  encode_for_list(res, *idx, new_vectors.data_handle(), elem_of<T>(), n, label, codes.as<uint8_t>());
  const uint32_t offset = extend_list_prepare(res, ix, new_indices.data_handle(), n, label);
  detail::launch_pack_codes(list_codes(ix, label), codes.as<uint8_t>(), true, uint32_t(n), offset,
                            ix.pq_dim, ix.pq_bits, res.stream());
  finish_edit(res, ix, label);
}

#define CUVS_INSTANTIATE_EXTEND_LIST(T)                                                                  \
  template void extend_list<T>(cuvs::resources const&, index<int64_t>*, device_matrix_view<const T>,     \
                               device_vector_view<const int64_t>, uint32_t);
CUVS_INSTANTIATE_EXTEND_LIST(float)
CUVS_INSTANTIATE_EXTEND_LIST(_Float16)
CUVS_INSTANTIATE_EXTEND_LIST(int8_t)
CUVS_INSTANTIATE_EXTEND_LIST(uint8_t)
#undef CUVS_INSTANTIATE_EXTEND_LIST

}  // namespace codepacker

void erase_list(cuvs::resources const& res, index<int64_t>* idx, uint32_t label)
{
  index_impl& ix = checked(idx, label);
  if (ix.h_list_sizes[label] == 0) { return; }
  hipStream_t s = res.stream();
  // the move below copies as many rows of each list as the device-side sizes say: none of this one
  detail::launch_fill_u32(ix.list_sizes.as<uint32_t>() + label, 0, 1, s);
  ix.h_list_sizes[label] = 0;
  detail::relayout_lists(res, ix, std::vector<uint32_t>(ix.h_list_sizes));
  finish_edit(res, ix);
}

void resize_list(cuvs::resources const& res, index<int64_t>* idx, uint32_t label, uint32_t new_used_size)
{
  index_impl& ix      = checked(idx, label);
  const uint32_t old  = ix.h_list_sizes[label];
  if (new_used_size == old) { return; }
  hipStream_t s = res.stream();
  // the move copies as many rows of each list as the device-side sizes say: min(old, new) of this one
  if (new_used_size < old) { detail::launch_fill_u32(ix.list_sizes.as<uint32_t>() + label, new_used_size, 1, s); }
  std::vector<uint32_t> sizes(ix.h_list_sizes);
  ix.h_list_sizes[label] = std::min(old, new_used_size);
  sizes[label]           = new_used_size;
  detail::relayout_lists(res, ix, sizes);
  // the move copies whole groups of 32 rows: what a smaller size leaves behind in the last group
  // is cleared, so that slots past a list's end hold zero codes as everywhere else
  const uint32_t n_pad = round_up_u32(new_used_size, kIndexGroupSize) - new_used_size;
  if (new_used_size < old && n_pad != 0) {
    device_buffer zeros(size_t(n_pad) * ix.pq_dim);
    CUVS_HIP_TRY(hipMemsetAsync(zeros.ptr, 0, zeros.bytes, s));
    detail::launch_pack_codes(list_codes(ix, label), zeros.as<uint8_t>(), false, n_pad, new_used_size, ix.pq_dim,
                              ix.pq_bits, s);
    CUVS_HIP_TRY(hipStreamSynchronize(s));  // `zeros` goes out of scope
  }
  finish_edit(res, ix);
}

void reset_index(cuvs::resources const& res, index<int64_t>* idx)
{
  CUVS_EXPECTS(idx != nullptr && idx->impl() != nullptr, "index must not be null");
  index_impl& ix = *idx->impl();
  hipStream_t s  = res.stream();
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // the arenas are released below
  ix.codes_arena = device_buffer();
  ix.ids_arena   = device_buffer();
  ix.h_list_sizes.assign(ix.n_lists, 0);
  ix.h_row_offsets.assign(ix.n_lists + 1, 0);
  ix.recompute_internal_state(s);
  finish_edit(res, ix);
}

void extract_centers(cuvs::resources const& res, const index<int64_t>& idx, float* cluster_centers)
{
  CUVS_EXPECTS(idx.impl() != nullptr && cluster_centers != nullptr, "index and output must not be null");
  const index_impl& ix = *idx.impl();
  CUVS_HIP_TRY(hipMemcpy2DAsync(cluster_centers, size_t(ix.dim) * sizeof(float), ix.centers.ptr,
                                size_t(ix.dim_ext) * sizeof(float), size_t(ix.dim) * sizeof(float),
                                ix.n_lists, hipMemcpyDefault, res.stream()));
}

void pad_centers_with_norms(cuvs::resources const& res, device_matrix_view<const float> centers,
                            device_matrix_view<float> padded_centers)
{
  const int64_t n = centers.extent(0), dim = centers.extent(1), dim_ext = padded_centers.extent(1);
  CUVS_EXPECTS(padded_centers.extent(0) == n, "centers and padded_centers must have the same number of rows");
  CUVS_EXPECTS(dim > 0 && dim_ext > dim, "padded_centers needs at least one column more than centers");
  if (n == 0) { return; }
  hipStream_t s    = res.stream();
  const float* src = centers.data_handle();
  device_buffer stage;
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, src) != hipSuccess || attr.type == hipMemoryTypeUnregistered) {
    (void)hipGetLastError();
    stage.allocate(size_t(n) * dim * sizeof(float));
    CUVS_HIP_TRY(hipMemcpyAsync(stage.ptr, src, stage.bytes, hipMemcpyHostToDevice, s));
    src = stage.as<float>();
  }
  detail::launch_set_centers(src, uint32_t(n), uint32_t(dim), uint32_t(dim_ext), padded_centers.data_handle(), s);
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // the staging copy goes out of scope
}

void rotate_padded_centers(cuvs::resources const& res, device_matrix_view<const float> padded_centers,
                           device_matrix_view<const float> rotation_matrix,
                           device_matrix_view<float> rotated_centers)
{
  const int64_t n = padded_centers.extent(0), dim_ext = padded_centers.extent(1);
  const int64_t rot_dim = rotation_matrix.extent(0), dim = rotation_matrix.extent(1);
  CUVS_EXPECTS(rotated_centers.extent(0) == n && rotated_centers.extent(1) == rot_dim,
               "rotated_centers must be [n_centers, rot_dim]");
  CUVS_EXPECTS(dim_ext > dim, "padded_centers must be wider than the rotation matrix's dim");
  if (n == 0) { return; }
  hipStream_t s = res.stream();
  // the rows without their padding, then the rotation applied to each: y = R x
  device_buffer flat(size_t(n) * dim * sizeof(float)), rot_t(size_t(rot_dim) * dim * sizeof(float));
  CUVS_HIP_TRY(hipMemcpy2DAsync(flat.ptr, size_t(dim) * sizeof(float), padded_centers.data_handle(),
                                size_t(dim_ext) * sizeof(float), size_t(dim) * sizeof(float), size_t(n),
                                hipMemcpyDeviceToDevice, s));
  std::vector<float> r(size_t(rot_dim) * dim), rt(size_t(rot_dim) * dim);
  CUVS_HIP_TRY(hipMemcpyAsync(r.data(), rotation_matrix.data_handle(), r.size() * sizeof(float),
                              hipMemcpyDefault, s));
  CUVS_HIP_TRY(hipStreamSynchronize(s));
  for (int64_t o = 0; o < rot_dim; o++) {
    for (int64_t d = 0; d < dim; d++) { rt[size_t(d) * rot_dim + o] = r[size_t(o) * dim + d]; }
  }
  CUVS_HIP_TRY(hipMemcpyAsync(rot_t.ptr, rt.data(), rt.size() * sizeof(float), hipMemcpyHostToDevice, s));
  detail::launch_rotate(flat.as<float>(), rot_t.as<float>(), uint32_t(n), uint32_t(dim), uint32_t(rot_dim),
                        false, false, CUDA_R_32F, rotated_centers.data_handle(), s);
  CUVS_HIP_TRY(hipStreamSynchronize(s));  // the temporaries go out of scope
}

void make_rotation_matrix(cuvs::resources const& res, device_matrix_view<float> rotation_matrix,
                          bool force_random_rotation)
{
  const int64_t rot_dim = rotation_matrix.extent(0), dim = rotation_matrix.extent(1);
  CUVS_EXPECTS(rot_dim >= dim && dim > 0, "the rotation matrix is [rot_dim, dim] with rot_dim >= dim");
  const std::vector<float> r = detail::make_rotation(uint32_t(rot_dim), uint32_t(dim), force_random_rotation);
  CUVS_HIP_TRY(hipMemcpyAsync(rotation_matrix.data_handle(), r.data(), r.size() * sizeof(float),
                              hipMemcpyHostToDevice, res.stream()));
  CUVS_HIP_TRY(hipStreamSynchronize(res.stream()));  // `r` goes out of scope
}

void recompute_internal_state(cuvs::resources const& res, index<int64_t>* idx)
{
  CUVS_EXPECTS(idx != nullptr && idx->impl() != nullptr, "index must not be null");
  idx->impl()->recompute_internal_state(res.stream());
  finish_edit(res, *idx->impl());
}

}  // namespace helpers
}  // namespace cuvs::neighbors::ivf_pq
