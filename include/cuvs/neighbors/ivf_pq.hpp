/*
 * C++ API of the IVF-PQ search path for AMD Instinct MI355X (gfx950).
 *
 * Same namespace, type names, field names, defaults and argument meaning as the cuVS header
 * cpp/include/cuvs/neighbors/ivf_pq.hpp (index_params :47-151, search_params :160-213,
 * index :475-675, search overloads :1821-1963, extend, build from a precomputed model), with
 * cuvs::resources / cuvs::device_matrix_view standing in for the RAFT types.
 */
#pragma once

#include <cuvs/core/data_type.h>
#include <cuvs/core/resources.hpp>

#include <cstdint>
#include <memory>
#include <iosfwd>
#include <string>

// The library is built with hidden visibility; what this header declares is its C++ interface
// (the reference marks the same namespaces CUVS_EXPORT).
#pragma GCC visibility push(default)

namespace cuvs::distance {
/** Numeric values of cuvs::distance::DistanceType (cpp/include/cuvs/distance/distance.hpp). */
enum class DistanceType : int {
  L2Expanded     = 0,
  L2SqrtExpanded = 1,
  CosineExpanded = 2,
  L2Unexpanded     = 4,
  L2SqrtUnexpanded = 5,
  InnerProduct   = 6,
};
}  // namespace cuvs::distance

namespace cuvs::neighbors {

/** cpp/include/cuvs/neighbors/common.hpp:125-132 */
struct index_params {
  cuvs::distance::DistanceType metric = cuvs::distance::DistanceType::L2Expanded;
  float metric_arg                    = 2.0f;
};
struct search_params {};

namespace filtering {
/** cpp/include/cuvs/neighbors/common.hpp:1342-1480 -- only these two filters reach IVF-PQ search. */
struct base_filter {
  virtual ~base_filter() = default;
};
struct none_sample_filter : public base_filter {};
/** Bit i set = source id i may be returned. `bits` is a device array of ceil(n_bits / 32) words. */
struct bitset_filter : public base_filter {
  const uint32_t* bits = nullptr;
  int64_t n_bits       = 0;
  bitset_filter(const uint32_t* b, int64_t n) : bits(b), n_bits(n) {}
};
}  // namespace filtering

namespace ivf_pq {

enum class codebook_gen { PER_SUBSPACE = 0, PER_CLUSTER = 1 };
enum class list_layout { FLAT = 0, INTERLEAVED = 1 };

constexpr uint32_t kIndexGroupSize   = 32;  // rows interleaved per group  (ivf_pq.hpp:222)
constexpr uint32_t kIndexGroupVecLen = 16;  // bytes per interleaved chunk (ivf_pq.hpp:224)

struct index_params : cuvs::neighbors::index_params {
  uint32_t n_lists                      = 1024;
  uint32_t kmeans_n_iters               = 20;
  double kmeans_trainset_fraction       = 0.5;
  uint32_t pq_bits                      = 8;
  uint32_t pq_dim                       = 0;
  codebook_gen codebook_kind            = codebook_gen::PER_SUBSPACE;
  list_layout codes_layout              = list_layout::INTERLEAVED;
  bool force_random_rotation            = false;
  bool conservative_memory_allocation   = false;
  bool add_data_on_build                = true;
  uint32_t max_train_points_per_pq_code = 256;
};

struct search_params : cuvs::neighbors::search_params {
  uint32_t n_probes                 = 20;
  int lut_dtype                     = CUDA_R_32F;
  int internal_distance_dtype       = CUDA_R_32F;
  double preferred_shmem_carveout   = 1.0;
  int coarse_search_dtype           = CUDA_R_32F;
  uint32_t max_internal_batch_size  = 4096;
};

#pragma GCC visibility pop
namespace detail {
struct index_impl;  // the index's contents: not part of the interface
}
#pragma GCC visibility push(default)

/** Element type of query / dataset rows. */
enum class elem_type : int { f32 = 0, f16 = 1, i8 = 2, u8 = 3 };

/**
 * IVF-PQ index contents in device memory: coarse centres with fused norms, rotation matrix,
 * PQ codebooks, and per-list interleaved codes + source ids.  Only IdxT = int64_t exists.
 */
template <typename IdxT>
class index {
  static_assert(sizeof(IdxT) == 8, "only int64_t ids are supported");

 public:
  index();
  ~index();
  index(index&&) noexcept;
  index& operator=(index&&) noexcept;

  int64_t size() const;
  uint32_t dim() const;
  uint32_t dim_ext() const;
  uint32_t rot_dim() const;
  uint32_t pq_bits() const;
  uint32_t pq_dim() const;
  uint32_t pq_len() const;
  uint32_t pq_book_size() const;
  uint32_t n_lists() const;
  cuvs::distance::DistanceType metric() const;
  codebook_gen codebook_kind() const;
  list_layout codes_layout() const;
  bool conservative_memory_allocation() const;

  const float* centers() const;          // [n_lists, dim_ext]
  const float* centers_rot() const;      // [n_lists, rot_dim]
  const float* rotation_matrix() const;  // [rot_dim, dim]
  const float* pq_centers() const;       // [pq_dim | n_lists, pq_len, pq_book_size]
  const uint32_t* list_sizes() const;    // device [n_lists]
  const uint8_t* const* data_ptrs() const;
  const IdxT* const* inds_ptrs() const;
  /** Host prefix sums of list sizes sorted in descending order, [n_lists + 1]. */
  const int64_t* accum_sorted_sizes() const;

  detail::index_impl* impl() const { return impl_.get(); }

 private:
  std::unique_ptr<detail::index_impl> impl_;
};

/** Index from a trained model (cuVS: build(res, params, dim, pq_centers, centers, centers_rot,
 *  rotation_matrix), cpp/include/cuvs/neighbors/ivf_pq.hpp).  All inputs are device float32;
 *  they are copied. */
index<int64_t> build(cuvs::resources const& res,
                     const index_params& params,
                     uint32_t dim,
                     const float* pq_centers,
                     const float* centers,
                     const float* centers_rot,
                     const float* rotation_matrix);

/** Train an index on a dataset and (params.add_data_on_build) add the dataset to it
 *  (cuVS: ivf_pq::build(res, params, dataset), cpp/include/cuvs/neighbors/ivf_pq.hpp;
 *  cpp/src/neighbors/ivf_pq/ivf_pq_build.cuh:1240-1410).  `dataset` is [n_rows, dim] row-major in
 *  device or host memory. */
index<int64_t> build(cuvs::resources const& res,
                     const index_params& params,
                     const void* dataset,
                     elem_type type,
                     int64_t n_rows,
                     uint32_t dim);

template <typename T>
index<int64_t> build(cuvs::resources const& res,
                     const index_params& params,
                     device_matrix_view<const T> dataset);

/** ivf_pq.hpp:732-890 -- the same, into an index object the caller holds. */
template <typename T>
void build(cuvs::resources const& res,
           const index_params& params,
           device_matrix_view<const T> dataset,
           index<int64_t>* idx);

/** A deep copy of an index: model, lists and tables in memory of its own (cuVS detail::clone,
 *  ivf_pq_build.cuh:962-996, shares the list data between the two until one of them is extended). */
index<int64_t> clone(cuvs::resources const& res, const index<int64_t>& source);

/** Encode and append rows.  `new_vectors` and `new_indices` are device pointers; a null
 *  `new_indices` numbers the rows consecutively from the current size.  A non-null `labels`
 *  (device uint32 [n]) overrides the nearest-centre assignment. */
void extend(cuvs::resources const& res,
            const void* new_vectors,
            elem_type type,
            int64_t n_rows,
            const int64_t* new_indices,
            index<int64_t>* idx,
            const uint32_t* labels = nullptr);

template <typename T>
void extend(cuvs::resources const& res,
            device_matrix_view<const T> new_vectors,
            const int64_t* new_indices,
            index<int64_t>* idx);

/** ivf_pq.hpp:1296-1737 (the forms that return an index) -- `orig` stays as it is; the result holds
 *  its rows and the new ones. */
template <typename T>
index<int64_t> extend(cuvs::resources const& res,
                      device_matrix_view<const T> new_vectors,
                      const int64_t* new_indices,
                      const index<int64_t>& orig);

/** Labels and bit-contiguous codes of rows, without modifying the index (cuVS: transform). */
void transform(cuvs::resources const& res,
               const index<int64_t>& idx,
               const void* vectors,
               elem_type type,
               int64_t n_rows,
               uint32_t* labels_out,
               uint8_t* codes_out);

/** cuVS: ivf_pq::search (cpp/include/cuvs/neighbors/ivf_pq.hpp:1821-1963), T in
 *  {float, _Float16, int8_t, uint8_t}. */
template <typename T>
void search(cuvs::resources const& res,
            const search_params& params,
            const index<int64_t>& idx,
            device_matrix_view<const T> queries,
            device_matrix_view<int64_t> neighbors,
            device_matrix_view<float> distances,
            const cuvs::neighbors::filtering::base_filter& sample_filter =
              cuvs::neighbors::filtering::none_sample_filter{});

/** Type-erased form used by the C layer. */
void search(cuvs::resources const& res,
            const search_params& params,
            const index<int64_t>& idx,
            const void* queries,
            elem_type type,
            int64_t n_queries,
            int64_t query_dim,
            int64_t* neighbors,
            float* distances,
            int64_t k,
            const cuvs::neighbors::filtering::base_filter& sample_filter);

/** Coarse step only: clusters_to_probe is device uint32 [n_queries, min(n_probes, n_lists)]. */
void select_clusters(cuvs::resources const& res,
                     const search_params& params,
                     const index<int64_t>& idx,
                     const void* queries,
                     elem_type type,
                     int64_t n_queries,
                     uint32_t* clusters_to_probe);

/** cuVS helpers::codepacker::unpack_contiguous_list_data. */
void unpack_contiguous_list_data(cuvs::resources const& res,
                                 const index<int64_t>& idx,
                                 uint8_t* out_codes,
                                 uint32_t n_rows,
                                 uint32_t label,
                                 uint32_t offset);

void serialize(cuvs::resources const& res, const std::string& filename, const index<int64_t>& idx);
void deserialize(cuvs::resources const& res, const std::string& filename, index<int64_t>* idx);
/** The same format on a stream (cuVS ivf_pq.hpp:2034-2036, 2084-2086): several indexes, or an index
 *  and what a caller keeps beside it, can share one file. */
void serialize(cuvs::resources const& res, std::ostream& os, const index<int64_t>& idx);
void deserialize(cuvs::resources const& res, std::istream& is, index<int64_t>* idx);

/**
 * Reading and editing single lists of an index (cuVS: namespace ivf_pq::helpers,
 * cpp/include/cuvs/neighbors/ivf_pq.hpp:2559-3376).  All tensors are device memory; rows of a list
 * are addressed by their position in the list.  The functions taking `index*` change it and, like
 * `extend`, must not run concurrently with searches on it.
 */
namespace helpers {
namespace codepacker {

/** ivf_pq.hpp:2597 -- codes of rows offset .. offset + codes.extent(0) - 1 of a bare list buffer
 *  (interleaved groups of 32 rows, as `index::lists()[label]->data` in the reference; here a
 *  pointer: the extents follow from pq_dim = codes.extent(1) and pq_bits), one code per byte. */
void unpack(cuvs::resources const& res,
            const uint8_t* list_data,
            uint32_t pq_bits,
            uint32_t offset,
            device_matrix_view<uint8_t> codes);

/** ivf_pq.hpp:2669 -- writes `codes` [n_rows, pq_dim], one code per byte, into the rows from
 *  `offset` on of a bare list buffer.  The buffer may be one of an index's own lists
 *  (`index::data_ptrs()[label]`): the index notices, and its next search first refreshes the copies
 *  of leading and widened codes it keeps next to the lists (as pack_list_data does at once).  List
 *  memory written by any other means (a kernel of the caller's) MUST be followed by
 *  helpers::recompute_internal_state before the index is searched again. */
void pack(cuvs::resources const& res,
          device_matrix_view<const uint8_t> codes,
          uint32_t pq_bits,
          uint32_t offset,
          uint8_t* list_data);

/** ivf_pq.hpp:2637 -- the same rows of a bare list buffer as bit strings: row r of `codes` holds
 *  ceildiv(pq_dim * pq_bits, 8) bytes, code j in bits [j * pq_bits, (j + 1) * pq_bits). */
void unpack_contiguous(cuvs::resources const& res,
                       const uint8_t* list_data,
                       uint32_t pq_bits,
                       uint32_t offset,
                       uint32_t n_rows,
                       uint32_t pq_dim,
                       uint8_t* codes);

/** ivf_pq.hpp:2705 -- writes `n_rows` bit strings of that form into the rows from `offset` on of a
 *  bare list buffer (one of an index's own lists included, as for `pack`). */
void pack_contiguous(cuvs::resources const& res,
                     const uint8_t* codes,
                     uint32_t n_rows,
                     uint32_t pq_dim,
                     uint32_t pq_bits,
                     uint32_t offset,
                     uint8_t* list_data);

/** ivf_pq.hpp:2818 -- codes of rows offset .. offset + out_codes.extent(0) - 1 of list `label`, one
 *  code per byte: out_codes is [n_take, pq_dim]. */
void unpack_list_data(cuvs::resources const& res,
                      const index<int64_t>& idx,
                      device_matrix_view<uint8_t> out_codes,
                      uint32_t label,
                      uint32_t offset);

/** ivf_pq.hpp:2854 -- the same for the rows at positions `in_cluster_indices`. */
void unpack_list_data(cuvs::resources const& res,
                      const index<int64_t>& idx,
                      device_vector_view<const uint32_t> in_cluster_indices,
                      device_matrix_view<uint8_t> out_codes,
                      uint32_t label);

/** ivf_pq.hpp:2895 -- rows as bit strings of ceil(pq_dim * pq_bits / 8) bytes. */
void unpack_contiguous_list_data(cuvs::resources const& res,
                                 const index<int64_t>& idx,
                                 uint8_t* out_codes,
                                 uint32_t n_rows,
                                 uint32_t label,
                                 uint32_t offset);

/** ivf_pq.hpp:2739 -- overwrites the codes of rows offset .. offset + new_codes.extent(0) - 1 of
 *  list `label` (which must exist already) with `new_codes` [n_rows, pq_dim], one code per byte. */
void pack_list_data(cuvs::resources const& res,
                    index<int64_t>* idx,
                    device_matrix_view<const uint8_t> new_codes,
                    uint32_t label,
                    uint32_t offset);

/** ivf_pq.hpp:2782 -- the same from bit-contiguous rows. */
void pack_contiguous_list_data(cuvs::resources const& res,
                               index<int64_t>* idx,
                               const uint8_t* new_codes,
                               uint32_t n_rows,
                               uint32_t label,
                               uint32_t offset);

/** ivf_pq.hpp:2932-2950 -- decodes rows offset .. of list `label` to vectors of the original space:
 *  out_vectors [n_take, dim] = rotation^T (rotated centre + codebook entries), mapped to T
 *  (float, _Float16, int8_t, uint8_t). */
template <typename T>
void reconstruct_list_data(cuvs::resources const& res,
                           const index<int64_t>& idx,
                           device_matrix_view<T> out_vectors,
                           uint32_t label,
                           uint32_t offset);

/** ivf_pq.hpp:2987-3002 -- the same for the rows at positions `in_cluster_indices`. */
template <typename T>
void reconstruct_list_data(cuvs::resources const& res,
                           const index<int64_t>& idx,
                           device_vector_view<const uint32_t> in_cluster_indices,
                           device_matrix_view<T> out_vectors,
                           uint32_t label);

/** ivf_pq.hpp:3035 -- appends rows given by their codes ([n_rows, pq_dim], one per byte) and source
 *  indices to list `label`, in the order given. */
void extend_list_with_codes(cuvs::resources const& res,
                            index<int64_t>* idx,
                            device_matrix_view<const uint8_t> new_codes,
                            device_vector_view<const int64_t> new_indices,
                            uint32_t label);

/** ivf_pq.hpp:3074 -- the same from bit-contiguous rows [n_rows, ceil(pq_dim * pq_bits / 8)]. */
void extend_list_with_contiguous_codes(cuvs::resources const& res,
                                       index<int64_t>* idx,
                                       device_matrix_view<const uint8_t> new_codes,
                                       device_vector_view<const int64_t> new_indices,
                                       uint32_t label);

/** ivf_pq.hpp:3109-3119 -- encodes `new_vectors` against list `label` (no nearest-centre search) and
 *  appends them in the order given. */
template <typename T>
void extend_list(cuvs::resources const& res,
                 index<int64_t>* idx,
                 device_matrix_view<const T> new_vectors,
                 device_vector_view<const int64_t> new_indices,
                 uint32_t label);

}  // namespace codepacker

/** ivf_pq.hpp:3362-3366 -- list `label` holds `new_used_size` rows from now on: its first
 *  min(old, new) rows keep their codes and ids, rows added by a larger size hold zero codes and
 *  the id of an empty slot until they are written (pack_list_data; extend_list_with_codes does both
 *  steps).  The reference resizes a list object (`index.lists()[label]`) given its spec and old
 *  size; the lists of this index share one allocation, so the call names the index and the list. */
void resize_list(cuvs::resources const& res, index<int64_t>* idx, uint32_t label, uint32_t new_used_size);

/** ivf_pq.hpp:3144 -- list `label` becomes empty. */
void erase_list(cuvs::resources const& res, index<int64_t>* idx, uint32_t label);

/** ivf_pq.hpp:3166 -- every list becomes empty; the trained model stays. */
void reset_index(cuvs::resources const& res, index<int64_t>* idx);

/** ivf_pq.hpp:3231-3236 -- the cluster centres without the norm column: `cluster_centers` is
 *  [n_lists, dim] float in device or host memory. */
void extract_centers(cuvs::resources const& res, const index<int64_t>& idx, float* cluster_centers);

/** ivf_pq.hpp:3179-3195 -- `padded_centers` [n_centers, dim_ext] (device) = the rows of `centers`
 *  [n_centers, dim] (device or host), their squared L2 norm in column dim, zeros behind it: the form
 *  `build` from a precomputed model takes. */
void pad_centers_with_norms(cuvs::resources const& res,
                            device_matrix_view<const float> centers,
                            device_matrix_view<float> padded_centers);

/** ivf_pq.hpp:3208 -- `rotated_centers` [n_centers, rot_dim] = rotation_matrix [rot_dim, dim] applied
 *  to the first dim columns of `padded_centers`. */
void rotate_padded_centers(cuvs::resources const& res,
                           device_matrix_view<const float> padded_centers,
                           device_matrix_view<const float> rotation_matrix,
                           device_matrix_view<float> rotated_centers);

/** ivf_pq.hpp:3292 -- fills `rotation_matrix` [rot_dim, dim] (device): the identity when rot_dim == dim
 *  and no random rotation is asked for, else a matrix with orthonormal columns. */
void make_rotation_matrix(cuvs::resources const& res,
                          device_matrix_view<float> rotation_matrix,
                          bool force_random_rotation);

/** ivf_pq.hpp:3265 -- rebuilds the tables derived from the list sizes and addresses, and the copies
 *  of leading / widened codes the searches read: to be called after list memory was written
 *  directly. */
void recompute_internal_state(cuvs::resources const& res, index<int64_t>* idx);

}  // namespace helpers

}  // namespace ivf_pq
}  // namespace cuvs::neighbors

#pragma GCC visibility pop
