/*
 * extern "C" layer of the IVF-PQ path.  Each function replaces the cuVS entry point of the same
 * name in c/src/neighbors/ivf_pq.cpp (line numbers in include/cuvs/neighbors/ivf_pq.h); the
 * checks, their order and the error texts follow that file.
 */
#include "c_common.hpp"

#include <cuvs/neighbors/ivf_pq.h>

#include <cstring>

namespace {

namespace ivfpq = cuvs::neighbors::ivf_pq;
using ivfpq::codebook_gen;
using ivfpq::elem_type;
using ivfpq::index_params;
using ivfpq::list_layout;
using ivfpq::search_params;
using cuvs::core::expect_tensor;
using cuvs::core::is_dlpack_device_compatible;
using cuvs::core::res_of;
using cuvs::core::tensor_data;
using cuvs::core::translate_exceptions;

ivfpq::index<int64_t>* index_of(cuvsIvfPqIndex_t index)
{
  CUVS_EXPECTS(index != nullptr, "index handle must not be null");
  CUVS_EXPECTS(index->addr != 0, "the index has not been built or loaded");
  return reinterpret_cast<ivfpq::index<int64_t>*>(index->addr);
}

/** c/src/neighbors/ivf_pq.cpp:39-48 -- field-by-field: the C and C++ structs order fields differently */
search_params convert_search_params(const cuvsIvfPqSearchParams& p)
{
  search_params out;
  out.n_probes                 = p.n_probes;
  out.lut_dtype                = int(p.lut_dtype);
  out.internal_distance_dtype  = int(p.internal_distance_dtype);
  out.preferred_shmem_carveout = p.preferred_shmem_carveout;
  out.coarse_search_dtype      = int(p.coarse_search_dtype);
  out.max_internal_batch_size  = p.max_internal_batch_size;
  return out;
}

/** c/src/neighbors/ivf_pq.cpp:22-38 */
index_params convert_index_params(const cuvsIvfPqIndexParams& p)
{
  index_params out;
  out.metric                         = static_cast<cuvs::distance::DistanceType>(int(p.metric));
  out.metric_arg                     = p.metric_arg;
  out.add_data_on_build              = p.add_data_on_build;
  out.n_lists                        = p.n_lists;
  out.kmeans_n_iters                 = p.kmeans_n_iters;
  out.kmeans_trainset_fraction       = p.kmeans_trainset_fraction;
  out.pq_bits                        = p.pq_bits;
  out.pq_dim                         = p.pq_dim;
  out.codebook_kind                  = static_cast<codebook_gen>(int(p.codebook_kind));
  out.force_random_rotation          = p.force_random_rotation;
  out.conservative_memory_allocation = p.conservative_memory_allocation;
  out.max_train_points_per_pq_code   = p.max_train_points_per_pq_code;
  out.codes_layout                   = static_cast<list_layout>(int(p.codes_layout));
  return out;
}

bool elem_type_of(const DLDataType& dt, elem_type* out)
{
  if (dt.code == kDLFloat && dt.bits == 32) { *out = elem_type::f32; return true; }
  if (dt.code == kDLFloat && dt.bits == 16) { *out = elem_type::f16; return true; }
  if (dt.code == kDLInt && dt.bits == 8) { *out = elem_type::i8; return true; }
  if (dt.code == kDLUInt && dt.bits == 8) { *out = elem_type::u8; return true; }
  return false;
}

struct view_ctx {
  int64_t shape[3];
  int64_t strides[3];
};

void view_deleter(DLManagedTensor* self)
{
  if (self != nullptr && self->manager_ctx != nullptr) {
    delete static_cast<view_ctx*>(self->manager_ctx);
    self->manager_ctx       = nullptr;
    self->dl_tensor.shape   = nullptr;
    self->dl_tensor.strides = nullptr;
  }
}

/** Non-owning device view (role of cuvs::core::to_dlpack, c/src/core/detail/interop.hpp:143-174). */
void make_view(DLManagedTensor* out, const void* data, int ndim, const int64_t* shape,
               const int64_t* strides, uint8_t code, uint8_t bits)
{
  CUVS_EXPECTS(out != nullptr, "output tensor must not be null");
  auto* ctx = new view_ctx();
  for (int i = 0; i < ndim; i++) {
    ctx->shape[i]   = shape[i];
    ctx->strides[i] = strides != nullptr ? strides[i] : 0;
  }
  std::memset(out, 0, sizeof(*out));
  out->dl_tensor.data               = const_cast<void*>(data);
  out->dl_tensor.device.device_type = kDLROCM;
  int dev                           = 0;
  (void)hipGetDevice(&dev);
  out->dl_tensor.device.device_id = dev;
  out->dl_tensor.ndim             = ndim;
  out->dl_tensor.dtype            = DLDataType{code, bits, 1};
  out->dl_tensor.shape            = ctx->shape;
  out->dl_tensor.strides          = strides != nullptr ? ctx->strides : nullptr;
  out->dl_tensor.byte_offset      = 0;
  out->manager_ctx                = ctx;
  out->deleter                    = view_deleter;
}

}  // namespace

namespace cuvs::core {

void ivf_pq_search_tensors(cuvs::resources& res, cuvsIvfPqSearchParams_t params,
                           cuvsIvfPqIndex_t index_c, DLManagedTensor* queries_t,
                           DLManagedTensor* neighbors_t, DLManagedTensor* distances_t,
                           DLManagedTensor* bitset_t, int64_t n_bits)
{
  CUVS_EXPECTS(params != nullptr, "search_params must not be null");
  CUVS_EXPECTS(queries_t && neighbors_t && distances_t, "tensors must not be null");
  auto& queries   = queries_t->dl_tensor;
  auto& neighbors = neighbors_t->dl_tensor;
  auto& distances = distances_t->dl_tensor;
  // c/src/neighbors/ivf_pq.cpp:315-325
  CUVS_EXPECTS(is_dlpack_device_compatible(queries), "queries should have device compatible memory");
  CUVS_EXPECTS(is_dlpack_device_compatible(neighbors),
               "neighbors should have device compatible memory");
  CUVS_EXPECTS(is_dlpack_device_compatible(distances),
               "distances should have device compatible memory");
  CUVS_EXPECTS(neighbors.dtype.code == kDLInt && neighbors.dtype.bits == 64,
               "neighbors should be of type int64_t");
  CUVS_EXPECTS(distances.dtype.code == kDLFloat && distances.dtype.bits == 32,
               "distances should be of type float32");
  elem_type t;
  CUVS_EXPECTS(elem_type_of(queries.dtype, &t), "Unsupported queries DLtensor dtype: %d and bits: %d",
               int(queries.dtype.code), int(queries.dtype.bits));
  expect_tensor(queries_t, "queries", 2, queries.dtype.code, queries.dtype.bits);
  expect_tensor(neighbors_t, "neighbors", 2, kDLInt, 64);
  expect_tensor(distances_t, "distances", 2, kDLFloat, 32);
  auto* idx = index_of(index_c);
  // search_with_filtering (ivf_pq_search.cuh:1088-1096)
  CUVS_EXPECTS(queries.shape[0] == neighbors.shape[0] && queries.shape[0] == distances.shape[0],
               "Number of rows in output neighbors and distances matrices must equal the number of "
               "queries.");
  CUVS_EXPECTS(neighbors.shape[1] == distances.shape[1],
               "Number of columns in output neighbors and distances matrices must equal k");
  const auto sp = convert_search_params(*params);
  if (bitset_t != nullptr) {
    expect_tensor(bitset_t, "bitset", 1, kDLUInt, 32);
    CUVS_EXPECTS(is_dlpack_device_compatible(bitset_t->dl_tensor),
                 "bitset should have device compatible memory");
    CUVS_EXPECTS(n_bits >= 0 && (n_bits + 31) / 32 <= bitset_t->dl_tensor.shape[0],
                 "bitset is shorter than n_bits");
    cuvs::neighbors::filtering::bitset_filter f(static_cast<const uint32_t*>(tensor_data(bitset_t)),
                                                n_bits);
    ivfpq::search(res, sp, *idx, tensor_data(queries_t), t, queries.shape[0], queries.shape[1],
           static_cast<int64_t*>(tensor_data(neighbors_t)),
           static_cast<float*>(tensor_data(distances_t)), neighbors.shape[1], f);
  } else {
    cuvs::neighbors::filtering::none_sample_filter f;
    ivfpq::search(res, sp, *idx, tensor_data(queries_t), t, queries.shape[0], queries.shape[1],
           static_cast<int64_t*>(tensor_data(neighbors_t)),
           static_cast<float*>(tensor_data(distances_t)), neighbors.shape[1], f);
  }
}

}  // namespace cuvs::core

namespace {

void do_search(cuvsResources_t res, cuvsIvfPqSearchParams_t params, cuvsIvfPqIndex_t index_c,
               DLManagedTensor* queries_t, DLManagedTensor* neighbors_t,
               DLManagedTensor* distances_t, DLManagedTensor* bitset_t, int64_t n_bits)
{
  cuvs::core::ivf_pq_search_tensors(*res_of(res), params, index_c, queries_t, neighbors_t,
                                    distances_t, bitset_t, n_bits);
}

void do_extend(cuvsResources_t res, DLManagedTensor* new_vectors, DLManagedTensor* new_indices,
               DLManagedTensor* labels, cuvsIvfPqIndex_t index)
{
  CUVS_EXPECTS(new_vectors != nullptr, "new_vectors must not be null");
  auto& vectors = new_vectors->dl_tensor;
  const bool on_device = is_dlpack_device_compatible(vectors);
  if (new_indices != nullptr) {
    // c/src/neighbors/ivf_pq.cpp:130-134
    CUVS_EXPECTS(on_device == is_dlpack_device_compatible(new_indices->dl_tensor),
                 "extend inputs must both either be on device memory or host memory");
  }
  elem_type t;
  CUVS_EXPECTS(elem_type_of(vectors.dtype, &t), "Unsupported index dtype: %d and bits: %d",
               int(vectors.dtype.code), int(vectors.dtype.bits));
  expect_tensor(new_vectors, "new_vectors", 2, vectors.dtype.code, vectors.dtype.bits);
  auto* idx = index_of(index);
  CUVS_EXPECTS(vectors.shape[1] == int64_t(idx->dim()),
               "new_vectors should have the same dimension as the index");
  const int64_t* ids = nullptr;
  if (new_indices != nullptr) {
    expect_tensor(new_indices, "new_indices", 1, kDLInt, 64);
    CUVS_EXPECTS(new_indices->dl_tensor.shape[0] == vectors.shape[0],
                 "new_indices must have one id per new vector");
    ids = static_cast<const int64_t*>(tensor_data(new_indices));
  }
  const uint32_t* lab = nullptr;
  if (labels != nullptr) {
    expect_tensor(labels, "labels", 1, kDLUInt, 32);
    CUVS_EXPECTS(labels->dl_tensor.shape[0] == vectors.shape[0], "labels must have one entry per new vector");
    lab = static_cast<const uint32_t*>(tensor_data(labels));
  }
  // c/src/neighbors/ivf_pq.cpp:405-409: an index built from a precomputed model learns its
  // element type from the first extend
  if (index->dtype.code == 0 && index->dtype.bits == 0) {
    index->dtype.code = vectors.dtype.code;
    index->dtype.bits = vectors.dtype.bits;
  }
  ivfpq::extend(*res_of(res), tensor_data(new_vectors), t, vectors.shape[0], ids, idx, lab);
}

}  // namespace

extern "C" {

cuvsError_t cuvsIvfPqIndexParamsCreate(cuvsIvfPqIndexParams_t* params)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(params != nullptr, "params must not be null");
    auto* p                           = new cuvsIvfPqIndexParams();
    p->metric                         = L2Expanded;
    p->metric_arg                     = 2.0f;
    p->add_data_on_build              = true;
    p->n_lists                        = 1024;
    p->kmeans_n_iters                 = 20;
    p->kmeans_trainset_fraction       = 0.5;
    p->pq_bits                        = 8;
    p->pq_dim                         = 0;
    p->codebook_kind                  = CUVS_IVF_PQ_CODEBOOK_GEN_PER_SUBSPACE;
    p->force_random_rotation          = false;
    p->conservative_memory_allocation = false;
    p->max_train_points_per_pq_code   = 256;
    p->codes_layout                   = CUVS_IVF_PQ_LIST_LAYOUT_INTERLEAVED;
    *params                           = p;
  });
}

cuvsError_t cuvsIvfPqIndexParamsDestroy(cuvsIvfPqIndexParams_t params)
{
  return translate_exceptions([=] { delete params; });
}

cuvsError_t cuvsIvfPqSearchParamsCreate(cuvsIvfPqSearchParams_t* params)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(params != nullptr, "params must not be null");
    auto* p                     = new cuvsIvfPqSearchParams();
    p->n_probes                 = 20;
    p->lut_dtype                = CUDA_R_32F;
    p->internal_distance_dtype  = CUDA_R_32F;
    p->coarse_search_dtype      = CUDA_R_32F;
    p->max_internal_batch_size  = 4096;
    p->preferred_shmem_carveout = 1.0;
    *params                     = p;
  });
}

cuvsError_t cuvsIvfPqSearchParamsDestroy(cuvsIvfPqSearchParams_t params)
{
  return translate_exceptions([=] { delete params; });
}

cuvsError_t cuvsIvfPqIndexCreate(cuvsIvfPqIndex_t* index)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(index != nullptr, "index must not be null");
    *index = new cuvsIvfPqIndex{};
  });
}

cuvsError_t cuvsIvfPqIndexDestroy(cuvsIvfPqIndex_t index_c_ptr)
{
  return translate_exceptions([=] {
    if (index_c_ptr == nullptr) { return; }
    delete reinterpret_cast<ivfpq::index<int64_t>*>(index_c_ptr->addr);
    delete index_c_ptr;
  });
}

#define SCALAR_GETTER(fn, expr)                                    \
  cuvsError_t fn(cuvsIvfPqIndex_t index, int64_t* out)             \
  {                                                                \
    return translate_exceptions([=] {                              \
      CUVS_EXPECTS(out != nullptr, "output pointer must not be null"); \
      auto* idx = index_of(index);                                 \
      *out      = int64_t(expr);                                   \
    });                                                            \
  }
SCALAR_GETTER(cuvsIvfPqIndexGetNLists, idx->n_lists())
SCALAR_GETTER(cuvsIvfPqIndexGetDim, idx->dim())
SCALAR_GETTER(cuvsIvfPqIndexGetSize, idx->size())
SCALAR_GETTER(cuvsIvfPqIndexGetPqDim, idx->pq_dim())
SCALAR_GETTER(cuvsIvfPqIndexGetPqBits, idx->pq_bits())
SCALAR_GETTER(cuvsIvfPqIndexGetPqLen, idx->pq_len())

cuvsError_t cuvsIvfPqIndexGetCenters(cuvsIvfPqIndex_t index, DLManagedTensor* centers)
{
  return translate_exceptions([=] {
    auto* idx = index_of(index);
    // [n_lists, dim] view over the padded rows (c/src/neighbors/ivf_pq.cpp:152-164)
    const int64_t shape[2]   = {int64_t(idx->n_lists()), int64_t(idx->dim())};
    const int64_t strides[2] = {int64_t(idx->dim_ext()), 1};
    make_view(centers, idx->centers(), 2, shape, strides, kDLFloat, 32);
  });
}

cuvsError_t cuvsIvfPqIndexGetCentersPadded(cuvsIvfPqIndex_t index, DLManagedTensor* centers)
{
  return translate_exceptions([=] {
    auto* idx              = index_of(index);
    const int64_t shape[2] = {int64_t(idx->n_lists()), int64_t(idx->dim_ext())};
    make_view(centers, idx->centers(), 2, shape, nullptr, kDLFloat, 32);
  });
}

cuvsError_t cuvsIvfPqIndexGetPqCenters(cuvsIvfPqIndex_t index, DLManagedTensor* pq_centers)
{
  return translate_exceptions([=] {
    auto* idx = index_of(index);
    const int64_t n_books =
      idx->codebook_kind() == codebook_gen::PER_SUBSPACE ? idx->pq_dim() : idx->n_lists();
    const int64_t shape[3] = {n_books, int64_t(idx->pq_len()), int64_t(idx->pq_book_size())};
    make_view(pq_centers, idx->pq_centers(), 3, shape, nullptr, kDLFloat, 32);
  });
}

cuvsError_t cuvsIvfPqIndexGetCentersRot(cuvsIvfPqIndex_t index, DLManagedTensor* centers_rot)
{
  return translate_exceptions([=] {
    auto* idx              = index_of(index);
    const int64_t shape[2] = {int64_t(idx->n_lists()), int64_t(idx->rot_dim())};
    make_view(centers_rot, idx->centers_rot(), 2, shape, nullptr, kDLFloat, 32);
  });
}

cuvsError_t cuvsIvfPqIndexGetRotationMatrix(cuvsIvfPqIndex_t index, DLManagedTensor* rotation_matrix)
{
  return translate_exceptions([=] {
    auto* idx              = index_of(index);
    const int64_t shape[2] = {int64_t(idx->rot_dim()), int64_t(idx->dim())};
    make_view(rotation_matrix, idx->rotation_matrix(), 2, shape, nullptr, kDLFloat, 32);
  });
}

cuvsError_t cuvsIvfPqIndexGetListSizes(cuvsIvfPqIndex_t index, DLManagedTensor* list_sizes)
{
  return translate_exceptions([=] {
    auto* idx              = index_of(index);
    const int64_t shape[1] = {int64_t(idx->n_lists())};
    make_view(list_sizes, idx->list_sizes(), 1, shape, nullptr, kDLUInt, 32);
  });
}

cuvsError_t cuvsIvfPqIndexUnpackContiguousListData(cuvsResources_t res,
                                                   cuvsIvfPqIndex_t index,
                                                   DLManagedTensor* out_codes,
                                                   uint32_t label,
                                                   uint32_t offset)
{
  return translate_exceptions([=] {
    auto* idx = index_of(index);
    expect_tensor(out_codes, "out_codes", 2, kDLUInt, 8);
    CUVS_EXPECTS(is_dlpack_device_compatible(out_codes->dl_tensor),
                 "device_type mismatch between return mdspan and DLTensor");
    const int64_t row_bytes = (int64_t(idx->pq_dim()) * idx->pq_bits() + 7) / 8;
    CUVS_EXPECTS(out_codes->dl_tensor.shape[1] == row_bytes,
                 "out_codes must have ceildiv(pq_dim * pq_bits, 8) = %lld columns",
                 static_cast<long long>(row_bytes));
    ivfpq::unpack_contiguous_list_data(*res_of(res), *idx, static_cast<uint8_t*>(tensor_data(out_codes)),
                                uint32_t(out_codes->dl_tensor.shape[0]), label, offset);
  });
}

cuvsError_t cuvsIvfPqIndexGetListIndices(cuvsIvfPqIndex_t index, uint32_t label,
                                         DLManagedTensor* out_labels)
{
  return translate_exceptions([=] {
    auto* idx = index_of(index);
    auto& ix  = *idx->impl();
    CUVS_EXPECTS(label < ix.n_lists, "label (%u) must be smaller than n_lists (%u)", label, ix.n_lists);
    const int64_t shape[1] = {int64_t(ix.h_list_sizes[label])};
    make_view(out_labels, ix.ids_arena.as<int64_t>() + ix.h_row_offsets[label], 1, shape, nullptr,
              kDLInt, 64);
  });
}

cuvsError_t cuvsIvfPqBuild(cuvsResources_t res,
                           cuvsIvfPqIndexParams_t params,
                           DLManagedTensor* dataset_tensor,
                           cuvsIvfPqIndex_t index)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(params != nullptr && index != nullptr, "params and index must not be null");
    CUVS_EXPECTS(dataset_tensor != nullptr, "dataset must not be null");
    // c/src/neighbors/ivf_pq.cpp:377-403: device or host dataset of float32, float16, int8 or uint8
    auto& ds = dataset_tensor->dl_tensor;
    elem_type t;
    CUVS_EXPECTS(elem_type_of(ds.dtype, &t), "Unsupported dataset DLtensor dtype: %d and bits: %d",
                 int(ds.dtype.code), int(ds.dtype.bits));
    expect_tensor(dataset_tensor, "dataset", 2, ds.dtype.code, ds.dtype.bits);
    auto ip   = convert_index_params(*params);
    auto* idx = new ivfpq::index<int64_t>(
      ivfpq::build(*res_of(res), ip, tensor_data(dataset_tensor), t, ds.shape[0], uint32_t(ds.shape[1])));
    if (index->addr != 0) { delete reinterpret_cast<ivfpq::index<int64_t>*>(index->addr); }
    index->addr       = reinterpret_cast<uintptr_t>(idx);
    index->dtype.code = ds.dtype.code;
    index->dtype.bits = ds.dtype.bits;
  });
}

cuvsError_t cuvsIvfPqBuildPrecomputed(cuvsResources_t res,
                                      cuvsIvfPqIndexParams_t params,
                                      uint32_t dim,
                                      DLManagedTensor* pq_centers_tensor,
                                      DLManagedTensor* centers_tensor,
                                      DLManagedTensor* centers_rot_tensor,
                                      DLManagedTensor* rotation_matrix_tensor,
                                      cuvsIvfPqIndex_t index)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(params != nullptr && index != nullptr, "params and index must not be null");
    CUVS_EXPECTS(pq_centers_tensor && centers_tensor && centers_rot_tensor && rotation_matrix_tensor,
                 "model tensors must not be null");
    // c/src/neighbors/ivf_pq.cpp:503-530
    CUVS_EXPECTS(is_dlpack_device_compatible(pq_centers_tensor->dl_tensor),
                 "pq_centers should have device compatible memory");
    CUVS_EXPECTS(is_dlpack_device_compatible(centers_tensor->dl_tensor),
                 "centers should have device compatible memory");
    CUVS_EXPECTS(is_dlpack_device_compatible(centers_rot_tensor->dl_tensor),
                 "centers_rot should have device compatible memory");
    CUVS_EXPECTS(is_dlpack_device_compatible(rotation_matrix_tensor->dl_tensor),
                 "rotation_matrix should have device compatible memory");
    auto is_f32 = [](DLManagedTensor* t) {
      return t->dl_tensor.dtype.code == kDLFloat && t->dl_tensor.dtype.bits == 32;
    };
    CUVS_EXPECTS(is_f32(pq_centers_tensor), "pq_centers must be float32");
    CUVS_EXPECTS(is_f32(centers_tensor), "centers must be float32");
    CUVS_EXPECTS(is_f32(centers_rot_tensor), "centers_rot must be float32");
    CUVS_EXPECTS(is_f32(rotation_matrix_tensor), "rotation_matrix must be float32");
    expect_tensor(pq_centers_tensor, "pq_centers", 3, kDLFloat, 32);
    expect_tensor(centers_tensor, "centers", 2, kDLFloat, 32);
    expect_tensor(centers_rot_tensor, "centers_rot", 2, kDLFloat, 32);
    expect_tensor(rotation_matrix_tensor, "rotation_matrix", 2, kDLFloat, 32);

    auto ip            = convert_index_params(*params);
    const auto& pqc    = pq_centers_tensor->dl_tensor;
    const auto& cen    = centers_tensor->dl_tensor;
    const auto& cen_r  = centers_rot_tensor->dl_tensor;
    const auto& rot    = rotation_matrix_tensor->dl_tensor;
    // consistency of the extents with the parameters (role of the checks in the precomputed
    // build overload of cuVS)
    ip.n_lists = uint32_t(cen.shape[0]);
    CUVS_EXPECTS(cen.shape[0] > 0, "centers must have at least one row");
    const int64_t book = int64_t(1) << ip.pq_bits;
    CUVS_EXPECTS(ip.pq_bits >= 4 && ip.pq_bits <= 8, "pq_bits must be within [4, 8], got %u", ip.pq_bits);
    CUVS_EXPECTS(pqc.shape[2] == book, "pq_centers.extent(2) (%lld) must equal 1 << pq_bits (%lld)",
                 static_cast<long long>(pqc.shape[2]), static_cast<long long>(book));
    const int64_t pq_len = pqc.shape[1];
    CUVS_EXPECTS(pq_len > 0 && cen_r.shape[1] % pq_len == 0,
                 "centers_rot.extent(1) must be a multiple of pq_len");
    const int64_t pq_dim = cen_r.shape[1] / pq_len;
    if (ip.pq_dim == 0) { ip.pq_dim = uint32_t(pq_dim); }
    CUVS_EXPECTS(int64_t(ip.pq_dim) == pq_dim, "pq_dim (%u) is inconsistent with centers_rot [%lld] / pq_len %lld",
                 ip.pq_dim, static_cast<long long>(cen_r.shape[1]), static_cast<long long>(pq_len));
    CUVS_EXPECTS(pq_len == (int64_t(dim) + pq_dim - 1) / pq_dim,
                 "pq_centers.extent(1) (%lld) must equal ceildiv(dim, pq_dim)", static_cast<long long>(pq_len));
    const int64_t n_books = ip.codebook_kind == codebook_gen::PER_SUBSPACE ? pq_dim : cen.shape[0];
    CUVS_EXPECTS(pqc.shape[0] == n_books, "pq_centers.extent(0) (%lld) must be %lld for this codebook_kind",
                 static_cast<long long>(pqc.shape[0]), static_cast<long long>(n_books));
    const int64_t dim_ext = ((int64_t(dim) + 1 + 7) / 8) * 8;
    CUVS_EXPECTS(cen.shape[1] == dim_ext, "centers must have round_up(dim + 1, 8) = %lld columns, got %lld",
                 static_cast<long long>(dim_ext), static_cast<long long>(cen.shape[1]));
    CUVS_EXPECTS(cen_r.shape[0] == cen.shape[0], "centers_rot must have n_lists rows");
    CUVS_EXPECTS(rot.shape[0] == cen_r.shape[1] && rot.shape[1] == int64_t(dim),
                 "rotation_matrix must be [rot_dim, dim]");

    auto* idx = new ivfpq::index<int64_t>(ivfpq::build(*res_of(res), ip, dim,
                                          static_cast<const float*>(tensor_data(pq_centers_tensor)),
                                          static_cast<const float*>(tensor_data(centers_tensor)),
                                          static_cast<const float*>(tensor_data(centers_rot_tensor)),
                                          static_cast<const float*>(tensor_data(rotation_matrix_tensor))));
    if (index->addr != 0) { delete reinterpret_cast<ivfpq::index<int64_t>*>(index->addr); }
    index->addr       = reinterpret_cast<uintptr_t>(idx);
    index->dtype.code = 0;  // set by the first extend
    index->dtype.bits = 0;
  });
}

cuvsError_t cuvsIvfPqSearch(cuvsResources_t res,
                            cuvsIvfPqSearchParams_t params,
                            cuvsIvfPqIndex_t index,
                            DLManagedTensor* queries,
                            DLManagedTensor* neighbors,
                            DLManagedTensor* distances)
{
  return translate_exceptions(
    [=] { do_search(res, params, index, queries, neighbors, distances, nullptr, 0); });
}

cuvsError_t cuvsAmdIvfPqSearchWithBitset(cuvsResources_t res,
                                         cuvsIvfPqSearchParams_t params,
                                         cuvsIvfPqIndex_t index,
                                         DLManagedTensor* queries,
                                         DLManagedTensor* neighbors,
                                         DLManagedTensor* distances,
                                         DLManagedTensor* bitset,
                                         int64_t n_bits)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(bitset != nullptr, "bitset must not be null");
    do_search(res, params, index, queries, neighbors, distances, bitset, n_bits);
  });
}

cuvsError_t cuvsAmdIvfPqSelectClusters(cuvsResources_t res,
                                       cuvsIvfPqSearchParams_t params,
                                       cuvsIvfPqIndex_t index,
                                       DLManagedTensor* queries_t,
                                       DLManagedTensor* probes_t)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(params != nullptr, "search_params must not be null");
    CUVS_EXPECTS(queries_t && probes_t, "tensors must not be null");
    auto& queries = queries_t->dl_tensor;
    CUVS_EXPECTS(is_dlpack_device_compatible(queries), "queries should have device compatible memory");
    CUVS_EXPECTS(is_dlpack_device_compatible(probes_t->dl_tensor),
                 "clusters_to_probe should have device compatible memory");
    elem_type t;
    CUVS_EXPECTS(elem_type_of(queries.dtype, &t), "Unsupported queries DLtensor dtype: %d and bits: %d",
                 int(queries.dtype.code), int(queries.dtype.bits));
    expect_tensor(queries_t, "queries", 2, queries.dtype.code, queries.dtype.bits);
    expect_tensor(probes_t, "clusters_to_probe", 2, kDLUInt, 32);
    auto* idx = index_of(index);
    CUVS_EXPECTS(queries.shape[1] == int64_t(idx->dim()),
                 "Number of query dimensions should equal number of dimensions in the index.");
    const auto sp    = convert_search_params(*params);
    const int64_t P  = std::min<int64_t>(sp.n_probes, idx->n_lists());
    CUVS_EXPECTS(probes_t->dl_tensor.shape[0] == queries.shape[0] && probes_t->dl_tensor.shape[1] == P,
                 "clusters_to_probe must be [n_queries, min(n_probes, n_lists)]");
    ivfpq::select_clusters(*res_of(res), sp, *idx, tensor_data(queries_t), t, queries.shape[0],
                    static_cast<uint32_t*>(tensor_data(probes_t)));
  });
}

cuvsError_t cuvsIvfPqExtend(cuvsResources_t res,
                            DLManagedTensor* new_vectors,
                            DLManagedTensor* new_indices,
                            cuvsIvfPqIndex_t index)
{
  return translate_exceptions([=] { do_extend(res, new_vectors, new_indices, nullptr, index); });
}

cuvsError_t cuvsAmdIvfPqExtendLabeled(cuvsResources_t res,
                                      DLManagedTensor* new_vectors,
                                      DLManagedTensor* new_indices,
                                      DLManagedTensor* labels,
                                      cuvsIvfPqIndex_t index)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(labels != nullptr, "labels must not be null");
    do_extend(res, new_vectors, new_indices, labels, index);
  });
}

cuvsError_t cuvsIvfPqTransform(cuvsResources_t res,
                               cuvsIvfPqIndex_t index,
                               DLManagedTensor* input_dataset,
                               DLManagedTensor* output_labels,
                               DLManagedTensor* output_dataset)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(input_dataset && output_labels && output_dataset, "tensors must not be null");
    // c/src/neighbors/ivf_pq.cpp:596-612
    CUVS_EXPECTS(is_dlpack_device_compatible(input_dataset->dl_tensor),
                 "input_dataset should have device compatible memory");
    CUVS_EXPECTS(is_dlpack_device_compatible(output_labels->dl_tensor),
                 "output_labels should have device compatible memory");
    CUVS_EXPECTS(is_dlpack_device_compatible(output_dataset->dl_tensor),
                 "output_dataset should have device compatible memory");
    CUVS_EXPECTS(output_labels->dl_tensor.dtype.code == kDLUInt && output_labels->dl_tensor.dtype.bits == 32,
                 "output_labels must have a uint32 dtype ");
    CUVS_EXPECTS(output_dataset->dl_tensor.dtype.code == kDLUInt && output_dataset->dl_tensor.dtype.bits == 8,
                 "output_dataset must have a uint8 dtype");
    auto& ds = input_dataset->dl_tensor;
    elem_type t;
    CUVS_EXPECTS(elem_type_of(ds.dtype, &t), "Unsupported input_dataset DLtensor dtype: %d and bits: %d",
                 int(ds.dtype.code), int(ds.dtype.bits));
    expect_tensor(input_dataset, "input_dataset", 2, ds.dtype.code, ds.dtype.bits);
    expect_tensor(output_labels, "output_labels", 1, kDLUInt, 32);
    expect_tensor(output_dataset, "output_dataset", 2, kDLUInt, 8);
    auto* idx = index_of(index);
    CUVS_EXPECTS(ds.shape[1] == int64_t(idx->dim()), "input_dataset should have the same dimension as the index");
    const int64_t row_bytes = (int64_t(idx->pq_dim()) * idx->pq_bits() + 7) / 8;
    CUVS_EXPECTS(output_labels->dl_tensor.shape[0] == ds.shape[0] &&
                   output_dataset->dl_tensor.shape[0] == ds.shape[0] &&
                   output_dataset->dl_tensor.shape[1] == row_bytes,
                 "output extents must be [n] and [n, ceildiv(pq_dim * pq_bits, 8)]");
    ivfpq::transform(*res_of(res), *idx, tensor_data(input_dataset), t, ds.shape[0],
              static_cast<uint32_t*>(tensor_data(output_labels)),
              static_cast<uint8_t*>(tensor_data(output_dataset)));
  });
}

cuvsError_t cuvsIvfPqSerialize(cuvsResources_t res, const char* filename, cuvsIvfPqIndex_t index)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(filename != nullptr, "filename must not be null");
    ivfpq::serialize(*res_of(res), std::string(filename), *index_of(index));
  });
}

cuvsError_t cuvsIvfPqDeserialize(cuvsResources_t res, const char* filename, cuvsIvfPqIndex_t index)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(filename != nullptr && index != nullptr, "filename and index must not be null");
    auto* idx = new ivfpq::index<int64_t>();
    try {
      ivfpq::deserialize(*res_of(res), std::string(filename), idx);
    } catch (...) {
      delete idx;
      throw;
    }
    if (index->addr != 0) { delete reinterpret_cast<ivfpq::index<int64_t>*>(index->addr); }
    index->addr = reinterpret_cast<uintptr_t>(idx);
  });
}

cuvsError_t cuvsAmdIvfPqSetSearchTuning(cuvsResources_t res, const cuvsAmdIvfPqSearchTuning* tuning)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(tuning != nullptr, "tuning must not be null");
    CUVS_EXPECTS(tuning->early_stop >= 0 && tuning->early_stop <= 2, "early_stop must be 0, 1 or 2");
    auto& t        = res_of(res)->tuning;
    t.early_stop   = tuning->early_stop;
    t.generic_scan = tuning->generic_scan != 0;
    t.plain_coarse = tuning->plain_coarse != 0;
    t.serial_batches = tuning->serial_batches != 0;
  });
}

cuvsError_t cuvsAmdIvfPqProfilingEnable(cuvsResources_t res, bool enable)
{
  return translate_exceptions([=] { res_of(res)->profiling = enable; });
}

cuvsError_t cuvsAmdIvfPqGetSearchProfile(cuvsResources_t res, cuvsAmdIvfPqSearchProfile* profile)
{
  return translate_exceptions([=] {
    CUVS_EXPECTS(profile != nullptr, "profile must not be null");
    auto* r = res_of(res);
    r->sync();
    const auto& p            = r->last_profile;
    profile->n_queries       = p.n_queries;
    profile->n_probes        = p.n_probes;
    profile->k               = p.k;
    profile->n_scan_launches = p.n_scan_launches;
    profile->coarse_ms       = p.coarse_ms;
    profile->rotate_ms       = p.rotate_ms;
    profile->scan_ms         = p.scan_ms;
    profile->merge_ms        = p.merge_ms;
    profile->total_ms        = p.total_ms;
    profile->scan_bytes      = p.scan_bytes;
    profile->scan_rows       = p.scan_rows;
    profile->lead_scan_ms      = p.lead_scan_ms;
    profile->screen_ms         = p.screen_ms;
    profile->survivor_scan_ms  = p.survivor_scan_ms;
    profile->scan_kernel       = p.scan_kernel;
    profile->lead_bytes        = p.lead_bytes;
    profile->screen_bytes      = p.screen_bytes;
    profile->survivor_bytes    = p.survivor_bytes;
    profile->n_screened_pairs  = p.n_screened_pairs;
    profile->n_surviving_pairs = p.n_surviving_pairs;
    profile->n_far_pairs       = p.n_far_pairs;
  });
}

}  // extern "C"
