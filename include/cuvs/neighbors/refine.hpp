/*
 * C++ API of the refinement step (cuVS cpp/include/cuvs/neighbors/refine.hpp:62-68 and the
 * overloads for half, int8_t and uint8_t that follow it).
 */
#pragma once

#include <cuvs/core/resources.hpp>
#include <cuvs/distance/distance.h>
#include <cuvs/neighbors/ivf_pq.hpp>

// The library is built with hidden visibility; what this header declares is its C++ interface
// (the reference marks the same namespaces CUVS_EXPORT).
#pragma GCC visibility push(default)

namespace cuvs::neighbors {

/** For each query the exact distance to each of its candidates, the k = indices.extent(1) nearest
 *  kept, ascending (descending similarity for InnerProduct).  T: float, _Float16, int8_t, uint8_t. */
template <typename T>
void refine(cuvs::resources const& res,
            device_matrix_view<const T> dataset,
            device_matrix_view<const T> queries,
            device_matrix_view<const int64_t> neighbor_candidates,
            device_matrix_view<int64_t> indices,
            device_matrix_view<float> distances,
            cuvs::distance::DistanceType metric = cuvs::distance::DistanceType::L2Unexpanded);

/** The same on matrices in host memory (cuVS refine.hpp:287-293 and the overloads for half, int8_t
 *  and uint8_t that follow it).  The reference computes these on the CPU; here the candidate rows
 *  are gathered into pinned memory, a batch of queries at a time, and the device kernel above
 *  ranks them: same results as the device overload.  Returns when the outputs are complete. */
template <typename T>
void refine(cuvs::resources const& res,
            host_matrix_view<const T> dataset,
            host_matrix_view<const T> queries,
            host_matrix_view<const int64_t> neighbor_candidates,
            host_matrix_view<int64_t> indices,
            host_matrix_view<float> distances,
            cuvs::distance::DistanceType metric = cuvs::distance::DistanceType::L2Unexpanded);

/** refine.hpp:107-113 and 332-338: float rows with 32-bit ids, on the device and in host memory
 *  (an output slot that cannot be filled holds 0xFFFFFFFF). */
void refine(cuvs::resources const& res,
            device_matrix_view<const float> dataset,
            device_matrix_view<const float> queries,
            device_matrix_view<const uint32_t> neighbor_candidates,
            device_matrix_view<uint32_t> indices,
            device_matrix_view<float> distances,
            cuvs::distance::DistanceType metric = cuvs::distance::DistanceType::L2Unexpanded);
void refine(cuvs::resources const& res,
            host_matrix_view<const float> dataset,
            host_matrix_view<const float> queries,
            host_matrix_view<const uint32_t> neighbor_candidates,
            host_matrix_view<uint32_t> indices,
            host_matrix_view<float> distances,
            cuvs::distance::DistanceType metric = cuvs::distance::DistanceType::L2Unexpanded);

/** Type-erased entry point behind the C API. */
void refine(cuvs::resources const& res, const void* dataset, const void* queries,
            ivf_pq::elem_type type, int64_t n_rows, int64_t n_queries, int64_t dim,
            const int64_t* candidates, int64_t n_candidates, int64_t* indices, float* distances,
            int64_t k, cuvs::distance::DistanceType metric);

/** Type-erased entry point for matrices in host memory. */
void refine_host(cuvs::resources const& res, const void* dataset, const void* queries,
                 ivf_pq::elem_type type, int64_t n_rows, int64_t n_queries, int64_t dim,
                 const int64_t* candidates, int64_t n_candidates, int64_t* indices, float* distances,
                 int64_t k, cuvs::distance::DistanceType metric);

}  // namespace cuvs::neighbors

#pragma GCC visibility pop
