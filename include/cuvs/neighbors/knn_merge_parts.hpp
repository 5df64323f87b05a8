/*
 * C++ API of the step that merges the per-shard results of a row-sharded search
 * (cuVS cpp/include/cuvs/neighbors/knn_merge_parts.hpp:36-100).
 */
#pragma once

#include <cuvs/core/resources.hpp>

#include <cstdint>

// The library is built with hidden visibility; what this header declares is its C++ interface
// (the reference marks the same namespaces CUVS_EXPORT).
#pragma GCC visibility push(default)

namespace cuvs::neighbors {

/** in_keys / in_ids: [n_parts * n_samples, k], part-major (all rows of part 0, then part 1, ...),
 *  each row ascending or not; out_keys / out_ids: [n_samples, k], the k smallest keys of the
 *  n_parts * k candidates of each row in ascending order (equal keys: the lower part, then the
 *  lower column, first), ids shifted by translations[part].  n_parts * k <= 8192.
 *  IdT: int64_t, int32_t, uint32_t. */
template <typename IdT>
void knn_merge_parts(cuvs::resources const& res,
                     device_matrix_view<const float> in_keys,
                     device_matrix_view<const IdT> in_ids,
                     device_matrix_view<float> out_keys,
                     device_matrix_view<IdT> out_ids,
                     const IdT* translations,
                     int64_t n_parts);

}  // namespace cuvs::neighbors

#pragma GCC visibility pop
