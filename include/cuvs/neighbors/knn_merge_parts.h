/*
 * C entry point for merging the per-shard results of a row-sharded search.  The reference has this
 * step only in C++ (cpp/include/cuvs/neighbors/knn_merge_parts.hpp:36-100, used by the multi-GPU
 * search, cpp/src/neighbors/mg/snmg.cuh); the C symbol below is an addition of this library.
 */
#ifndef CUVS_AMD_NEIGHBORS_KNN_MERGE_PARTS_H
#define CUVS_AMD_NEIGHBORS_KNN_MERGE_PARTS_H

#include <cuvs/core/c_api.h>
#include <dlpack/dlpack.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/**
 * (no C counterpart in the reference; C++: knn_merge_parts.hpp:36-100)
 *
 * in_keys float32 [n_parts * n_samples, k] and in_ids int64 [n_parts * n_samples, k], part-major;
 * translations int64 [n_parts]; out_keys float32 [n_samples, k], out_ids int64 [n_samples, k]:
 * per row the k smallest keys of all parts, ascending, ids shifted by their part's translation.
 * All tensors must be accessible from the device; n_parts * k <= 8192.
 */
CUVS_EXPORT cuvsError_t cuvsAmdKnnMergeParts(cuvsResources_t res,
                                             DLManagedTensor* in_keys,
                                             DLManagedTensor* in_ids,
                                             DLManagedTensor* translations,
                                             DLManagedTensor* out_keys,
                                             DLManagedTensor* out_ids);

#ifdef __cplusplus
}
#endif
#endif
