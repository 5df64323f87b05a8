/*
 * C API of the refinement step that follows an approximate search: exact distances between each
 * query and its candidates, the k nearest kept.  Mirrors cuVS c/include/cuvs/neighbors/refine.h:22-62.
 */
#ifndef CUVS_AMD_NEIGHBORS_REFINE_H
#define CUVS_AMD_NEIGHBORS_REFINE_H

#include <cuvs/core/c_api.h>
#include <cuvs/distance/distance.h>
#include <dlpack/dlpack.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/**
 * (c/include/cuvs/neighbors/refine.h:52-58, implementation c/src/neighbors/refine.cpp:62-135)
 *
 * dataset [n_rows, dim] and queries [n_queries, dim] of one element type (float32, float16, int8,
 * uint8), candidates int64 [n_queries, n_candidates], indices int64 [n_queries, k], distances
 * float32 [n_queries, k], k <= n_candidates.  The tensors are either all accessible from the
 * device (device, managed or pinned host memory) or all in plain host memory (kDLCPU); host
 * matrices are staged through the device, a batch of queries at a time, and the call returns when
 * the outputs are complete.  Candidate ids outside [0, n_rows) are skipped; rows of the output
 * that cannot be filled hold id -1 and the largest float.
 */
CUVS_EXPORT cuvsError_t cuvsRefine(cuvsResources_t res,
                                   DLManagedTensor* dataset,
                                   DLManagedTensor* queries,
                                   DLManagedTensor* candidates,
                                   cuvsDistanceType metric,
                                   DLManagedTensor* indices,
                                   DLManagedTensor* distances);

#ifdef __cplusplus
}
#endif
#endif
