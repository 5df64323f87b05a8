/*
 * C ABI of the IVF-PQ search path for AMD Instinct MI355X (gfx950).
 *
 * Every declaration without the `cuvsAmd` prefix has the name, argument meaning and error
 * behaviour of the cuVS entry point it replaces; the comment above it cites that entry point
 * as  <file>:<line>  relative to the cuVS source tree (header c/include/cuvs/neighbors/ivf_pq.h,
 * implementation c/src/neighbors/ivf_pq.cpp).  Functions prefixed `cuvsAmd` have no counterpart
 * in the cuVS C API; each says which internal cuVS step it exposes and why.
 *
 * All functions return CUVS_SUCCESS (1) or CUVS_ERROR (0); after an error the message is
 * available on the calling thread through cuvsGetLastErrorText().  Tensors are borrowed for the
 * duration of the call.  Work is queued on the stream of the resources handle and is
 * asynchronous: call cuvsStreamSync() before reading results on the host.
 */
#ifndef CUVS_AMD_IVF_PQ_H
#define CUVS_AMD_IVF_PQ_H

#include <cuvs/core/c_api.h>
#include <cuvs/distance/distance.h>
#include <dlpack/dlpack.h>
#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/** ivf_pq.h:28-31 */
enum cuvsIvfPqCodebookGen {
  CUVS_IVF_PQ_CODEBOOK_GEN_PER_SUBSPACE = 0,
  CUVS_IVF_PQ_CODEBOOK_GEN_PER_CLUSTER  = 1,
};

/** ivf_pq.h:37-40 -- search requires INTERLEAVED */
enum cuvsIvfPqListLayout {
  CUVS_IVF_PQ_LIST_LAYOUT_FLAT        = 0,
  CUVS_IVF_PQ_LIST_LAYOUT_INTERLEAVED = 1,
};

/** ivf_pq.h:46-137 -- same fields in the same order.  The training knobs (kmeans_*,
 *  max_train_points_per_pq_code, add_data_on_build, force_random_rotation) are carried but unused:
 *  this library takes a trained model through cuvsIvfPqBuildPrecomputed. */
struct cuvsIvfPqIndexParams {
  cuvsDistanceType metric;
  float metric_arg;
  bool add_data_on_build;
  uint32_t n_lists;
  uint32_t kmeans_n_iters;
  double kmeans_trainset_fraction;
  uint32_t pq_bits;
  uint32_t pq_dim;
  enum cuvsIvfPqCodebookGen codebook_kind;
  bool force_random_rotation;
  bool conservative_memory_allocation;
  uint32_t max_train_points_per_pq_code;
  enum cuvsIvfPqListLayout codes_layout;
};
typedef struct cuvsIvfPqIndexParams* cuvsIvfPqIndexParams_t;

/** ivf_pq.h:146 -- defaults of c/src/neighbors/ivf_pq.cpp:348-365 */
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexParamsCreate(cuvsIvfPqIndexParams_t* index_params);
/** ivf_pq.h:153 */
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexParamsDestroy(cuvsIvfPqIndexParams_t index_params);

/** ivf_pq.h:165-219 -- same fields in the same order (this order differs from the C++ struct).
 *  lut_dtype: CUDA_R_32F | CUDA_R_16F | CUDA_R_8U.  internal_distance_dtype: CUDA_R_32F | CUDA_R_16F.
 *  coarse_search_dtype: CUDA_R_32F | CUDA_R_16F.  preferred_shmem_carveout is accepted and ignored
 *  (LDS is not carved out of a cache on CDNA). */
struct cuvsIvfPqSearchParams {
  uint32_t n_probes;
  cudaDataType_t lut_dtype;
  cudaDataType_t internal_distance_dtype;
  cudaDataType_t coarse_search_dtype;
  uint32_t max_internal_batch_size;
  double preferred_shmem_carveout;
};
typedef struct cuvsIvfPqSearchParams* cuvsIvfPqSearchParams_t;

/** ivf_pq.h:228 -- defaults of c/src/neighbors/ivf_pq.cpp:372-382 */
CUVS_EXPORT cuvsError_t cuvsIvfPqSearchParamsCreate(cuvsIvfPqSearchParams_t* params);
/** ivf_pq.h:235 */
CUVS_EXPORT cuvsError_t cuvsIvfPqSearchParamsDestroy(cuvsIvfPqSearchParams_t params);

/** ivf_pq.h:250-255 */
typedef struct {
  uintptr_t addr;
  DLDataType dtype;
} cuvsIvfPqIndex;
typedef cuvsIvfPqIndex* cuvsIvfPqIndex_t;

/** ivf_pq.h:262 */
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexCreate(cuvsIvfPqIndex_t* index);
/** ivf_pq.h:268 */
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexDestroy(cuvsIvfPqIndex_t index);

/** ivf_pq.h:271-288 -- scalar getters */
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetNLists(cuvsIvfPqIndex_t index, int64_t* n_lists);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetDim(cuvsIvfPqIndex_t index, int64_t* dim);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetSize(cuvsIvfPqIndex_t index, int64_t* size);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetPqDim(cuvsIvfPqIndex_t index, int64_t* pq_dim);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetPqBits(cuvsIvfPqIndex_t index, int64_t* pq_bits);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetPqLen(cuvsIvfPqIndex_t index, int64_t* pq_len);

/** ivf_pq.h:296-351 -- non-owning device views.  The `shape`/`strides` arrays are allocated by the
 *  library and released by the tensor's `deleter`. */
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetCenters(cuvsIvfPqIndex_t index, DLManagedTensor* centers);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetCentersPadded(cuvsIvfPqIndex_t index,
                                                       DLManagedTensor* centers);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetPqCenters(cuvsIvfPqIndex_t index,
                                                   DLManagedTensor* pq_centers);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetCentersRot(cuvsIvfPqIndex_t index,
                                                    DLManagedTensor* centers_rot);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetRotationMatrix(cuvsIvfPqIndex_t index,
                                                        DLManagedTensor* rotation_matrix);
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetListSizes(cuvsIvfPqIndex_t index,
                                                   DLManagedTensor* list_sizes);

/** ivf_pq.h:370-374 -- bit-contiguous codes of rows [offset, offset + n_rows) of one list:
 *  out_codes is a device uint8 matrix [n_rows, ceil(pq_dim * pq_bits / 8)]. */
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexUnpackContiguousListData(cuvsResources_t res,
                                                               cuvsIvfPqIndex_t index,
                                                               DLManagedTensor* out_codes,
                                                               uint32_t label,
                                                               uint32_t offset);
/** ivf_pq.h:384-386 -- int64 source ids of one list (view of length list size). */
CUVS_EXPORT cuvsError_t cuvsIvfPqIndexGetListIndices(cuvsIvfPqIndex_t index,
                                                     uint32_t label,
                                                     DLManagedTensor* out_labels);

/** ivf_pq.h:455-462 -- index from a trained model held in device memory: pq_centers
 *  [pq_dim | n_lists, pq_len, 1 << pq_bits], centers [n_lists, round_up(dim + 1, 8)] (column `dim`
 *  holds the squared norm), centers_rot [n_lists, pq_len * pq_dim], rotation_matrix
 *  [pq_len * pq_dim, dim]; all float32.  The model tensors are copied (the reference keeps views
 *  and asks the caller to keep them alive; copying is the safe superset).  The index starts empty;
 *  populate it with cuvsIvfPqExtend. */
CUVS_EXPORT cuvsError_t cuvsIvfPqBuildPrecomputed(cuvsResources_t res,
                                                  cuvsIvfPqIndexParams_t params,
                                                  uint32_t dim,
                                                  DLManagedTensor* pq_centers,
                                                  DLManagedTensor* centers,
                                                  DLManagedTensor* centers_rot,
                                                  DLManagedTensor* rotation_matrix,
                                                  cuvsIvfPqIndex_t index);

/** ivf_pq.h:426-429 -- trains an index on `dataset` ([n_rows, dim] of float32, float16, int8 or
 *  uint8, in device or host memory) and, with params->add_data_on_build, adds the dataset to it. */
CUVS_EXPORT cuvsError_t cuvsIvfPqBuild(cuvsResources_t res,
                                       cuvsIvfPqIndexParams_t params,
                                       DLManagedTensor* dataset,
                                       cuvsIvfPqIndex_t index);

/** ivf_pq.h:536-541 -- the hot path.  queries: device [n_queries, dim] row-major of float32,
 *  float16, int8 or uint8; neighbors: device int64 [n_queries, k]; distances: device float32
 *  [n_queries, k]; k is neighbors.shape[1].  Rows come back ordered by ascending internal score
 *  (the reference leaves the order unspecified).  Slots that cannot be filled hold INT64_MAX. */
CUVS_EXPORT cuvsError_t cuvsIvfPqSearch(cuvsResources_t res,
                                        cuvsIvfPqSearchParams_t search_params,
                                        cuvsIvfPqIndex_t index,
                                        DLManagedTensor* queries,
                                        DLManagedTensor* neighbors,
                                        DLManagedTensor* distances);

/** ivf_pq.h:565 and :574 */
CUVS_EXPORT cuvsError_t cuvsIvfPqSerialize(cuvsResources_t res,
                                           const char* filename,
                                           cuvsIvfPqIndex_t index);
CUVS_EXPORT cuvsError_t cuvsIvfPqDeserialize(cuvsResources_t res,
                                             const char* filename,
                                             cuvsIvfPqIndex_t index);

/** ivf_pq.h:591-594 -- encode new_vectors [n, dim] (device or host; float32, float16, int8, uint8)
 *  and append them with their int64 ids (NULL = consecutive ids continuing from the index size). */
CUVS_EXPORT cuvsError_t cuvsIvfPqExtend(cuvsResources_t res,
                                        DLManagedTensor* new_vectors,
                                        DLManagedTensor* new_indices,
                                        cuvsIvfPqIndex_t index);

/** ivf_pq.h:612-616 -- list labels (uint32 [n]) and bit-contiguous codes
 *  (uint8 [n, ceil(pq_dim * pq_bits / 8)]) of the input vectors, without touching the index. */
CUVS_EXPORT cuvsError_t cuvsIvfPqTransform(cuvsResources_t res,
                                           cuvsIvfPqIndex_t index,
                                           DLManagedTensor* input_dataset,
                                           DLManagedTensor* output_labels,
                                           DLManagedTensor* output_dataset);

/* ------------------------------------------------------------------------------------------ */
/* Entry points without a counterpart in the cuVS C API.                                       */
/* ------------------------------------------------------------------------------------------ */

/** Coarse step of the search on its own: clusters_to_probe is a device uint32
 *  [n_queries, min(n_probes, n_lists)] matrix, each row ascending by (coarse score, list id).
 *  Exposes cuVS's internal select_clusters (cpp/src/neighbors/ivf_pq/ivf_pq_search.cuh:60-168) so
 *  that probe lists can be compared bit for bit with an external implementation. */
CUVS_EXPORT cuvsError_t cuvsAmdIvfPqSelectClusters(cuvsResources_t res,
                                                   cuvsIvfPqSearchParams_t search_params,
                                                   cuvsIvfPqIndex_t index,
                                                   DLManagedTensor* queries,
                                                   DLManagedTensor* clusters_to_probe);

/** cuvsIvfPqSearch restricted by a bitset over source ids (bit i set = id i may be returned):
 *  the C form of the C++ overload that takes cuvs::neighbors::filtering::bitset_filter
 *  (cpp/include/cuvs/neighbors/ivf_pq.hpp:1821-1963).  bitset: device uint32 [ceil(n_bits / 32)]. */
CUVS_EXPORT cuvsError_t cuvsAmdIvfPqSearchWithBitset(cuvsResources_t res,
                                                     cuvsIvfPqSearchParams_t search_params,
                                                     cuvsIvfPqIndex_t index,
                                                     DLManagedTensor* queries,
                                                     DLManagedTensor* neighbors,
                                                     DLManagedTensor* distances,
                                                     DLManagedTensor* bitset,
                                                     int64_t n_bits);

/** cuvsIvfPqSearch for callers that cannot allocate device memory: code under HIP graph capture,
 *  tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the cuVS C API.  Same
 *  arguments, checks and results as cuvsIvfPqSearch (it runs the same kernels on the stream of
 *  `res`), but the workspace between the stages of the search is a fixed array of
 *  CUVS_AMD_NO_ALLOC_WORKSPACE_BYTES in the library's device image instead of the handle's cached
 *  allocation, and the call makes no hipMalloc / hipFree.  The queries run in internal batches
 *  that fit that array (roughly 4 * n_lists + 32 * n_probes * k + 100 * n_probes + 12 * dim bytes
 *  per query: a few hundred queries a batch at 16384 lists, 64 probes, k = 10; results do not
 *  depend on the batching); only a single query that does not fit fails, with a message that
 *  states the bytes needed.  Every GPU holds one such array: calls on different streams take
 *  turns on it (each waits for an event recorded behind the call before it, except under stream
 *  capture); calls issued by several host threads at once, and captured calls replayed side by
 *  side, race on it.  Profiling (cuvsAmdIvfPqProfilingEnable) does not apply to this call. */
#define CUVS_AMD_NO_ALLOC_WORKSPACE_BYTES ((size_t)32 << 20)
CUVS_EXPORT cuvsError_t cuvsAmdIvfPqSearchNoAlloc(cuvsResources_t res,
                                                  cuvsIvfPqSearchParams_t search_params,
                                                  cuvsIvfPqIndex_t index,
                                                  DLManagedTensor* queries,
                                                  DLManagedTensor* neighbors,
                                                  DLManagedTensor* distances);

/** cuvsIvfPqExtend with list labels chosen by the caller (device uint32 [n]) instead of the
 *  library's own nearest-centre assignment; the C form of extending lists the way the C++ helper
 *  cuvs::neighbors::ivf_pq::helpers::extend_list does for pre-assigned rows.  For callers that
 *  assign lists themselves (e.g. with a faster approximate assignment). */
CUVS_EXPORT cuvsError_t cuvsAmdIvfPqExtendLabeled(cuvsResources_t res,
                                                  DLManagedTensor* new_vectors,
                                                  DLManagedTensor* new_indices,
                                                  DLManagedTensor* labels,
                                                  cuvsIvfPqIndex_t index);

/** Per-stage device times of the most recent search on this resources handle, measured with HIP
 *  events on the handle's stream, and the algorithmic size of the scanned code stream.  Counterpart
 *  of the NVTX ranges cuVS wraps around the same stages (ivf_pq_search.cuh:74-79,436-441). */
typedef struct {
  uint32_t n_queries;
  uint32_t n_probes;
  uint32_t k;
  uint32_t n_scan_launches;  /* launches of the LUT + code-scan kernel */
  float coarse_ms;           /* query mapping, centre scores, probe selection */
  float rotate_ms;           /* rotation, chunk indices, pair ordering */
  float scan_ms;             /* LUT construction + code scan + per-pair top-k */
  float merge_ms;            /* per-query merge, distance and id post-processing */
  float total_ms;
  uint64_t scan_bytes; /* sum over (query, probe) of round_up(list size, 32) * bytes per row */
  uint64_t scan_rows;  /* sum over (query, probe) of list size */
  /* L2 early stop (all zero when the search did not use it): the scan stage is three launches */
  float lead_scan_ms;      /* full scan of each query's leading probes + bound per query */
  float screen_ms;         /* first-chunk screening of all other pairs */
  float survivor_scan_ms;  /* full scan of the pairs the screen kept */
  uint32_t scan_kernel;    /* which kernel scanned pairs in full: 0 scan_kernel (generic), 1 scan_stream_kernel,
                              2 scan_fast_kernel, 3 scan_direct_kernel, 4 scan_nibble_kernel,
                              5 scan_nibble_pack_kernel, 6 scan_slab_kernel */
  uint64_t lead_bytes;     /* scan_bytes share of the leading pairs */
  uint64_t screen_bytes;   /* sum over screened pairs of round_up(list size, 32) * bytes read per row (8) */
  uint64_t survivor_bytes; /* scan_bytes share of the pairs the screen kept */
  uint64_t n_screened_pairs;
  uint64_t n_surviving_pairs;
  uint64_t n_far_pairs;    /* screened pairs dropped without reading a row: |query - centre| minus the
                              list's radius already lies past the query's bound */
} cuvsAmdIvfPqSearchProfile;

/** Choices the search otherwise makes by itself, fixed on one resources handle: for measurements
 *  and tests that compare the library's code paths (no result depends on them).
 *  early_stop: 0 = the library decides per batch whether the L2 early stop (leading lists in full,
 *  the others screened on their leading codes, survivors in full) pays; 1 = never, every probed
 *  list is streamed in full by the scan kernel; 2 = whenever the search's parameters allow it.
 *  generic_scan != 0: every search goes through the generic scan kernel.  plain_coarse != 0: coarse
 *  search by the fp32 contraction and selection instead of the two-precision selection.
 *  serial_batches != 0: the internal batches of a search (max_internal_batch_size) run one after the
 *  other on the handle's stream; by default up to four of them run side by side on streams of the
 *  handle's own, each with its own workspace, and the handle's stream continues after all of them. */
typedef struct {
  int32_t early_stop;
  int32_t generic_scan;
  int32_t plain_coarse;
  int32_t serial_batches;
  int32_t reserved_[4]; /* zero */
} cuvsAmdIvfPqSearchTuning;
CUVS_EXPORT cuvsError_t cuvsAmdIvfPqSetSearchTuning(cuvsResources_t res,
                                                    const cuvsAmdIvfPqSearchTuning* tuning);

/** Turn event timing of the search stages on or off (off by default: timing adds event records and
 *  one device reduction per search). */
CUVS_EXPORT cuvsError_t cuvsAmdIvfPqProfilingEnable(cuvsResources_t res, bool enable);
/** Synchronises the stream and reads the profile of the last search made with profiling on. */
CUVS_EXPORT cuvsError_t cuvsAmdIvfPqGetSearchProfile(cuvsResources_t res,
                                                     cuvsAmdIvfPqSearchProfile* profile);

#ifdef __cplusplus
}
#endif
#endif
