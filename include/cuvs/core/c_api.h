/*
 * Core C ABI: resources handle, stream control, error reporting, device allocation.
 * Each declaration replaces the cuVS entry point of the same name
 * (c/include/cuvs/core/c_api.h, implementation c/src/core/c_api.cpp); the stream type is a
 * HIP stream instead of a CUDA stream.
 */
#ifndef CUVS_AMD_C_API_H
#define CUVS_AMD_C_API_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#include <hip/hip_runtime_api.h>

#include <dlpack/dlpack.h>

#include <cuvs/core/data_type.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CUVS_EXPORT __attribute__((visibility("default")))

/** The stream handle exchanged with callers is a HIP stream. */
typedef hipStream_t cudaStream_t;

/** c_api.h:27 */
typedef enum { CUVS_ERROR = 0, CUVS_SUCCESS = 1 } cuvsError_t;

/** c_api.h:32 -- text of the last error on this thread, NULL when the last call succeeded. */
CUVS_EXPORT const char* cuvsGetLastErrorText(void);
/** c_api.h:38 */
CUVS_EXPORT void cuvsSetLastErrorText(const char* error);

/** c_api.h:51-67 */
typedef enum {
  CUVS_LOG_LEVEL_TRACE    = 0,
  CUVS_LOG_LEVEL_DEBUG    = 1,
  CUVS_LOG_LEVEL_INFO     = 2,
  CUVS_LOG_LEVEL_WARN     = 3,
  CUVS_LOG_LEVEL_ERROR    = 4,
  CUVS_LOG_LEVEL_CRITICAL = 5,
  CUVS_LOG_LEVEL_OFF      = 6
} cuvsLogLevel_t;
CUVS_EXPORT cuvsLogLevel_t cuvsGetLogLevel(void);
CUVS_EXPORT void cuvsSetLogLevel(cuvsLogLevel_t level);

/** c_api.h:80 -- opaque handle: one stream plus a reusable device workspace. Not thread-safe. */
typedef uintptr_t cuvsResources_t;

/** c_api.h:88 */
CUVS_EXPORT cuvsError_t cuvsResourcesCreate(cuvsResources_t* res);
/** c_api.h:113 -- a handle like cuvsResourcesCreate's that also counts every allocation and release
 *  the library makes (device memory from any of the three sources, pinned host memory) until it is
 *  destroyed, and writes samples to `csv_path` from a background thread: the header at once, then a
 *  row after each burst of activity, at least `sample_interval_ms` apart, flushed as written, and a
 *  last row on destruction.  Columns: elapsed_ms, device_current_bytes, device_peak_bytes,
 *  pinned_current_bytes, pinned_peak_bytes, allocations, deallocations.  One at a time per process. */
CUVS_EXPORT cuvsError_t cuvsResourcesCreateWithMemoryTracking(cuvsResources_t* res, const char* csv_path,
                                                              int64_t sample_interval_ms);
/** c_api.h:123 */
CUVS_EXPORT cuvsError_t cuvsResourcesDestroy(cuvsResources_t res);
/** c_api.h:133 */
CUVS_EXPORT cuvsError_t cuvsStreamSet(cuvsResources_t res, cudaStream_t stream);
/** c_api.h:142 */
CUVS_EXPORT cuvsError_t cuvsStreamGet(cuvsResources_t res, cudaStream_t* stream);
/** c_api.h:150 */
CUVS_EXPORT cuvsError_t cuvsStreamSync(cuvsResources_t res);
/** c_api.h:159 */
CUVS_EXPORT cuvsError_t cuvsDeviceIdGet(cuvsResources_t res, int* device_id);
/** c_api.h:175 -- gives the handle a device memory pool of its own: `initial_size_bytes` are
 *  reserved now, the pool grows on demand and never shrinks before the handle is destroyed.  The
 *  handle's search workspace and cuvsRMMAlloc / cuvsRMMFree on it are then served from the pool. */
CUVS_EXPORT cuvsError_t cuvsResourcesSetWorkspacePool(cuvsResources_t res, size_t initial_size_bytes);
/** c_api.h:184-214 -- handles over several GPUs of one process.  This library drives one GPU: the
 *  four calls exist so that callers of the whole C API link, and every one of them fails with
 *  CUVS_ERROR and a message that says so (row-sharded search across GPUs is a merge of per-GPU
 *  answers, cuvsAmdKnnMergeParts; the exchange itself is the caller's). */
CUVS_EXPORT cuvsError_t cuvsMultiGpuResourcesCreate(cuvsResources_t* res);
CUVS_EXPORT cuvsError_t cuvsMultiGpuResourcesCreateWithDeviceIds(cuvsResources_t* res, DLManagedTensor* device_ids);
CUVS_EXPORT cuvsError_t cuvsMultiGpuResourcesDestroy(cuvsResources_t res);
CUVS_EXPORT cuvsError_t cuvsMultiGpuResourcesSetMemoryPool(cuvsResources_t res, int percent_of_free_memory);
/** c_api.h:230 -- device memory, ordered on the handle's stream. */
CUVS_EXPORT cuvsError_t cuvsRMMAlloc(cuvsResources_t res, void** ptr, size_t bytes);
/** c_api.h:240 */
CUVS_EXPORT cuvsError_t cuvsRMMFree(cuvsResources_t res, void* ptr, size_t bytes);
/** c_api.h:256 -- from now on the whole process (cuvsRMMAlloc and the library's own buffers)
 *  draws device memory from one pool: `initial_pool_size_percent` of the free memory reserved at
 *  once, growing up to `max_pool_size_percent`; `managed` takes the pool's blocks from
 *  hipMallocManaged.  Memory handed out before stays valid and is released where it came from. */
CUVS_EXPORT cuvsError_t cuvsRMMPoolMemoryResourceEnable(int initial_pool_size_percent,
                                                        int max_pool_size_percent, bool managed);
/** c_api.h:270 -- cuvsRMMAlloc / cuvsRMMFree become hipMallocAsync / hipFreeAsync on the handle's stream. */
CUVS_EXPORT cuvsError_t cuvsRMMAsyncMemoryResourceEnable(void);
/** c_api.h:276 -- back to plain hipMalloc / hipFree. */
CUVS_EXPORT cuvsError_t cuvsRMMMemoryResourceReset(void);
/** c_api.h:284 -- pinned host memory. */
CUVS_EXPORT cuvsError_t cuvsRMMHostAlloc(void** ptr, size_t bytes);
/** c_api.h:292 */
CUVS_EXPORT cuvsError_t cuvsRMMHostFree(void* ptr, size_t bytes);
/** c_api.h:301 */
CUVS_EXPORT cuvsError_t cuvsVersionGet(uint16_t* major, uint16_t* minor, uint16_t* patch);
/** c_api.h:318 -- copies `src` into the allocated `dst` of the same shape and dtype on the handle's
 *  stream; either side may be host or device memory, and 2-D tensors may have padded rows. */
CUVS_EXPORT cuvsError_t cuvsMatrixCopy(cuvsResources_t res, DLManagedTensor* src, DLManagedTensor* dst);
/** c_api.h:329 -- makes `dst` a view of rows [start, end) of the 1-D or 2-D `src` (no copy); the
 *  view's deleter frees the shape and stride arrays it owns. */
CUVS_EXPORT cuvsError_t cuvsMatrixSliceRows(cuvsResources_t res, DLManagedTensor* src, int64_t start,
                                            int64_t end, DLManagedTensor* dst);

#ifdef __cplusplus
}
#endif
#endif
