/*
 * Core C ABI: resources handle, stream control, error reporting, device allocation.
 * Each declaration replaces the cuVS entry point of the same name
 * (c/include/cuvs/core/c_api.h, implementation c/src/core/c_api.cpp); the stream type is a
 * HIP stream instead of a CUDA stream.
 */
#ifndef CUVS_AMD_C_API_H
#define CUVS_AMD_C_API_H

#include <stddef.h>
#include <stdint.h>

#include <hip/hip_runtime_api.h>

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
/** c_api.h:175 -- caps the size of the cached workspace to the given percentage of device memory. */
CUVS_EXPORT cuvsError_t cuvsResourcesSetWorkspacePool(cuvsResources_t res, int percent_of_free_memory);
/** c_api.h:230 */
CUVS_EXPORT cuvsError_t cuvsRMMAlloc(cuvsResources_t res, void** ptr, size_t bytes);
/** c_api.h:240 */
CUVS_EXPORT cuvsError_t cuvsRMMFree(cuvsResources_t res, void* ptr, size_t bytes);
/** c_api.h:301 */
CUVS_EXPORT cuvsError_t cuvsVersionGet(uint16_t* major, uint16_t* minor, uint16_t* patch);

#ifdef __cplusplus
}
#endif
#endif
