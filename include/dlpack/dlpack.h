/*
 * Minimal DLPack tensor ABI (struct layout of DLPack v0.8, the version the cuVS C API
 * exchanges: c/include/cuvs/neighbors/ivf_pq.h:10 includes <dlpack/dlpack.h>).
 * Only the types that cross this library's C boundary are declared.
 */
#ifndef CUVS_AMD_DLPACK_H
#define CUVS_AMD_DLPACK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  kDLCPU         = 1,
  kDLCUDA        = 2,
  kDLCUDAHost    = 3,
  kDLROCM        = 10,
  kDLROCMHost    = 11,
  kDLCUDAManaged = 13,
} DLDeviceType;

typedef struct {
  DLDeviceType device_type;
  int32_t device_id;
} DLDevice;

typedef enum {
  kDLInt    = 0U,
  kDLUInt   = 1U,
  kDLFloat  = 2U,
  kDLBfloat = 4U,
} DLDataTypeCode;

typedef struct {
  uint8_t code;
  uint8_t bits;
  uint16_t lanes;
} DLDataType;

typedef struct {
  void* data;
  DLDevice device;
  int32_t ndim;
  DLDataType dtype;
  int64_t* shape;
  int64_t* strides; /* in elements; NULL means compact row-major */
  uint64_t byte_offset;
} DLTensor;

typedef struct DLManagedTensor {
  DLTensor dl_tensor;
  void* manager_ctx;
  void (*deleter)(struct DLManagedTensor* self);
} DLManagedTensor;

#ifdef __cplusplus
}
#endif
#endif
