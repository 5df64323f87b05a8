/*
 * Element-type tags of `lut_dtype`, `internal_distance_dtype` and `coarse_search_dtype`.
 * cuVS takes these as cudaDataType_t; the names and numeric values are kept
 * (32F = 0, 16F = 2, 8I = 3, 8U = 8; hipDataType uses the same numbers).
 */
#ifndef CUVS_AMD_DATA_TYPE_H
#define CUVS_AMD_DATA_TYPE_H

typedef enum {
  CUDA_R_32F = 0,
  CUDA_R_16F = 2,
  CUDA_R_8I  = 3,
  CUDA_R_8U  = 8,
} cudaDataType_t;

#endif
