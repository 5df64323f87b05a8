/*
 * CPU oracle for IVF-PQ search -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain C++ restatement of the search semantics of NVIDIA cuVS
 * (cpp/src/neighbors/ivf_pq/ivf_pq_search.cuh and the kernel fragments under
 * cpp/src/neighbors/ivf_pq/detail/jit_lto_kernels/).  It exists so that the HIP
 * engine can be checked against an independent implementation; nothing in the
 * shipped library includes, links or calls it.  Only the tests, the smoke check
 * and the benchmark's CPU-baseline leg may use it.
 *
 * All entry points are extern "C" with plain pointers so that ctypes can drive
 * them.  Every pointer is a host pointer.
 */
#ifndef IVF_PQ_ORACLE_H
#define IVF_PQ_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* numeric values follow cuvs::distance::DistanceType (c/include/cuvs/distance/distance.h:15-60) */
enum { ORC_L2Expanded = 0, ORC_L2SqrtExpanded = 1, ORC_CosineExpanded = 2, ORC_InnerProduct = 6 };
/* numeric values follow cudaDataType_t / hipDataType as used by search_params */
enum { ORC_R_32F = 0, ORC_R_16F = 2, ORC_R_8I = 3, ORC_R_8U = 8 };
/* codebook_gen (cpp/include/cuvs/neighbors/ivf_pq.hpp:36-39) */
enum { ORC_PER_SUBSPACE = 0, ORC_PER_CLUSTER = 1 };
/* element type of query / dataset rows */
enum { ORC_T_F32 = 0, ORC_T_F16 = 1, ORC_T_I8 = 2, ORC_T_U8 = 3 };

typedef struct {
  int32_t metric;
  int32_t codebook_kind;
  uint32_t n_lists;
  uint32_t dim;
  uint32_t pq_dim;
  uint32_t pq_bits;
  const float* centers;            /* [n_lists, dim_ext], column `dim` holds the squared norm */
  const float* centers_rot;        /* [n_lists, rot_dim] */
  const float* rotation_matrix;    /* [rot_dim, dim] */
  const float* pq_centers;         /* [pq_dim | n_lists, pq_len, 1 << pq_bits] */
  const uint32_t* list_sizes;      /* [n_lists] */
  const uint8_t* const* list_data; /* [n_lists] interleaved codes of each list */
  const int64_t* const* list_inds; /* [n_lists] source ids of each list */
} orc_index;

typedef struct {
  uint32_t n_probes;
  int32_t lut_dtype;               /* ORC_R_32F | ORC_R_16F | ORC_R_8U */
  int32_t internal_distance_dtype; /* ORC_R_32F | ORC_R_16F */
  int32_t coarse_search_dtype;     /* ORC_R_32F | ORC_R_16F | ORC_R_8I */
} orc_search_params;

/* derived dimensions (cpp/src/neighbors/ivf_pq_index.cu:78-111) */
uint32_t orc_dim_ext(uint32_t dim);
uint32_t orc_pq_len(uint32_t dim, uint32_t pq_dim);
uint32_t orc_rot_dim(uint32_t dim, uint32_t pq_dim);

/* scalar conversions */
uint16_t orc_float_to_half(float v);
float orc_half_to_float(uint16_t h);
uint16_t orc_half_add(uint16_t a, uint16_t b);
uint8_t orc_fp8_encode(float v, int is_signed);
float orc_fp8_decode(uint8_t u, int is_signed);
uint16_t orc_fp8_decode_half(uint8_t u, int is_signed);

/* interleaved list layout (cpp/include/cuvs/neighbors/ivf_pq.hpp:222-296,
 * cpp/src/neighbors/ivf_pq/ivf_pq_codepacking.cuh:29-168) */
uint64_t orc_list_bytes(uint32_t n_rows, uint32_t pq_dim, uint32_t pq_bits);
void orc_pack_list(const uint8_t* codes, uint32_t n_rows, uint32_t pq_dim, uint32_t pq_bits,
                   uint32_t row_offset, uint8_t* list_data);
void orc_unpack_list(const uint8_t* list_data, uint32_t n_rows, uint32_t pq_dim, uint32_t pq_bits,
                     uint32_t row_offset, uint8_t* codes);
/* bit-contiguous rows of ceil(pq_dim*pq_bits/8) bytes each */
void orc_unpack_list_contiguous(const uint8_t* list_data, uint32_t n_rows, uint32_t pq_dim,
                                uint32_t pq_bits, uint32_t row_offset, uint8_t* out);

/* coarse probe selection only: probes[n_queries, n_probes], ascending (score, list id) */
int orc_select_clusters(const orc_index* index, const orc_search_params* params,
                        const void* queries, int query_type, uint32_t n_queries,
                        uint32_t* probes, float* probe_scores, int n_threads);

/* lookup table of one (query, list) pair, stored in the LUT element type:
 * 4, 2 or 1 bytes per entry, [pq_dim << pq_bits] entries */
int orc_make_lut(const orc_index* index, const orc_search_params* params, const void* query,
                 int query_type, uint32_t label, void* lut_out);

/* full search; neighbors/distances are [n_queries, k], each row ascending by
 * (internal score, sample id).  filter_bitset may be NULL (no filter); bit i set = row id i kept. */
int orc_search(const orc_index* index, const orc_search_params* params, const void* queries,
               int query_type, uint32_t n_queries, uint32_t k, const uint32_t* filter_bitset,
               int64_t filter_nbits, int64_t* neighbors, float* distances, uint32_t* probes_out,
               int n_threads);

/* encode: labels by the coarse quantiser, then per-subspace nearest codebook entry
 * (cpp/src/neighbors/ivf_pq/ivf_pq_build.cuh:140-206, ivf_pq_process_and_fill_codes.cuh:84-126) */
int orc_encode(const orc_index* index, const void* rows, int row_type, uint64_t n_rows,
               uint32_t* labels, uint8_t* codes, int n_threads);

/* refinement (cpp/src/neighbors/refine/refine_device.cuh:35-135, refine_host.hpp): exact distance of
 * every query to each of its candidate rows, the k best kept in ascending (distance, candidate
 * slot) order.  metric: ORC_L2Expanded (squared), ORC_L2SqrtExpanded, ORC_InnerProduct (largest
 * first).  fp32 / fp16 rows accumulate in fp32 ascending dimension; int8 / uint8 rows in exact
 * 32-bit integers, as the reference's accumulator types for them.  Candidates outside [0, n_rows)
 * are skipped; unfilled outputs hold id -1 and FLT_MAX. */
int orc_refine(const void* dataset, const void* queries, int row_type, int64_t n_rows,
               uint32_t n_queries, uint32_t dim, const int64_t* candidates, uint32_t n_candidates,
               uint32_t k, int metric, int64_t* indices, float* distances);

const char* orc_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
