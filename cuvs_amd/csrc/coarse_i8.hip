/*
 * Coarse search in 8-bit integers (select_clusters for int8_t,
 * cpp/src/neighbors/ivf_pq/ivf_pq_search.cuh:170-256; centres quantised as in
 * cpp/src/neighbors/ivf_pq_index.cu:661-738): an experimental mode of the reference.
 *
 * Rows have dim_ext_int8 = round_up(dim + 2, 16) columns.  Centre side: column c < dim holds
 * trunc(clamp(128 c)); the squared norm x is split as y = clamp(x * 64 / (m - 1)) with
 * m = dim_ext_int8 - dim: the columns past `dim` hold round(y), column `dim` holds
 * trunc(clamp(128 (y - round(y)))).  Query side: trunc(clamp(128 q)) of the mapped element (which
 * is x >> 1 for uint8 and x for int8 elements), 1 - m in column `dim`, then -128 (L2) or 0 (inner
 * product, cosine).  The score is alpha times the integer dot product, alpha = -2 (L2) or -1.
 *
 * The query rows are padded to the same dim_ext_int8 columns: the reference's driver takes the row
 * length of the int8 centre matrix as `dim_ext` for this mode (ivf_pq_search.cuh:929-931).
 *
 * Scores leave this file as floats whose order (as the selection kernels see it through
 * order_f32) is the order of the int32 scores, so that the probe selection is shared with the
 * other precisions and ranks by (integer score, list) exactly.
 */
#include "device_utils.cuh"

#define CUVS_LAUNCH_CHECK() CUVS_HIP_TRY(hipGetLastError())

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

constexpr uint32_t kI8Threads = 256;
constexpr uint32_t kI8Queries = 16;  // queries per block

__device__ __forceinline__ int clamp_i8(float v)
{
  return int(fmaxf(-128.0f, fminf(127.0f, v)));  // conversion truncates toward zero
}

/** ct8[w][l]: bytes 4w .. 4w+3 of list l's quantised row, lists padded to l_pad with zero rows. */
__global__ void pack_centers_i8_kernel(const float* __restrict__ centers, uint32_t n_lists,
                                       uint32_t dim, uint32_t dim_ext, uint32_t l_pad,
                                       uint32_t n_words, uint32_t* __restrict__ ct8)
{
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= uint64_t(n_words) * l_pad) { return; }
  const uint32_t w = uint32_t(i / l_pad);
  const uint32_t l = uint32_t(i - uint64_t(w) * l_pad);
  uint32_t word    = 0;
  if (l < n_lists) {
    const float* row = centers + uint64_t(l) * dim_ext;
    const float x    = row[dim];
    const float f    = 64.0f / float(n_words * 4u - dim - 1u);
    const float y    = fmaxf(-128.0f, fminf(127.0f, x * f));
    const float ry   = roundf(y);
    const float z    = fmaxf(-128.0f, fminf(127.0f, (y - ry) * 128.0f));
#pragma unroll
    for (uint32_t b = 0; b < 4; b++) {
      const uint32_t d = w * 4u + b;
      const int v      = d < dim ? clamp_i8(row[d] * 128.0f) : (d == dim ? int(z) : int(ry));
      word |= (uint32_t(v) & 0xFFu) << (8u * b);
    }
  }
  ct8[i] = word;
}

/** Float whose order_f32 key grows with the int32 score.  Key 0x7FFFFFFF is skipped: it is the
 *  pattern of -0, which order_f32 folds into +0. */
__device__ __forceinline__ float score_as_ordered_float(int32_t s)
{
  uint32_t k = uint32_t(s) ^ 0x80000000u;
  k += k >= 0x7FFFFFFFu ? 1u : 0u;
  return unorder_f32(k);
}

__global__ __launch_bounds__(kI8Threads) void coarse_scores_i8_kernel(
  const float* __restrict__ qf, const uint32_t* __restrict__ ct8, uint32_t n_queries,
  uint32_t n_lists, uint32_t l_pad, uint32_t dim, uint32_t n_words, int ip_like,
  float* __restrict__ scores)
{
  extern __shared__ __align__(16) unsigned char dyn_smem[];
  uint32_t* sq      = reinterpret_cast<uint32_t*>(dyn_smem);  // [kI8Queries][n_words]
  const uint32_t q0 = blockIdx.y * kI8Queries;
  const uint32_t l  = blockIdx.x * kI8Threads + threadIdx.x;
  const int m       = int(n_words * 4u - dim);
  const int nf      = ip_like ? 0 : -128;
  for (uint32_t i = threadIdx.x; i < kI8Queries * n_words; i += kI8Threads) {
    const uint32_t qi = i / n_words;
    const uint32_t w  = i - qi * n_words;
    uint32_t word     = 0;
    if (q0 + qi < n_queries) {
#pragma unroll
      for (uint32_t b = 0; b < 4; b++) {
        const uint32_t d = w * 4u + b;
        const int v      = d < dim ? clamp_i8(qf[uint64_t(q0 + qi) * dim + d] * 128.0f)
                                   : (d == dim ? 1 - m : nf);
        word |= (uint32_t(v) & 0xFFu) << (8u * b);
      }
    }
    sq[i] = word;
  }
  __syncthreads();
  int acc[kI8Queries];
#pragma unroll
  for (uint32_t qi = 0; qi < kI8Queries; qi++) { acc[qi] = 0; }
  for (uint32_t w = 0; w < n_words; w++) {
    const int c = l < l_pad ? int(ct8[uint64_t(w) * l_pad + l]) : 0;
#pragma unroll
    for (uint32_t qi = 0; qi < kI8Queries; qi++) {
      acc[qi] = __builtin_amdgcn_sdot4(c, int(sq[qi * n_words + w]), acc[qi], false);
    }
  }
  if (l >= n_lists) { return; }
  const int alpha = ip_like ? -1 : -2;
#pragma unroll
  for (uint32_t qi = 0; qi < kI8Queries; qi++) {
    if (q0 + qi < n_queries) {
      scores[uint64_t(q0 + qi) * n_lists + l] = score_as_ordered_float(alpha * acc[qi]);
    }
  }
}

}  // namespace

uint32_t coarse_i8_words(uint32_t dim) { return round_up_u32(dim + 2u, 16u) / 4u; }

void launch_pack_centers_i8(const float* centers, uint32_t n_lists, uint32_t dim, uint32_t dim_ext,
                            uint32_t* ct8, hipStream_t stream)
{
  const uint32_t l_pad   = coarse_pad(n_lists);
  const uint32_t n_words = coarse_i8_words(dim);
  const uint64_t total   = uint64_t(n_words) * l_pad;
  pack_centers_i8_kernel<<<uint32_t((total + 255) / 256), 256, 0, stream>>>(centers, n_lists, dim, dim_ext,
                                                                            l_pad, n_words, ct8);
  CUVS_LAUNCH_CHECK();
}

void launch_coarse_scores_i8(const float* qf, const uint32_t* ct8, uint32_t n_queries, uint32_t n_lists,
                             uint32_t dim, bool ip_like, float* scores, hipStream_t stream)
{
  if (n_queries == 0) { return; }
  const uint32_t l_pad   = coarse_pad(n_lists);
  const uint32_t n_words = coarse_i8_words(dim);
  // the query tile lives in LDS; also keeps |score| <= 2 * 128 * 128 * 4 n_words far from the NaN
  // patterns at both ends of the key range
  const size_t smem = size_t(kI8Queries) * n_words * 4;
  CUVS_EXPECTS(smem <= 32 * 1024, "coarse_search_dtype = CUDA_R_8I supports dim <= 2030 (got %u)", dim);
  dim3 grid((n_lists + kI8Threads - 1) / kI8Threads, (n_queries + kI8Queries - 1) / kI8Queries);
  CUVS_EXPECTS(grid.y <= 65535u, "too many queries in one batch for the 8-bit coarse search");
  coarse_scores_i8_kernel<<<grid, kI8Threads, smem, stream>>>(qf, ct8, n_queries, n_lists, l_pad, dim,
                                                              n_words, ip_like ? 1 : 0, scores);
  CUVS_LAUNCH_CHECK();
}

}  // namespace cuvs::neighbors::ivf_pq::detail
