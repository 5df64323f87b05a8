/*
 * Coarse scores on the matrix cores: scores[q, l] = alpha * sum_{d < dim_ext} q_ext[q, d] * c_ext[l, d]
 * with c_ext = stored centre rows (column `dim` holds ||c||^2, zero padding after it) and
 * q_ext = [mapped query, qnorm, 0 ...] (select_clusters, cpp/src/neighbors/ivf_pq/ivf_pq_search.cuh:60-168).
 *
 * v_mfma_f32_32x32x2_f32 accumulates its two k steps one after the other with a fused
 * multiply-add, so a chain of these instructions over ascending k gives each output exactly the
 * value of the scalar loop `acc = fmaf(c[d], q[d], acc)`: the result does not depend on tiling and
 * equals the vector-ALU kernel's bit for bit.  Trailing zero columns add exact zeros.
 *
 * Both operands are read k-major (`qt[d][query]`, `ct[d][list]`, leading dimensions padded to the
 * 128-wide block tile and zero-filled), so that global loads, LDS writes and the per-lane MFMA
 * operand reads are all contiguous across lanes.  A block of 4 waves computes 128 queries x 128
 * lists, each wave a 64 x 64 quadrant as 2 x 2 MFMA tiles; K advances in slabs of 8 through a
 * double-buffered 2 x 8 KB of LDS with one barrier per slab.
 */
#include "device_utils.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr uint32_t kGemmTile = 128;  // block tile in both directions
constexpr uint32_t kGemmSlab = 8;    // k values per LDS slab

__device__ __forceinline__ float round_half(float v) { return float(_Float16(v)); }

template <typename T>
__device__ __forceinline__ float map_value(T v);
template <>
__device__ __forceinline__ float map_value<float>(float v) { return v; }
template <>
__device__ __forceinline__ float map_value<_Float16>(_Float16 v) { return float(v); }
template <>
__device__ __forceinline__ float map_value<int8_t>(int8_t v) { return float(v) * (1.0f / 128.0f); }
template <>
__device__ __forceinline__ float map_value<uint8_t>(uint8_t v) { return float(v) * (1.0f / 256.0f); }

/** qt[d][q] for d < dim_ext, q < q_pad: mapped query elements, then qnorm, then zeros. */
template <typename T>
__global__ void map_queries_t_kernel(const T* __restrict__ in, uint32_t n_queries, uint32_t dim,
                                     uint32_t dim_ext, uint32_t q_pad, float qnorm,
                                     float* __restrict__ qt)
{
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= uint64_t(dim_ext) * q_pad) { return; }
  const uint32_t d = uint32_t(i / q_pad);
  const uint32_t q = uint32_t(i - uint64_t(d) * q_pad);
  float v          = 0.0f;
  if (q < n_queries) {
    if (d < dim) {
      v = map_value<T>(in[uint64_t(q) * dim + d]);
    } else if (d == dim) {
      v = qnorm;
    }
  }
  qt[i] = v;
}

/** ct[d][l] = centers[l][d] for l < n_lists, zero for the padding lists. */
__global__ void transpose_centers_kernel(const float* __restrict__ centers, uint32_t n_lists,
                                         uint32_t dim_ext, uint32_t l_pad, float* __restrict__ ct)
{
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= uint64_t(dim_ext) * l_pad) { return; }
  const uint32_t d = uint32_t(i / l_pad);
  const uint32_t l = uint32_t(i - uint64_t(d) * l_pad);
  ct[i]            = l < n_lists ? centers[uint64_t(l) * dim_ext + d] : 0.0f;
}

template <bool HALF>
__global__ __launch_bounds__(256, 2) void coarse_scores_mfma_kernel(const float* __restrict__ qt,
                                                                    const float* __restrict__ ct,
                                                                    uint32_t n_queries,
                                                                    uint32_t n_lists,
                                                                    uint32_t dim_ext, uint32_t q_pad,
                                                                    uint32_t l_pad, float alpha,
                                                                    float* __restrict__ scores)
{
  __shared__ __align__(16) float sa[2][kGemmSlab][kGemmTile];  // queries
  __shared__ __align__(16) float sb[2][kGemmSlab][kGemmTile];  // lists
  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = tid >> 6;
  const uint32_t wq   = wid >> 1;  // wave's query half of the block tile
  const uint32_t wl   = wid & 1u;  // wave's list half
  const uint32_t q0   = blockIdx.y * kGemmTile;
  const uint32_t l0   = blockIdx.x * kGemmTile;
  // loader role: one float4 of each operand per slab
  const uint32_t lk = tid >> 5;          // 0..7: k inside the slab
  const uint32_t lc = (tid & 31u) * 4u;  // column inside the tile
  const float* gq   = qt + uint64_t(lk) * q_pad + q0 + lc;
  const float* gc   = ct + uint64_t(lk) * l_pad + l0 + lc;

  v16f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
#pragma unroll
      for (int r = 0; r < 16; r++) { acc[i][j][r] = 0.0f; }
    }
  }

  const uint32_t n_slabs = dim_ext / kGemmSlab;  // dim_ext is a multiple of 8
  float4 pq = *reinterpret_cast<const float4*>(gq);
  float4 pc = *reinterpret_cast<const float4*>(gc);
  for (uint32_t s = 0; s < n_slabs; s++) {
    const uint32_t buf = s & 1u;
    if (HALF) {
      pq = make_float4(round_half(pq.x), round_half(pq.y), round_half(pq.z), round_half(pq.w));
      pc = make_float4(round_half(pc.x), round_half(pc.y), round_half(pc.z), round_half(pc.w));
    }
    *reinterpret_cast<float4*>(&sa[buf][lk][lc]) = pq;
    *reinterpret_cast<float4*>(&sb[buf][lk][lc]) = pc;
    __syncthreads();  // slab s visible; everyone is past slab s - 1, so its buffer is free next time
    if (s + 1 < n_slabs) {
      pq = *reinterpret_cast<const float4*>(gq + uint64_t(s + 1) * kGemmSlab * q_pad);
      pc = *reinterpret_cast<const float4*>(gc + uint64_t(s + 1) * kGemmSlab * l_pad);
    }
#pragma unroll
    for (uint32_t kk = 0; kk < kGemmSlab; kk += 2) {
      const uint32_t k = kk + (lane >> 5);
      float a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; i++) { a[i] = sa[buf][k][wq * 64u + i * 32u + (lane & 31u)]; }
#pragma unroll
      for (int j = 0; j < 2; j++) { b[j] = sb[buf][k][wl * 64u + j * 32u + (lane & 31u)]; }
#pragma unroll
      for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
      }
    }
  }

  // element r of a tile: row (r / 4) * 8 + (lane / 32) * 4 + r % 4 (query), column lane % 32 (list)
#pragma unroll
  for (int i = 0; i < 2; i++) {
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const uint32_t l = l0 + wl * 64u + j * 32u + (lane & 31u);
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const uint32_t q = q0 + wq * 64u + i * 32u + (r >> 2) * 8u + (lane >> 5) * 4u + (r & 3);
        if (q < n_queries && l < n_lists) {
          float v = alpha * acc[i][j][r];
          if (HALF) { v = round_half(v); }
          scores[uint64_t(q) * n_lists + l] = v;
        }
      }
    }
  }
}

inline uint32_t blocks_of(uint64_t n, uint32_t block) { return uint32_t((n + block - 1) / block); }

}  // namespace

uint32_t coarse_pad(uint32_t n) { return (n + kGemmTile - 1) / kGemmTile * kGemmTile; }

void launch_transpose_centers(const float* centers, uint32_t n_lists, uint32_t dim_ext, float* ct,
                              hipStream_t stream)
{
  if (n_lists == 0) { return; }
  const uint32_t l_pad = coarse_pad(n_lists);
  const uint64_t n     = uint64_t(dim_ext) * l_pad;
  transpose_centers_kernel<<<blocks_of(n, 256), 256, 0, stream>>>(centers, n_lists, dim_ext, l_pad, ct);
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_map_queries_t(const void* queries, elem_type type, uint32_t n_queries, uint32_t dim,
                          uint32_t dim_ext, bool ip_like, float* qt, hipStream_t stream)
{
  if (n_queries == 0) { return; }
  const uint32_t q_pad = coarse_pad(n_queries);
  const uint64_t n     = uint64_t(dim_ext) * q_pad;
  const float qnorm    = ip_like ? 0.0f : -0.5f;
  const uint32_t grid  = blocks_of(n, 256);
  switch (type) {
    case elem_type::f32:
      map_queries_t_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(queries), n_queries, dim, dim_ext, q_pad, qnorm, qt);
      break;
    case elem_type::f16:
      map_queries_t_kernel<_Float16><<<grid, 256, 0, stream>>>(static_cast<const _Float16*>(queries), n_queries, dim, dim_ext, q_pad, qnorm, qt);
      break;
    case elem_type::i8:
      map_queries_t_kernel<int8_t><<<grid, 256, 0, stream>>>(static_cast<const int8_t*>(queries), n_queries, dim, dim_ext, q_pad, qnorm, qt);
      break;
    case elem_type::u8:
      map_queries_t_kernel<uint8_t><<<grid, 256, 0, stream>>>(static_cast<const uint8_t*>(queries), n_queries, dim, dim_ext, q_pad, qnorm, qt);
      break;
  }
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_coarse_scores_mfma(const float* qt, const float* ct, uint32_t n_queries, uint32_t n_lists,
                               uint32_t dim_ext, bool ip_like, bool half_inputs, float* scores,
                               hipStream_t stream)
{
  if (n_queries == 0 || n_lists == 0) { return; }
  const uint32_t q_pad = coarse_pad(n_queries);
  const uint32_t l_pad = coarse_pad(n_lists);
  const float alpha    = ip_like ? -1.0f : -2.0f;
  dim3 grid(l_pad / kGemmTile, q_pad / kGemmTile);
  if (half_inputs) {
    coarse_scores_mfma_kernel<true><<<grid, 256, 0, stream>>>(qt, ct, n_queries, n_lists, dim_ext, q_pad, l_pad, alpha, scores);
  } else {
    coarse_scores_mfma_kernel<false><<<grid, 256, 0, stream>>>(qt, ct, n_queries, n_lists, dim_ext, q_pad, l_pad, alpha, scores);
  }
  CUVS_HIP_TRY(hipGetLastError());
}

}  // namespace cuvs::neighbors::ivf_pq::detail
