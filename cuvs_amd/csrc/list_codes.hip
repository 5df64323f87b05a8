/*
 * Reading and writing the codes of one list outside the search: one code per byte or
 * bit-contiguous rows <-> the interleaved list layout, and decoding rows back to vectors.
 * Role of cuVS' unpack_list_data / pack_list_data kernels (ivf_pq_list_data_impl.cuh:43-170) and
 * reconstruct_list_data_kernel (ivf_pq_build.cuh:520-592).  None of this is on the search path:
 * one thread per row, plain loops.
 *
 * Layout of a list (cpp/include/cuvs/neighbors/ivf_pq.hpp:222-296): rows in groups of 32; a row's
 * codes are cut into chunks of floor(128 / pq_bits) codes, each chunk a 16-byte little-endian
 * bit string with code jj at bit jj * pq_bits; chunk c of row i sits at byte
 * ((i / 32) * n_chunks + c) * 512 + (i % 32) * 16.
 */
#include "device_utils.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

constexpr uint32_t kRowBlock = 256;

__device__ __forceinline__ uint64_t row_base(uint32_t i, uint32_t n_chunks)
{
  return uint64_t(i >> 5) * n_chunks * 512u + uint64_t(i & 31u) * 16u;
}

/** Code j of the row whose first chunk starts at `row0`. */
__device__ __forceinline__ uint32_t stored_code(const uint8_t* row0, uint32_t j, uint32_t cpc,
                                                uint32_t pq_bits)
{
  const uint8_t* chunk = row0 + uint64_t(j / cpc) * 512u;
  const uint32_t bit   = (j % cpc) * pq_bits;
  uint32_t v           = chunk[bit >> 3];
  if ((bit & 7u) + pq_bits > 8u) { v |= uint32_t(chunk[(bit >> 3) + 1]) << 8; }
  return (v >> (bit & 7u)) & ((1u << pq_bits) - 1u);
}

/** Row r of the request: `offset + r`, or `rows[r]` when a selection is given. */
__device__ __forceinline__ uint32_t list_row(uint32_t r, uint32_t offset, const uint32_t* rows)
{
  return rows != nullptr ? rows[r] : offset + r;
}

__global__ __launch_bounds__(kRowBlock) void unpack_codes_kernel(const uint8_t* __restrict__ list_data,
                                                                 uint32_t n_rows, uint32_t offset,
                                                                 const uint32_t* __restrict__ rows,
                                                                 uint32_t pq_dim, uint32_t pq_bits,
                                                                 uint8_t* __restrict__ out)
{
  const uint32_t r = blockIdx.x * kRowBlock + threadIdx.x;
  if (r >= n_rows) { return; }
  const uint32_t cpc      = 128u / pq_bits;
  const uint32_t n_chunks = (pq_dim + cpc - 1u) / cpc;
  const uint8_t* row0     = list_data + row_base(list_row(r, offset, rows), n_chunks);
  for (uint32_t j = 0; j < pq_dim; j++) { out[uint64_t(r) * pq_dim + j] = uint8_t(stored_code(row0, j, cpc, pq_bits)); }
}

/** CONTIGUOUS: the input rows are bit strings of pq_dim * pq_bits bits; else one code per byte. */
template <bool CONTIGUOUS>
__global__ __launch_bounds__(kRowBlock) void pack_codes_kernel(uint8_t* __restrict__ list_data,
                                                               const uint8_t* __restrict__ codes,
                                                               uint32_t n_rows, uint32_t offset,
                                                               uint32_t pq_dim, uint32_t pq_bits)
{
  const uint32_t r = blockIdx.x * kRowBlock + threadIdx.x;
  if (r >= n_rows) { return; }
  const uint32_t cpc       = 128u / pq_bits;
  const uint32_t n_chunks  = (pq_dim + cpc - 1u) / cpc;
  const uint32_t mask      = (1u << pq_bits) - 1u;
  const uint32_t row_bytes = (pq_dim * pq_bits + 7u) / 8u;
  const uint8_t* in        = codes + uint64_t(r) * (CONTIGUOUS ? row_bytes : pq_dim);
  uint8_t* row0            = list_data + row_base(offset + r, n_chunks);
  for (uint32_t c = 0; c < n_chunks; c++) {
    uint32_t w[4] = {0u, 0u, 0u, 0u};  // the chunk as four little-endian words
    for (uint32_t jj = 0; jj < cpc; jj++) {
      const uint32_t j = c * cpc + jj;
      if (j >= pq_dim) { break; }
      uint32_t code;
      if (CONTIGUOUS) {
        const uint32_t ib = j * pq_bits;
        uint32_t v        = in[ib >> 3];
        if ((ib & 7u) + pq_bits > 8u) { v |= uint32_t(in[(ib >> 3) + 1]) << 8; }
        code = (v >> (ib & 7u)) & mask;
      } else {
        code = in[j] & mask;
      }
      const uint32_t bit = jj * pq_bits;
      w[bit >> 5] |= code << (bit & 31u);
      if ((bit & 31u) + pq_bits > 32u) { w[(bit >> 5) + 1] |= code >> (32u - (bit & 31u)); }
    }
    *reinterpret_cast<uint4*>(row0 + uint64_t(c) * 512u) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

/** out[r] = centre_rot[label] + the codebook entries of row r's codes, in the rotated space. */
__global__ __launch_bounds__(kRowBlock) void reconstruct_rot_kernel(
  const uint8_t* __restrict__ list_data, uint32_t n_rows, uint32_t offset,
  const uint32_t* __restrict__ rows, uint32_t pq_dim, uint32_t pq_bits, uint32_t pq_len,
  const float* __restrict__ book_base, int per_subspace, const float* __restrict__ center_rot,
  float* __restrict__ out)
{
  const uint32_t r = blockIdx.x * kRowBlock + threadIdx.x;
  if (r >= n_rows) { return; }
  const uint32_t cpc      = 128u / pq_bits;
  const uint32_t n_chunks = (pq_dim + cpc - 1u) / cpc;
  const uint32_t book     = 1u << pq_bits;
  const uint32_t rot_dim  = pq_dim * pq_len;
  const uint8_t* row0     = list_data + row_base(list_row(r, offset, rows), n_chunks);
  for (uint32_t j = 0; j < pq_dim; j++) {
    const uint32_t code = stored_code(row0, j, cpc, pq_bits);
    const float* cb     = book_base + (per_subspace ? uint64_t(j) * pq_len * book : 0);
    for (uint32_t t = 0; t < pq_len; t++) {
      out[uint64_t(r) * rot_dim + j * pq_len + t] = cb[uint64_t(t) * book + code] + center_rot[j * pq_len + t];
    }
  }
}

/** The inverse of the mapping applied to rows on the way in (cuVS utils::mapping<T>,
 *  detail/ann_utils.cuh:158-217): integer rows are scaled back by 128 / 256 and clamped. */
template <typename T>
__device__ __forceinline__ T unmap_value(float v);
template <>
__device__ __forceinline__ float unmap_value<float>(float v)
{
  return v;
}
template <>
__device__ __forceinline__ _Float16 unmap_value<_Float16>(float v)
{
  return static_cast<_Float16>(v);
}
template <>
__device__ __forceinline__ int8_t unmap_value<int8_t>(float v)
{
  return static_cast<int8_t>(fminf(fmaxf(v * 128.0f, -128.0f), 127.0f));
}
template <>
__device__ __forceinline__ uint8_t unmap_value<uint8_t>(float v)
{
  return static_cast<uint8_t>(fminf(fmaxf(v * 256.0f, 0.0f), 255.0f));
}

template <typename T>
__global__ void unmap_rows_kernel(const float* __restrict__ in, uint64_t n, T* __restrict__ out)
{
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) { out[i] = unmap_value<T>(in[i]); }
}

inline uint32_t blocks_for(uint64_t n, uint32_t block) { return uint32_t((n + block - 1) / block); }

/** One thread per (row slot, 16-code chunk): the codes of the packed row as bytes, in the layout of
 *  an 8-bit index (chunk c of row i at (i / 32) * n_chunks8 * 512 + c * 512 + (i % 32) * 16). */
__global__ __launch_bounds__(kRowBlock) void widen_codes_kernel(const uint8_t* __restrict__ packed,
                                                                uint8_t* __restrict__ wide, uint64_t n_slots,
                                                                uint32_t pq_dim, uint32_t pq_bits,
                                                                uint32_t n_chunks, uint32_t n_chunks8)
{
  const uint64_t t = uint64_t(blockIdx.x) * kRowBlock + threadIdx.x;
  if (t >= n_slots * n_chunks8) { return; }
  const uint64_t i    = t / n_chunks8;
  const uint32_t c8   = uint32_t(t - i * n_chunks8);
  const uint32_t cpc  = 128u / pq_bits;
  const uint8_t* row0 = packed + (i >> 5) * n_chunks * 512u + (i & 31u) * 16u;
  uint32_t w[4]       = {0, 0, 0, 0};
#pragma unroll
  for (uint32_t x = 0; x < 16; x++) {
    const uint32_t j = c8 * 16u + x;
    if (j < pq_dim) { w[x >> 2] |= stored_code(row0, j, cpc, pq_bits) << ((x & 3u) * 8u); }
  }
  *reinterpret_cast<uint4*>(wide + (i >> 5) * n_chunks8 * 512u + uint64_t(c8) * 512u + (i & 31u) * 16u) =
    make_uint4(w[0], w[1], w[2], w[3]);
}

/** One block per list: the largest squared length of a row's decoded residual. */
__global__ __launch_bounds__(kRowBlock) void list_radius_kernel(
  const uint8_t* const* __restrict__ data_ptrs, const uint32_t* __restrict__ list_sizes, uint32_t first_list,
  uint32_t pq_dim, uint32_t pq_bits, uint32_t pq_len, const float* __restrict__ pq_centers, int per_subspace,
  float* __restrict__ radius)
{
  __shared__ float wave_max[kRowBlock / 64];
  const uint32_t l        = first_list + blockIdx.x;
  const uint32_t n_rows   = list_sizes[l];
  const uint8_t* data     = data_ptrs[l];
  const uint32_t cpc      = 128u / pq_bits;
  const uint32_t n_chunks = (pq_dim + cpc - 1u) / cpc;
  const uint32_t book     = 1u << pq_bits;
  const float* book_base  = pq_centers + (per_subspace ? 0 : uint64_t(l) * pq_len * book);
  float best              = 0.0f;
  for (uint32_t i = threadIdx.x; i < n_rows; i += kRowBlock) {
    const uint8_t* row0 = data + row_base(i, n_chunks);
    float s             = 0.0f;
    for (uint32_t j = 0; j < pq_dim; j++) {
      const uint32_t code = stored_code(row0, j, cpc, pq_bits);
      const float* cb     = book_base + (per_subspace ? uint64_t(j) * pq_len * book : 0);
      for (uint32_t t = 0; t < pq_len; t++) {
        const float v = cb[uint64_t(t) * book + code];
        s             = fmaf(v, v, s);
      }
    }
    best = fmaxf(best, s);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) { best = fmaxf(best, __shfl_xor(best, off, 64)); }
  if ((threadIdx.x & 63u) == 0) { wave_max[threadIdx.x >> 6] = best; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (uint32_t w = 1; w < kRowBlock / 64; w++) { best = fmaxf(best, wave_max[w]); }
    // rounded up past what the fp32 sum of squares and the root can have lost
    radius[l] = sqrtf(best) * (1.0f + 1e-5f);
  }
}

/** dst[row][e] = e < book_size ? src[row][e] : 0 for 256 entries a row. */
__global__ void pad_codebooks_kernel(const float* __restrict__ src, float* __restrict__ dst, uint64_t n_rows,
                                     uint32_t book_size)
{
  const uint64_t t = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= n_rows * 256u) { return; }
  const uint64_t row = t >> 8;
  const uint32_t e   = uint32_t(t & 255u);
  dst[t]             = e < book_size ? src[row * book_size + e] : 0.0f;
}

}  // namespace

void launch_widen_codes(const uint8_t* packed, uint8_t* wide, uint64_t n_slots, uint32_t pq_dim,
                        uint32_t pq_bits, uint32_t n_chunks, uint32_t n_chunks8, hipStream_t stream)
{
  if (n_slots == 0) { return; }
  const uint64_t blocks = (n_slots * n_chunks8 + kRowBlock - 1) / kRowBlock;
  CUVS_EXPECTS(blocks <= 0x7FFFFFFFull, "too many row slots for one launch");
  widen_codes_kernel<<<uint32_t(blocks), kRowBlock, 0, stream>>>(packed, wide, n_slots, pq_dim, pq_bits, n_chunks,
                                                                n_chunks8);
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_list_radius(const uint8_t* const* data_ptrs, const uint32_t* list_sizes, uint32_t first_list,
                        uint32_t n, uint32_t pq_dim, uint32_t pq_bits, uint32_t pq_len, const float* pq_centers,
                        bool per_subspace, float* radius, hipStream_t stream)
{
  if (n == 0) { return; }
  list_radius_kernel<<<n, kRowBlock, 0, stream>>>(data_ptrs, list_sizes, first_list, pq_dim, pq_bits, pq_len,
                                                  pq_centers, per_subspace ? 1 : 0, radius);
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_pad_codebooks(const float* src, float* dst, uint64_t n_rows, uint32_t book_size, hipStream_t stream)
{
  if (n_rows == 0) { return; }
  const uint64_t blocks = (n_rows * 256u + 255u) / 256u;
  CUVS_EXPECTS(blocks <= 0x7FFFFFFFull, "too many codebook rows for one launch");
  pad_codebooks_kernel<<<uint32_t(blocks), 256, 0, stream>>>(src, dst, n_rows, book_size);
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_unpack_codes(const uint8_t* list_data, uint32_t n_rows, uint32_t offset,
                         const uint32_t* rows, uint32_t pq_dim, uint32_t pq_bits, uint8_t* out,
                         hipStream_t stream)
{
  if (n_rows == 0) { return; }
  unpack_codes_kernel<<<blocks_for(n_rows, kRowBlock), kRowBlock, 0, stream>>>(list_data, n_rows, offset, rows,
                                                                            pq_dim, pq_bits, out);
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_pack_codes(uint8_t* list_data, const uint8_t* codes, bool contiguous, uint32_t n_rows,
                       uint32_t offset, uint32_t pq_dim, uint32_t pq_bits, hipStream_t stream)
{
  if (n_rows == 0) { return; }
  const uint32_t grid = blocks_for(n_rows, kRowBlock);
  if (contiguous) {
    pack_codes_kernel<true><<<grid, kRowBlock, 0, stream>>>(list_data, codes, n_rows, offset, pq_dim, pq_bits);
  } else {
    pack_codes_kernel<false><<<grid, kRowBlock, 0, stream>>>(list_data, codes, n_rows, offset, pq_dim, pq_bits);
  }
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_reconstruct_rot(const uint8_t* list_data, uint32_t n_rows, uint32_t offset,
                            const uint32_t* rows, uint32_t pq_dim, uint32_t pq_bits, uint32_t pq_len,
                            const float* book_base, bool per_subspace, const float* center_rot,
                            float* out, hipStream_t stream)
{
  if (n_rows == 0) { return; }
  reconstruct_rot_kernel<<<blocks_for(n_rows, kRowBlock), kRowBlock, 0, stream>>>(
    list_data, n_rows, offset, rows, pq_dim, pq_bits, pq_len, book_base, per_subspace ? 1 : 0, center_rot, out);
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_unmap_rows(const float* in, uint64_t n_elems, elem_type type, void* out, hipStream_t stream)
{
  if (n_elems == 0) { return; }
  const uint32_t grid = blocks_for(n_elems, 256);
  switch (type) {
    case elem_type::f32:
      unmap_rows_kernel<float><<<grid, 256, 0, stream>>>(in, n_elems, static_cast<float*>(out));
      break;
    case elem_type::f16:
      unmap_rows_kernel<_Float16><<<grid, 256, 0, stream>>>(in, n_elems, static_cast<_Float16*>(out));
      break;
    case elem_type::i8:
      unmap_rows_kernel<int8_t><<<grid, 256, 0, stream>>>(in, n_elems, static_cast<int8_t*>(out));
      break;
    case elem_type::u8:
      unmap_rows_kernel<uint8_t><<<grid, 256, 0, stream>>>(in, n_elems, static_cast<uint8_t*>(out));
      break;
  }
  CUVS_HIP_TRY(hipGetLastError());
}

}  // namespace cuvs::neighbors::ivf_pq::detail
