/*
 * Refinement: exact distances between each query and its candidate rows, the k nearest kept
 * (cuVS refine_device, cpp/src/neighbors/refine/refine_device.cuh:35-135, which reuses the IVF-Flat
 * scan on a one-list-per-query index; here a direct kernel).
 *
 * One 256-thread block per query.  The query is staged in LDS as fp32 (integers exactly); wave w
 * takes candidates w, w + 4, ...: its lanes stride over the row with 16-byte loads where the row
 * allows, accumulate (q - x)^2 or q * x in fp32 (exact 32-bit integers for int8 / uint8 rows, as
 * the reference's accumulator type for those), and a wave reduction gives the distance.  Keys
 * (ordered distance, candidate slot) go to LDS; the block's selection keeps the k smallest and the
 * ids and distances are written in that order.
 */
#include "device_utils.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {


template <typename T>
struct refine_acc {
  using type = float;
};
template <>
struct refine_acc<int8_t> {
  using type = int32_t;
};
template <>
struct refine_acc<uint8_t> {
  using type = uint32_t;
};

template <typename T, bool IP>
__global__ __launch_bounds__(kBlock) void refine_kernel(const T* __restrict__ dataset,
                                                         const T* __restrict__ queries,
                                                         const int64_t* __restrict__ candidates,
                                                         int64_t n_rows, uint32_t dim,
                                                         uint32_t n_candidates, uint32_t k,
                                                         uint32_t out_cap, int sqrt_out,
                                                         int64_t* __restrict__ indices,
                                                         float* __restrict__ distances,
                                                         unsigned long long* __restrict__ scratch)
{
  using acc_t = typename refine_acc<T>::type;
  extern __shared__ __align__(16) unsigned char dyn_smem[];
  __shared__ select_smem sm;
  // keys [n_candidates] and the selection's output [out_cap]: in LDS, or (more candidates than LDS
  // holds) in the block's part of a global scratch buffer
  auto* keys = scratch != nullptr ? scratch + uint64_t(blockIdx.x) * (uint64_t(n_candidates) + out_cap)
                                  : reinterpret_cast<unsigned long long*>(dyn_smem);
  auto* out  = keys + n_candidates;
  auto* sq   = scratch != nullptr ? reinterpret_cast<acc_t*>(dyn_smem) : reinterpret_cast<acc_t*>(out + out_cap);  // [dim]
  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = tid >> 6;
  const uint32_t q    = blockIdx.x;
  for (uint32_t d = tid; d < dim; d += kBlock) { sq[d] = acc_t(queries[uint64_t(q) * dim + d]); }
  __syncthreads();

  for (uint32_t c = wid; c < n_candidates; c += kBlock / 64) {
    const int64_t id = candidates[uint64_t(q) * n_candidates + c];
    unsigned long long key = kInvalidKey;
    if (id >= 0 && id < n_rows) {  // uniform over the wave
      const T* row = dataset + uint64_t(id) * dim;
      acc_t acc    = acc_t(0);
      for (uint32_t d = lane; d < dim; d += 64u) {
        const acc_t x = acc_t(row[d]);
        if (IP) {
          acc += sq[d] * x;
        } else {
          const acc_t diff = sq[d] - x;  // unsigned wrap-around squares to the same value mod 2^32
          acc += diff * diff;
        }
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) { acc += __shfl_xor(acc, off, 64); }
      const float dist = float(acc);
      // smaller key = better: similarity is negated for the ordering
      const float ordered = IP ? -dist : dist;
      if (ordered == ordered) { key = (static_cast<unsigned long long>(order_f32(ordered)) << 32) | c; }
    }
    if (lane == 0) { keys[c] = key; }
  }
  __syncthreads();
  block_select_sorted([keys](uint32_t i) { return keys[i]; }, n_candidates, k, out, out_cap, sm);
  for (uint32_t r = tid; r < k; r += kBlock) {
    const unsigned long long key = out[r];
    int64_t id                   = -1;
    float d                      = FLT_MAX;
    if (key != kInvalidKey) {
      id = candidates[uint64_t(q) * n_candidates + uint32_t(key)];
      d  = unorder_f32(uint32_t(key >> 32));
      if (IP) { d = -d; }
      if (sqrt_out) { d = sqrtf(d); }
    }
    indices[uint64_t(q) * k + r]   = id;
    distances[uint64_t(q) * k + r] = d;
  }
}

template <typename T>
void launch_refine_typed(const void* dataset, const void* queries, const int64_t* candidates,
                         int64_t n_rows, uint32_t n_queries, uint32_t dim, uint32_t n_candidates,
                         uint32_t k, bool ip, bool sqrt_out, int64_t* indices, float* distances,
                         hipStream_t stream)
{
  const uint32_t out_cap = next_pow2(k);
  size_t smem            = size_t(n_candidates) * 8 + size_t(out_cap) * 8 + size_t(dim) * 4;
  // more than LDS holds: the keys live in a scratch buffer for the duration of the call
  device_buffer scratch;
  if (smem > 150 * 1024) {
    scratch.allocate(size_t(n_queries) * (size_t(n_candidates) + out_cap) * 8);
    smem = size_t(dim) * 4;
    CUVS_EXPECTS(smem <= 150 * 1024, "refine: dim (%u) is too large", dim);
  }
  auto* d_scratch = scratch.as<unsigned long long>();
  auto launch = [&](auto kernel) {
    if (smem > 32 * 1024) {
      CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
    }
    kernel<<<n_queries, kBlock, smem, stream>>>(static_cast<const T*>(dataset),
                                                static_cast<const T*>(queries), candidates, n_rows,
                                                dim, n_candidates, k, out_cap, sqrt_out ? 1 : 0,
                                                indices, distances, d_scratch);
    CUVS_HIP_TRY(hipGetLastError());
    // the buffer goes back when this function returns: the kernel must be through with it
    if (d_scratch != nullptr) { CUVS_HIP_TRY(hipStreamSynchronize(stream)); }
  };
  if (ip) {
    launch(refine_kernel<T, true>);
  } else {
    launch(refine_kernel<T, false>);
  }
}

}  // namespace

namespace {
__global__ void widen_ids_kernel(const uint32_t* __restrict__ in, int64_t* __restrict__ out, uint64_t n)
{
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) { out[i] = int64_t(in[i]); }
}
__global__ void narrow_ids_kernel(const int64_t* __restrict__ in, uint32_t* __restrict__ out, uint64_t n)
{
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) { out[i] = uint32_t(in[i]); }  // the id of an unfilled slot, -1, becomes 0xFFFFFFFF
}
}  // namespace

void launch_widen_ids(const uint32_t* in, int64_t* out, uint64_t n, hipStream_t stream)
{
  if (n == 0) { return; }
  widen_ids_kernel<<<uint32_t((n + 255) / 256), 256, 0, stream>>>(in, out, n);
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_narrow_ids(const int64_t* in, uint32_t* out, uint64_t n, hipStream_t stream)
{
  if (n == 0) { return; }
  narrow_ids_kernel<<<uint32_t((n + 255) / 256), 256, 0, stream>>>(in, out, n);
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_refine(const void* dataset, const void* queries, elem_type type,
                   const int64_t* candidates, int64_t n_rows, uint32_t n_queries, uint32_t dim,
                   uint32_t n_candidates, uint32_t k, bool ip, bool sqrt_out, int64_t* indices,
                   float* distances, hipStream_t stream)
{
  if (n_queries == 0) { return; }
  switch (type) {
    case elem_type::f32:
      launch_refine_typed<float>(dataset, queries, candidates, n_rows, n_queries, dim, n_candidates, k, ip, sqrt_out, indices, distances, stream);
      break;
    case elem_type::f16:
      launch_refine_typed<_Float16>(dataset, queries, candidates, n_rows, n_queries, dim, n_candidates, k, ip, sqrt_out, indices, distances, stream);
      break;
    case elem_type::i8:
      launch_refine_typed<int8_t>(dataset, queries, candidates, n_rows, n_queries, dim, n_candidates, k, ip, sqrt_out, indices, distances, stream);
      break;
    case elem_type::u8:
      launch_refine_typed<uint8_t>(dataset, queries, candidates, n_rows, n_queries, dim, n_candidates, k, ip, sqrt_out, indices, distances, stream);
      break;
  }
}

}  // namespace cuvs::neighbors::ivf_pq::detail
