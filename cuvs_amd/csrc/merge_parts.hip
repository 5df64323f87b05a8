/*
 * Merging the per-shard results of a row-sharded search.
 * Role of cuvs::neighbors::knn_merge_parts (cpp/include/cuvs/neighbors/knn_merge_parts.hpp,
 * cpp/src/neighbors/detail/knn_merge_parts.cuh:23-110): `in_keys` / `in_ids` hold n_parts blocks of
 * [n_samples, k] (part-major); row r of the output is the k smallest keys among the n_parts * k
 * candidates of row r, ascending, each id shifted by its part's translation.
 *
 * One workgroup per row: the candidates become 64-bit sort keys (ordered score bits, then position
 * part * k + column, which makes ties deterministic), are bitonic-sorted in LDS and the first k
 * are written out.
 */
#include "device_utils.cuh"

#include <algorithm>

namespace cuvs::neighbors::detail {

using cuvs::neighbors::ivf_pq::detail::order_f32;

namespace {

constexpr uint32_t kMergeThreads  = 256;
constexpr uint32_t kMergeMaxTotal = 8192;  // n_parts * k candidates of a row (64 KB of LDS)

template <typename IdT>
__global__ __launch_bounds__(kMergeThreads) void merge_parts_kernel(
  const float* __restrict__ in_keys, const IdT* __restrict__ in_ids, float* __restrict__ out_keys,
  IdT* __restrict__ out_ids, uint64_t n_samples, uint32_t n_parts, uint32_t k,
  const IdT* __restrict__ translations, uint32_t cap)
{
  extern __shared__ __align__(16) unsigned long long cand[];
  const uint64_t row   = blockIdx.x;
  const uint32_t total = n_parts * k;
  for (uint32_t i = threadIdx.x; i < cap; i += kMergeThreads) {
    unsigned long long key = ~0ull;
    if (i < total) {
      const uint32_t part = i / k, col = i - part * k;
      const float v       = in_keys[(uint64_t(part) * n_samples + row) * k + col];
      // NaN sorts last
      const uint32_t o = (v != v) ? 0xFFFFFFFFu : order_f32(v);
      key              = (static_cast<unsigned long long>(o) << 32) | i;
    }
    cand[i] = key;
  }
  __syncthreads();
  for (uint32_t size = 2; size <= cap; size <<= 1) {
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      for (uint32_t c = threadIdx.x; c < (cap >> 1); c += kMergeThreads) {
        const uint32_t i = (c / stride) * (2u * stride) + (c & (stride - 1u));
        const uint32_t j = i + stride;
        const bool up    = (i & size) == 0;
        const unsigned long long x = cand[i], y = cand[j];
        if ((x > y) == up) {
          cand[i] = y;
          cand[j] = x;
        }
      }
      __syncthreads();
    }
  }
  for (uint32_t t = threadIdx.x; t < k; t += kMergeThreads) {
    const uint32_t i    = uint32_t(cand[t]);  // low word: position among the candidates
    const uint32_t part = i / k, col = i - part * k;
    const uint64_t at   = (uint64_t(part) * n_samples + row) * k + col;
    out_keys[row * k + t] = in_keys[at];
    out_ids[row * k + t]  = IdT(in_ids[at] + translations[part]);
  }
}

}  // namespace

template <typename IdT>
void launch_merge_parts(const float* in_keys, const IdT* in_ids, float* out_keys, IdT* out_ids,
                        uint64_t n_samples, uint32_t n_parts, uint32_t k, const IdT* translations,
                        hipStream_t stream)
{
  if (n_samples == 0 || k == 0) { return; }
  const uint64_t total = uint64_t(n_parts) * k;
  CUVS_EXPECTS(n_parts > 0, "n_parts must be positive");
  CUVS_EXPECTS(total <= kMergeMaxTotal, "n_parts * k = %llu exceeds the supported %u candidates per row",
               static_cast<unsigned long long>(total), kMergeMaxTotal);
  CUVS_EXPECTS(n_samples <= 0x7FFFFFFFull, "too many rows");
  uint32_t cap = 2;
  while (cap < total) { cap <<= 1; }
  const size_t smem = size_t(cap) * 8;
  auto kernel       = merge_parts_kernel<IdT>;
  if (smem > 48 * 1024) {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
  }
  kernel<<<uint32_t(n_samples), kMergeThreads, smem, stream>>>(in_keys, in_ids, out_keys, out_ids, n_samples,
                                                               n_parts, k, translations, cap);
  CUVS_HIP_TRY(hipGetLastError());
}

template void launch_merge_parts<int64_t>(const float*, const int64_t*, float*, int64_t*, uint64_t, uint32_t,
                                          uint32_t, const int64_t*, hipStream_t);
template void launch_merge_parts<int32_t>(const float*, const int32_t*, float*, int32_t*, uint64_t, uint32_t,
                                          uint32_t, const int32_t*, hipStream_t);
template void launch_merge_parts<uint32_t>(const float*, const uint32_t*, float*, uint32_t*, uint64_t, uint32_t,
                                           uint32_t, const uint32_t*, hipStream_t);

}  // namespace cuvs::neighbors::detail
