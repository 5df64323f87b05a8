/*
 * Kernels of index training: balanced k-means for the coarse centres and for the PQ codebooks.
 * Role of cuVS cluster::kmeans_balanced (cpp/src/cluster/detail/kmeans_balanced.cuh: predict,
 * calc_centers_and_sizes, adjust_centers, balancing_em_iters) as ivf_pq::build uses it
 * (cpp/src/neighbors/ivf_pq/ivf_pq_build.cuh:328-515, :1275-1400).
 *
 * The expectation step of the coarse clustering is the search path's own coarse stage (matrix-core
 * score kernel + selection of the single best centre); the kernels here are the other steps:
 * gathering the training rows, accumulating and finishing the means, moving the centres of
 * underfull clusters next to overfull ones, and a whole k-means of a codebook inside one
 * workgroup (a codebook has at most 256 entries of a few dimensions: it lives in LDS, and so do
 * the partial sums).
 */
#include "device_utils.cuh"

#include <algorithm>

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

__device__ __forceinline__ uint32_t mix32(uint32_t x)
{
  x ^= x >> 16;
  x *= 0x7feb352du;
  x ^= x >> 15;
  x *= 0x846ca68bu;
  x ^= x >> 16;
  return x;
}

/** Row i of the training set = row i * ratio + (a hash of i) % ratio of the dataset. */
__global__ void gather_rows_kernel(const uint8_t* __restrict__ src, uint64_t row_bytes, uint64_t n_out,
                                   uint64_t ratio, uint32_t seed, uint8_t* __restrict__ dst)
{
  const uint64_t i = blockIdx.x;
  if (i >= n_out) { return; }
  const uint64_t row = i * ratio + (ratio > 1 ? mix32(uint32_t(i) ^ seed) % ratio : 0);
  const uint8_t* s   = src + row * row_bytes;
  uint8_t* d         = dst + i * row_bytes;
  for (uint64_t b = threadIdx.x; b < row_bytes; b += blockDim.x) { d[b] = s[b]; }
}

/** ext[l] = (centre l, its squared norm, zero padding) from flat centres [n_lists, dim]. */
__global__ void set_centers_kernel(const float* __restrict__ flat, uint32_t n_lists, uint32_t dim,
                                   uint32_t dim_ext, float* __restrict__ ext)
{
  const uint32_t l    = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
  const uint32_t lane = threadIdx.x & 63u;
  if (l >= n_lists) { return; }
  float ss = 0.0f;
  for (uint32_t d = lane; d < dim; d += 64) {
    const float v                 = flat[uint64_t(l) * dim + d];
    ext[uint64_t(l) * dim_ext + d] = v;
    ss                             = fmaf(v, v, ss);
  }
  for (int o = 32; o > 0; o >>= 1) { ss += __shfl_xor(ss, o); }
  for (uint32_t d = dim + lane; d < dim_ext; d += 64) {
    ext[uint64_t(l) * dim_ext + d] = d == dim ? ss : 0.0f;
  }
}

/** sums[label[i]] += x[i], counts[label[i]] += 1, member[label[i]] = i (any member). One wave a row. */
__global__ void accumulate_kernel(const float* __restrict__ x, const uint32_t* __restrict__ labels,
                                  uint64_t n_rows, uint32_t dim, float* __restrict__ sums,
                                  uint32_t* __restrict__ counts, uint32_t* __restrict__ member)
{
  const uint64_t i    = uint64_t(blockIdx.x) * (blockDim.x / 64) + threadIdx.x / 64;
  const uint32_t lane = threadIdx.x & 63u;
  if (i >= n_rows) { return; }
  const uint32_t l = labels[i];
  for (uint32_t d = lane; d < dim; d += 64) {
    atomicAdd(&sums[uint64_t(l) * dim + d], x[i * dim + d]);
  }
  if (lane == 0) {
    atomicAdd(&counts[l], 1u);
    member[l] = uint32_t(i);
  }
}

/** centre = mean of its rows (unchanged when it has none); unit length when `normalize`. */
__global__ void finish_centers_kernel(const float* __restrict__ sums, const uint32_t* __restrict__ counts,
                                      uint32_t n_lists, uint32_t dim, bool normalize,
                                      float* __restrict__ flat)
{
  const uint32_t l    = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
  const uint32_t lane = threadIdx.x & 63u;
  if (l >= n_lists) { return; }
  const uint32_t c = counts[l];
  float ss         = 0.0f;
  for (uint32_t d = lane; d < dim; d += 64) {
    float v = flat[uint64_t(l) * dim + d];
    if (c > 0) { v = sums[uint64_t(l) * dim + d] / float(c); }
    flat[uint64_t(l) * dim + d] = v;
    ss                          = fmaf(v, v, ss);
  }
  if (normalize) {
    for (int o = 32; o > 0; o >>= 1) { ss += __shfl_xor(ss, o); }
    const float nrm = sqrtf(ss);
    if (nrm > 0.0f) {
      for (uint32_t d = lane; d < dim; d += 64) { flat[uint64_t(l) * dim + d] /= nrm; }
    }
  }
}

/** centre[receiver] = centre[donor] + offset * (x[member[donor]] - centre[donor]) for every pair
 *  (adjust_centers_kernel, kmeans_balanced.cuh:520-565). */
__global__ void adjust_centers_kernel(const uint32_t* __restrict__ receivers,
                                      const uint32_t* __restrict__ donors, uint32_t n_pairs,
                                      const float* __restrict__ x, const uint32_t* __restrict__ member,
                                      uint32_t dim, float offset, float* __restrict__ flat)
{
  const uint32_t p    = blockIdx.x * (blockDim.x / 64) + threadIdx.x / 64;
  const uint32_t lane = threadIdx.x & 63u;
  if (p >= n_pairs) { return; }
  const uint32_t r = receivers[p], dn = donors[p];
  const uint64_t i = member[dn];
  for (uint32_t d = lane; d < dim; d += 64) {
    const float c               = flat[uint64_t(dn) * dim + d];
    flat[uint64_t(r) * dim + d] = c + offset * (x[i * dim + d] - c);
  }
}

/** diff[i] = x[i] - centre[label[i]] (first `dim` columns of the extended centres). */
__global__ void residual_kernel(const float* __restrict__ x, const uint32_t* __restrict__ labels,
                                const float* __restrict__ centers_ext, uint64_t n_rows, uint32_t dim,
                                uint32_t dim_ext, float* __restrict__ diff)
{
  const uint64_t i    = uint64_t(blockIdx.x) * (blockDim.x / 64) + threadIdx.x / 64;
  const uint32_t lane = threadIdx.x & 63u;
  if (i >= n_rows) { return; }
  const uint32_t l = labels[i];
  for (uint32_t d = lane; d < dim; d += 64) {
    diff[i * dim + d] = x[i * dim + d] - centers_ext[uint64_t(l) * dim_ext + d];
  }
}

constexpr uint32_t kBookThreads = 512;
constexpr uint32_t kMaxPqLen    = 32;

/**
 * Balanced k-means of one codebook per workgroup (train_per_subset / train_per_cluster,
 * ivf_pq_build.cuh:328-515: 2^pq_bits clusters of pq_len-dimensional residual pieces, L2, underfull
 * clusters re-seeded next to a random point of a cluster of at least average size, lower tolerance
 * 0.25, centroid offset 0.05).
 *
 * Group g is a subspace (samples = piece g of the first n_rows residual rows) or a list (samples =
 * all pq_dim pieces of the list's rows, `rows[offsets[g] .. offsets[g + 1])`, at most max_samples).
 * The codebook, the sums and the counts stay in LDS for all iterations; the result is written in
 * the index's layout [group][pq_len][book].
 */
__global__ __launch_bounds__(kBookThreads) void train_codebook_kernel(
  const float* __restrict__ res, uint32_t rot_dim, uint32_t pq_dim, uint32_t pq_len, uint32_t book,
  bool per_cluster, uint32_t n_rows, const uint32_t* __restrict__ rows,
  const uint32_t* __restrict__ offsets, uint32_t max_samples, uint32_t n_iters, uint32_t seed,
  float* __restrict__ pq_centers)
{
  extern __shared__ __align__(16) float smem[];
  float* cb       = smem;                   // [book][pq_len]
  float* sums     = cb + book * pq_len;     // [book][pq_len]
  float* fresh    = sums + book * pq_len;   // [book][pq_len]: re-seeded entries
  uint32_t* count = reinterpret_cast<uint32_t*>(fresh + book * pq_len);  // [book]
  uint32_t* moved = count + book;                                        // [book] flags

  const uint32_t g   = blockIdx.x;
  const uint32_t tid = threadIdx.x;
  uint32_t n_g;
  uint32_t first = 0;
  if (per_cluster) {
    first = offsets[g];
    const uint64_t avail = uint64_t(offsets[g + 1] - first) * pq_dim;
    n_g = uint32_t(avail < max_samples ? avail : max_samples);
  } else {
    n_g = n_rows < max_samples ? n_rows : max_samples;
  }
  float* out = pq_centers + uint64_t(g) * pq_len * book;
  if (n_g == 0) {
    for (uint32_t e = tid; e < pq_len * book; e += kBookThreads) { out[e] = 0.0f; }
    return;
  }
  auto sample_ptr = [&](uint32_t s) -> const float* {
    if (per_cluster) {
      return res + uint64_t(rows[first + s / pq_dim]) * rot_dim + (s % pq_dim) * pq_len;
    }
    return res + uint64_t(s) * rot_dim + g * pq_len;
  };
  auto nearest = [&](const float* x) -> uint32_t {
    float best    = 3.4e38f;
    uint32_t arg  = 0;
    for (uint32_t c = 0; c < book; c++) {
      float d = 0.0f;
      for (uint32_t t = 0; t < pq_len; t++) {
        const float df = x[t] - cb[c * pq_len + t];
        d              = fmaf(df, df, d);
      }
      if (d < best) {
        best = d;
        arg  = c;
      }
    }
    return arg;
  };

  // initial entries: samples spread evenly over the group
  for (uint32_t e = tid; e < book * pq_len; e += kBookThreads) {
    const uint32_t c = e / pq_len, t = e % pq_len;
    const uint32_t s = uint32_t((uint64_t(c) * n_g) / book) % n_g;
    cb[e]            = sample_ptr(s)[t];
  }
  __syncthreads();

  const float average = float(n_g) / float(book);
  for (uint32_t iter = 0; iter < n_iters; iter++) {
    for (uint32_t e = tid; e < book * pq_len; e += kBookThreads) { sums[e] = 0.0f; }
    for (uint32_t c = tid; c < book; c += kBookThreads) {
      count[c] = 0;
      moved[c] = 0;
    }
    __syncthreads();
    // expectation + accumulation
    for (uint32_t s = tid; s < n_g; s += kBookThreads) {
      float x[kMaxPqLen];
      const float* p = sample_ptr(s);
      for (uint32_t t = 0; t < pq_len; t++) { x[t] = p[t]; }
      const uint32_t c = nearest(x);
      for (uint32_t t = 0; t < pq_len; t++) { atomicAdd(&sums[c * pq_len + t], x[t]); }
      atomicAdd(&count[c], 1u);
    }
    __syncthreads();
    // maximisation
    for (uint32_t e = tid; e < book * pq_len; e += kBookThreads) {
      const uint32_t n = count[e / pq_len];
      if (n > 0) { cb[e] = sums[e] / float(n); }
    }
    __syncthreads();
    // balancing, except after the last iteration: the final entries are plain means
    if (iter + 1 < n_iters) {
      for (uint32_t c = tid; c < book; c += kBookThreads) {
        if (float(count[c]) >= 0.25f * average) { continue; }
        for (uint32_t attempt = 0; attempt < 16; attempt++) {
          const uint32_t s = mix32(seed ^ (g * 0x9e3779b9u) ^ (iter * 0x85ebca6bu) ^ (c * 0xc2b2ae35u) ^ attempt) % n_g;
          float x[kMaxPqLen];
          const float* p = sample_ptr(s);
          for (uint32_t t = 0; t < pq_len; t++) { x[t] = p[t]; }
          const uint32_t donor = nearest(x);
          if (float(count[donor]) >= average) {
            for (uint32_t t = 0; t < pq_len; t++) {
              const float dc        = cb[donor * pq_len + t];
              fresh[c * pq_len + t] = dc + 0.05f * (x[t] - dc);
            }
            moved[c] = 1;
            break;
          }
        }
      }
      __syncthreads();
      for (uint32_t e = tid; e < book * pq_len; e += kBookThreads) {
        if (moved[e / pq_len]) { cb[e] = fresh[e]; }
      }
      __syncthreads();
    }
  }
  for (uint32_t e = tid; e < book * pq_len; e += kBookThreads) {
    const uint32_t c = e / pq_len, t = e % pq_len;
    out[t * book + c] = cb[e];
  }
}

}  // namespace

#define CUVS_LAUNCH_CHECK() CUVS_HIP_TRY(hipGetLastError())

void launch_gather_rows(const void* src, uint64_t row_bytes, uint64_t n_out, uint64_t ratio,
                        uint32_t seed, void* dst, hipStream_t stream)
{
  if (n_out == 0) { return; }
  CUVS_EXPECTS(n_out <= 0x7FFFFFFFull, "too many training rows");
  gather_rows_kernel<<<uint32_t(n_out), 128, 0, stream>>>(static_cast<const uint8_t*>(src), row_bytes,
                                                          n_out, ratio, seed, static_cast<uint8_t*>(dst));
  CUVS_LAUNCH_CHECK();
}

void launch_set_centers(const float* flat, uint32_t n_lists, uint32_t dim, uint32_t dim_ext, float* ext,
                        hipStream_t stream)
{
  set_centers_kernel<<<(n_lists + 3) / 4, 256, 0, stream>>>(flat, n_lists, dim, dim_ext, ext);
  CUVS_LAUNCH_CHECK();
}

void launch_accumulate(const float* x, const uint32_t* labels, uint64_t n_rows, uint32_t dim,
                       float* sums, uint32_t* counts, uint32_t* member, hipStream_t stream)
{
  if (n_rows == 0) { return; }
  const uint64_t blocks = (n_rows + 3) / 4;
  CUVS_EXPECTS(blocks <= 0x7FFFFFFFull, "too many training rows");
  accumulate_kernel<<<uint32_t(blocks), 256, 0, stream>>>(x, labels, n_rows, dim, sums, counts, member);
  CUVS_LAUNCH_CHECK();
}

void launch_finish_centers(const float* sums, const uint32_t* counts, uint32_t n_lists, uint32_t dim,
                           bool normalize, float* flat, hipStream_t stream)
{
  finish_centers_kernel<<<(n_lists + 3) / 4, 256, 0, stream>>>(sums, counts, n_lists, dim, normalize, flat);
  CUVS_LAUNCH_CHECK();
}

void launch_adjust_centers(const uint32_t* receivers, const uint32_t* donors, uint32_t n_pairs,
                           const float* x, const uint32_t* member, uint32_t dim, float offset,
                           float* flat, hipStream_t stream)
{
  if (n_pairs == 0) { return; }
  adjust_centers_kernel<<<(n_pairs + 3) / 4, 256, 0, stream>>>(receivers, donors, n_pairs, x, member,
                                                               dim, offset, flat);
  CUVS_LAUNCH_CHECK();
}

void launch_residuals(const float* x, const uint32_t* labels, const float* centers_ext, uint64_t n_rows,
                      uint32_t dim, uint32_t dim_ext, float* diff, hipStream_t stream)
{
  if (n_rows == 0) { return; }
  const uint64_t blocks = (n_rows + 3) / 4;
  CUVS_EXPECTS(blocks <= 0x7FFFFFFFull, "too many training rows");
  residual_kernel<<<uint32_t(blocks), 256, 0, stream>>>(x, labels, centers_ext, n_rows, dim, dim_ext, diff);
  CUVS_LAUNCH_CHECK();
}

uint32_t train_codebook_max_pq_len() { return kMaxPqLen; }

void launch_train_codebooks(const float* res, uint32_t rot_dim, uint32_t pq_dim, uint32_t pq_len,
                            uint32_t book, bool per_cluster, uint32_t n_groups, uint32_t n_rows,
                            const uint32_t* rows, const uint32_t* offsets, uint32_t max_samples,
                            uint32_t n_iters, uint32_t seed, float* pq_centers, hipStream_t stream)
{
  CUVS_EXPECTS(pq_len <= kMaxPqLen, "codebook training supports pq_len up to %u (got %u)", kMaxPqLen,
               pq_len);
  const size_t smem = size_t(book) * pq_len * 4 * 3 + size_t(book) * 8;
  auto kernel       = train_codebook_kernel;
  if (smem > 48 * 1024) {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
  }
  kernel<<<n_groups, kBookThreads, smem, stream>>>(res, rot_dim, pq_dim, pq_len, book, per_cluster,
                                                   n_rows, rows, offsets, max_samples, n_iters, seed,
                                                   pq_centers);
  CUVS_LAUNCH_CHECK();
}

}  // namespace cuvs::neighbors::ivf_pq::detail
