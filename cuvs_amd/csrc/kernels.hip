/*
 * HIP kernels of the IVF-PQ search path for gfx950 (wave64, 160 KB LDS per CU).
 *
 * Stage order of one search batch (host driver: search.cpp):
 *   map_queries -> coarse_scores -> select_probes -> rotate -> chunk_indices -> order_pairs
 *   -> scan (LUT in LDS + code scan + per-pair top-k) -> merge (+ distance / id post-processing)
 * List maintenance: histogram, relocate_lists, encode, unpack_contiguous.
 *
 * Arithmetic that decides results is written with explicit fmaf / explicit rounding so that it is
 * reproducible against a scalar CPU implementation: dot products accumulate with one FMA per
 * element in ascending index order; lookup-table entries are built in fp32 and rounded once.
 */
#include "device_utils.cuh"
#include "scan_wave_select.cuh"

#include <algorithm>

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

/* ---------------------------------------------------------------------------------------- */
/* element mapping, coarse scores, probe selection                                           */
/* ---------------------------------------------------------------------------------------- */

__global__ void fill_u32_kernel(uint32_t* dst, uint32_t value, uint64_t n)
{
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) { dst[i] = value; }
}

template <typename T>
__device__ __forceinline__ float map_elem(T v);
template <>
__device__ __forceinline__ float map_elem<float>(float v)
{
  return v;
}
template <>
__device__ __forceinline__ float map_elem<_Float16>(_Float16 v)
{
  return float(v);
}
template <>
__device__ __forceinline__ float map_elem<int8_t>(int8_t v)
{
  return float(v) * (1.0f / 128.0f);
}
template <>
__device__ __forceinline__ float map_elem<uint8_t>(uint8_t v)
{
  return float(v) * (1.0f / 256.0f);
}

template <typename T>
__global__ void map_queries_kernel(const T* in, uint64_t n, float* out)
{
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) { out[i] = map_elem<T>(in[i]); }
}

__device__ __forceinline__ float round_to_half(float v) { return float(_Float16(v)); }

/**
 * 64 queries x 64 lists per block, 4 x 4 outputs per thread, K staged through LDS in slabs of 16.
 * Every output is one FMA chain over d = 0..dim-1 followed by the norm term, so the value does
 * not depend on the tiling.
 */
constexpr int kCoarseTile = 64;
constexpr int kCoarseK    = 16;

template <bool HALF>
__global__ __launch_bounds__(kBlock) void coarse_scores_kernel(const float* __restrict__ qf,
                                                                const float* __restrict__ centers,
                                                                uint32_t n_queries,
                                                                uint32_t n_lists, uint32_t dim,
                                                                uint32_t dim_ext, float qnorm,
                                                                float alpha,
                                                                float* __restrict__ scores)
{
  __shared__ float sq[kCoarseK][kCoarseTile + 4];
  __shared__ float sc[kCoarseK][kCoarseTile + 4];
  const uint32_t tid = threadIdx.x;
  const uint32_t tx  = tid & 15u;  // list direction
  const uint32_t ty  = tid >> 4;   // query direction
  const uint32_t q0  = blockIdx.y * kCoarseTile;
  const uint32_t l0  = blockIdx.x * kCoarseTile;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
#pragma unroll
    for (int j = 0; j < 4; j++) { acc[i][j] = 0.0f; }
  }
  const uint32_t lr = tid >> 4;   // 0..15: row within a load pass
  const uint32_t lc = tid & 15u;  // 0..15: column (k) within the slab
  for (uint32_t d0 = 0; d0 < dim; d0 += kCoarseK) {
#pragma unroll
    for (int pass = 0; pass < 4; pass++) {
      const uint32_t r = lr + 16u * pass;
      const uint32_t d = d0 + lc;
      float vq = 0.0f, vc = 0.0f;
      if (d < dim) {
        if (q0 + r < n_queries) { vq = qf[uint64_t(q0 + r) * dim + d]; }
        if (l0 + r < n_lists) { vc = centers[uint64_t(l0 + r) * dim_ext + d]; }
      }
      if (HALF) {
        vq = round_to_half(vq);
        vc = round_to_half(vc);
      }
      sq[lc][r] = vq;
      sc[lc][r] = vc;
    }
    __syncthreads();
    const uint32_t kmax = (dim - d0) < uint32_t(kCoarseK) ? (dim - d0) : uint32_t(kCoarseK);
    for (uint32_t kk = 0; kk < kmax; kk++) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; i++) { a[i] = sq[kk][ty * 4 + i]; }
#pragma unroll
      for (int j = 0; j < 4; j++) { b[j] = sc[kk][tx * 4 + j]; }
#pragma unroll
      for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++) { acc[i][j] = fmaf(b[j], a[i], acc[i][j]); }
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const uint32_t l = l0 + tx * 4 + j;
    if (l >= n_lists) { continue; }
    float nrm = centers[uint64_t(l) * dim_ext + dim];
    if (HALF) { nrm = round_to_half(nrm); }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t q = q0 + ty * 4 + i;
      if (q >= n_queries) { continue; }
      float v = alpha * fmaf(nrm, qnorm, acc[i][j]);
      if (HALF) { v = round_to_half(v); }
      scores[uint64_t(q) * n_lists + l] = v;
    }
  }
}

__global__ __launch_bounds__(kBlock) void select_probes_kernel(const float* __restrict__ scores,
                                                                uint32_t n_lists,
                                                                uint32_t n_probes,
                                                                uint32_t out_cap,
                                                                uint32_t* __restrict__ probes,
                                                                const uint8_t* __restrict__ only,
                                                                unsigned long long* __restrict__ out_global)
{
  extern __shared__ __align__(16) unsigned char dyn_smem[];
  __shared__ select_smem sm;
  const uint32_t q        = blockIdx.x;
  unsigned long long* out = out_global != nullptr ? out_global + uint64_t(q) * out_cap
                                                  : reinterpret_cast<unsigned long long*>(dyn_smem);
  if (only != nullptr && !only[q]) { return; }
  const float* row        = scores + uint64_t(q) * n_lists;
  auto key_of             = [row](uint32_t i) -> unsigned long long {
    const float v = row[i];
    if (v != v) { return kInvalidKey; }
    return (static_cast<unsigned long long>(order_f32(v)) << 32) | i;
  };
  block_select_sorted(key_of, n_lists, n_probes, out, out_cap, sm);
  for (uint32_t r = threadIdx.x; r < n_probes; r += kBlock) {
    const unsigned long long key = out[r];
    // fewer than n_probes comparable scores (NaN input): fall back to the slot number
    probes[uint64_t(q) * n_probes + r] = key == kInvalidKey ? (r % n_lists) : uint32_t(key);
  }
}

/*
 * Probe selection with the score row held in registers (n_probes <= 256).
 *
 * A block takes one query and walks its row in segments of 256 x PER scores (PER = 4, 16 or 64 by
 * the row's length: a short row is not padded to 16,384 loads), thread t holding scores t,
 * t + 256, ... of the segment as ordered 32-bit keys.  Bound: the smallest score of each
 * thread gives 256 distinct elements, so the n_probes-th smallest of those minima has at least
 * n_probes elements at or below it - and, for scores in no particular order, only a few more.
 * Everything at or below the bound (and the best of the earlier segments) is collected into a small
 * LDS list and sorted by (score, list id); one pass over HBM, no histogram atomics.  If the list
 * overflows (adversarially ordered rows) the block falls back to the radix selection.
 */
constexpr uint32_t kSelCap = 1024;

/** Ascending bitonic sort of one 32-bit key per lane across the wave. */
__device__ __forceinline__ uint32_t wave_sort_u32(uint32_t v, uint32_t lane)
{
#pragma unroll
  for (uint32_t size = 2; size <= 64; size <<= 1) {
#pragma unroll
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      const uint32_t other = __shfl_xor(v, int(stride), 64);
      const bool ascending = (lane & size) == 0 || size == 64;
      const bool low_half  = (lane & stride) == 0;
      const uint32_t lo    = v < other ? v : other;
      const uint32_t hi    = v < other ? other : v;
      v                    = (low_half == ascending) ? lo : hi;
    }
  }
  return v;
}

template <uint32_t kSelPerThread>
__global__ __launch_bounds__(kBlock, 3) void select_probes_fast_kernel(const float* __restrict__ scores,
                                                                     uint32_t n_lists,
                                                                     uint32_t n_probes,
                                                                     uint32_t* __restrict__ probes,
                                                                     const uint8_t* __restrict__ only)
{
  __shared__ unsigned long long cand[kSelCap];
  __shared__ unsigned long long ranked[kBlock];
  __shared__ uint32_t mins[kBlock];  // the four waves' minima, each wave's 64 sorted ascending
  __shared__ select_smem sm;
  __shared__ uint32_t s_bound, s_count;
  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = tid >> 6;
  const uint32_t q    = blockIdx.x;
  if (only != nullptr && !only[q]) { return; }
  const float* row    = scores + uint64_t(q) * n_lists;
  uint32_t have       = 0;  // sorted best-so-far in cand[0..have)
  bool overflow       = false;

  for (uint32_t seg0 = 0; seg0 < n_lists && !overflow; seg0 += kBlock * kSelPerThread) {
    uint32_t key[kSelPerThread];
    // all loads first, so that they are in flight together
    // uniform base + one per-thread offset, no clamping: the score buffer carries
    // kSelectSlackBytes of readable slack after its last row
    const float* seg = row + seg0;
#pragma unroll
    for (uint32_t j = 0; j < kSelPerThread; j++) { key[j] = __float_as_uint(seg[j * kBlock + tid]); }
    uint32_t mine = 0xFFFFFFFFu;
#pragma unroll
    for (uint32_t j = 0; j < kSelPerThread; j++) {
      const uint32_t i = seg0 + j * kBlock + tid;
      const float v    = __uint_as_float(key[j]);
      // past the end or NaN: never selected
      const uint32_t kk = (i < n_lists && v == v) ? order_f32(v) : 0xFFFFFFFFu;
      key[j]            = kk;
      mine              = kk < mine ? kk : mine;
    }
    if (tid == 0) {
      s_bound = 0xFFFFFFFFu;
      s_count = have;
    }
    // n_probes-th smallest of the 256 minima: sort per wave, then rank across the waves
    const uint32_t sorted_min = wave_sort_u32(mine, lane);
    mins[tid]                 = sorted_min;
    __syncthreads();
    uint32_t rank = lane;
#pragma unroll
    for (uint32_t w = 0; w < kBlock / 64; w++) {
      if (w == wid) { continue; }
      // elements of wave w's list ordered before (sorted_min, wid): `<=` for earlier waves
      const uint32_t* list = mins + w * 64u;
      uint32_t lo = 0, hi = 64;
#pragma unroll
      for (int step = 0; step < 6; step++) {
        const uint32_t mid = (lo + hi) >> 1;
        const uint32_t m   = list[mid];
        const bool before  = w < wid ? m <= sorted_min : m < sorted_min;
        lo                 = before ? mid + 1u : lo;
        hi                 = before ? hi : mid;
      }
      rank += lo;
    }
    if (rank == n_probes - 1u) { s_bound = sorted_min; }
    __syncthreads();
    uint32_t bound = s_bound;
    if (have == n_probes) {
      const uint32_t prev = uint32_t(cand[n_probes - 1] >> 32);
      bound               = prev < bound ? prev : bound;
    }
    // collect: only threads whose minimum is within the bound hold anything
    if (mine <= bound && mine != 0xFFFFFFFFu) {
#pragma unroll
      for (uint32_t j = 0; j < kSelPerThread; j++) {
        if (key[j] <= bound && key[j] != 0xFFFFFFFFu) {
          const uint32_t pos = atomicAdd(&s_count, 1u);
          if (pos < kSelCap) {
            cand[pos] = (static_cast<unsigned long long>(key[j]) << 32) | (seg0 + j * kBlock + tid);
          }
        }
      }
    }
    __syncthreads();
    const uint32_t total = s_count;
    if (total > kSelCap) {
      overflow = true;  // uniform
    } else if (total <= kBlock) {
      // few candidates: place each by counting the smaller ones
      unsigned long long mykey = kInvalidKey;
      uint32_t pos             = 0;
      if (tid < total) {
        mykey = cand[tid];
        for (uint32_t x = 0; x < total; x++) { pos += cand[x] < mykey ? 1u : 0u; }
      }
      __syncthreads();
      if (tid < total) { ranked[pos] = mykey; }
      __syncthreads();
      have = total < n_probes ? total : n_probes;
      if (tid < have) { cand[tid] = ranked[tid]; }
      __syncthreads();
    } else {
      const uint32_t n_sort = next_pow2_dev(total);
      for (uint32_t i = total + tid; i < n_sort; i += kBlock) { cand[i] = kInvalidKey; }
      __syncthreads();
      block_bitonic_sort(cand, n_sort);
      have = total < n_probes ? total : n_probes;
    }
  }
  if (overflow) {
    __syncthreads();
    auto key_of = [row](uint32_t i) -> unsigned long long {
      const float v = row[i];
      if (v != v) { return kInvalidKey; }
      return (static_cast<unsigned long long>(order_f32(v)) << 32) | i;
    };
    block_select_sorted(key_of, n_lists, n_probes, cand, next_pow2_dev(n_probes), sm);
    have = n_probes;  // unfilled slots hold kInvalidKey
  }
  for (uint32_t r = tid; r < n_probes; r += kBlock) {
    const unsigned long long k2 = r < have ? cand[r] : kInvalidKey;
    probes[uint64_t(q) * n_probes + r] = k2 == kInvalidKey ? (r % n_lists) : uint32_t(k2);
  }
}

/* ---------------------------------------------------------------------------------------- */
/* rotation, chunk indices, pair ordering                                                    */
/* ---------------------------------------------------------------------------------------- */

constexpr int kRotQueries = 4;

__global__ __launch_bounds__(kBlock) void rotate_kernel(const float* __restrict__ qf,
                                                         const float* __restrict__ rotation_t,
                                                         uint32_t n_queries, uint32_t dim,
                                                         uint32_t rot_dim, int identity,
                                                         int normalize, int mode,
                                                         float* __restrict__ rot_q)
{
  // mode 0: fp32 operands; 1: both rounded to binary16; 2: both as trunc(clamp(128 x)), an integer
  // dot product (exact in fp32 for dim <= 1024) times 1 / 128^2
  auto operand = [mode](float v) -> float {
    if (mode == 1) { return float(_Float16(v)); }
    if (mode == 2) { return float(int(fmaxf(-128.0f, fminf(127.0f, v * 128.0f)))); }
    return v;
  };
  extern __shared__ __align__(16) unsigned char dyn_smem[];
  float* sq           = reinterpret_cast<float*>(dyn_smem);  // [kRotQueries][dim]
  float* sr           = sq + kRotQueries * dim;              // [kRotQueries][rot_dim]
  __shared__ float s_norm[kRotQueries];
  const uint32_t q0   = blockIdx.x * kRotQueries;
  const uint32_t nq   = (n_queries - q0) < uint32_t(kRotQueries) ? (n_queries - q0) : kRotQueries;
  for (uint32_t i = threadIdx.x; i < nq * dim; i += kBlock) { sq[i] = operand(qf[uint64_t(q0) * dim + i]); }
  __syncthreads();
  for (uint32_t r = threadIdx.x; r < rot_dim; r += kBlock) {
    float acc[kRotQueries];
#pragma unroll
    for (int i = 0; i < kRotQueries; i++) { acc[i] = 0.0f; }
    if (identity) {
      // a diagonal of ones: exact in binary16; 127 as an 8-bit integer
      const float one = operand(1.0f);
#pragma unroll
      for (int i = 0; i < kRotQueries; i++) { acc[i] = (uint32_t(i) < nq) ? one * sq[i * dim + r] : 0.0f; }
    } else {
      for (uint32_t d = 0; d < dim; d++) {
        const float w = operand(rotation_t[uint64_t(d) * rot_dim + r]);
#pragma unroll
        for (int i = 0; i < kRotQueries; i++) {
          if (uint32_t(i) < nq) { acc[i] = fmaf(w, sq[i * dim + d], acc[i]); }
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kRotQueries; i++) {
      if (uint32_t(i) < nq) { sr[i * rot_dim + r] = mode == 2 ? acc[i] * (1.0f / 128.0f / 128.0f) : acc[i]; }
    }
  }
  __syncthreads();
  if (normalize) {
    // cosine: divide by the L2 norm; the sum of squares is one FMA chain in ascending order
    if (threadIdx.x < nq) {
      float ss = 0.0f;
      for (uint32_t r = 0; r < rot_dim; r++) {
        const float v = sr[threadIdx.x * rot_dim + r];
        ss            = fmaf(v, v, ss);
      }
      s_norm[threadIdx.x] = sqrtf(ss);
    }
    __syncthreads();
  }
  for (uint32_t i = threadIdx.x; i < nq * rot_dim; i += kBlock) {
    float v = sr[i];
    if (normalize) {
      const float nrm = s_norm[i / rot_dim];
      if (nrm > 0.0f) { v = v / nrm; }
    }
    rot_q[uint64_t(q0) * rot_dim + i] = v;
  }
}

/** Sort key of pair i: its list, the pairs past each query's leading probes in a second range.
 *  The leading pairs go through `rank`, when given: the list's position among all lists by size,
 *  largest first, so that they run from long lists to short ones and the pairs that share a block
 *  are of similar length (every one of them is scanned in full, a few per compute unit in all; the
 *  other pairs keep the order of the list numbers, which is the order of the lists in memory). */
__device__ __forceinline__ uint32_t pair_bin(uint32_t label, uint32_t i, uint32_t n_probes,
                                             uint32_t lead_probes, uint32_t n_lists,
                                             const uint32_t* __restrict__ rank)
{
  if ((i % n_probes) >= lead_probes) { return label + n_lists; }
  return rank != nullptr ? rank[label] : label;
}

/** One wave per query: inclusive prefix sums of the probed list sizes in probe order. */
__global__ __launch_bounds__(64) void chunk_indices_kernel(const uint32_t* __restrict__ list_sizes,
                                                            const uint32_t* __restrict__ probes,
                                                            uint32_t n_probes,
                                                            uint32_t row_chunk_bytes,
                                                            uint32_t* __restrict__ chunk_indices,
                                                            uint32_t* __restrict__ n_samples,
                                                            unsigned long long* stats,
                                                            uint32_t lead_probes,
                                                            uint32_t* __restrict__ query_max,
                                                            uint32_t* __restrict__ zero_words,
                                                            uint32_t n_zero_words)
{
  const uint32_t q    = blockIdx.x;
  const uint32_t lane = threadIdx.x;
  // start values of the scan that follows, set here to save two launches: every query's bound at
  // its largest, the survivor count at zero
  if (lane == 0 && query_max != nullptr) { query_max[q] = 0xFFFFFFFFu; }
  if (q == 0 && zero_words != nullptr) {
    for (uint32_t w = lane; w < n_zero_words; w += 64u) { zero_words[w] = 0u; }
  }
  uint32_t carry      = 0;
  unsigned long long padded_rows = 0, lead_rows = 0;
  for (uint32_t p0 = 0; p0 < n_probes; p0 += 64) {
    const uint32_t p = p0 + lane;
    uint32_t sz      = 0;
    if (p < n_probes) {
      const uint32_t label = probes[uint64_t(q) * n_probes + p];
      sz                   = list_sizes[label];
    }
    padded_rows += (sz + 31u) & ~31u;
    if (p < lead_probes) { lead_rows += (sz + 31u) & ~31u; }
    const uint32_t incl = wave_inclusive_scan(sz) + carry;
    if (p < n_probes) { chunk_indices[uint64_t(q) * n_probes + p] = incl; }
    carry = __shfl(incl, 63, 64);
  }
  if (lane == 0) { n_samples[q] = carry; }
  if (stats != nullptr) {
    // wave reduction of the padded row count
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) {
      padded_rows += __shfl_down(padded_rows, d, 64);
      lead_rows += __shfl_down(lead_rows, d, 64);
    }
    if (lane == 0) {
      // kStatSlots partial sums (the host adds them up): thousands of waves adding to one
      // address would serialise and show up in the stage times being measured
      unsigned long long* slot = stats + uint64_t(q % kStatSlots) * 4;
      atomicAdd(&slot[0], padded_rows * row_chunk_bytes);
      atomicAdd(&slot[1], static_cast<unsigned long long>(carry));
      atomicAdd(&slot[2], lead_rows * row_chunk_bytes);
    }
  }
}

__global__ void pair_histogram_kernel(const uint32_t* __restrict__ probes, uint32_t n_pairs,
                                      uint32_t n_probes, uint32_t lead_probes, uint32_t n_lists,
                                      const uint32_t* __restrict__ rank, uint32_t* __restrict__ counts)
{
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_pairs) { atomicAdd(&counts[pair_bin(probes[i], i, n_probes, lead_probes, n_lists, rank)], 1u); }
}

/** Single block of 1024 threads: cursors[l] = exclusive prefix sum of counts[l].  The counts pass
 *  through LDS in tiles of 32 per thread: loads and stores are coalesced, and a thread scans its 32
 *  consecutive values out of LDS (one padding word per 32 keeps the threads on different banks). */
constexpr uint32_t kScanThreads = 1024;
constexpr uint32_t kScanPer     = 32;
constexpr uint32_t kScanTile    = kScanThreads * kScanPer;
__global__ __launch_bounds__(kScanThreads) void exclusive_scan_kernel(const uint32_t* __restrict__ counts,
                                                                      uint32_t n,
                                                                      uint32_t* __restrict__ cursors)
{
  extern __shared__ __align__(16) uint32_t tile[];  // kScanTile + kScanThreads words
  __shared__ uint32_t wave_sums[kScanThreads / 64];
  const uint32_t tid = threadIdx.x;
  auto slot          = [](uint32_t i) { return i + (i >> 5); };
  uint32_t carry     = 0;
  for (uint32_t base = 0; base < n; base += kScanTile) {
    for (uint32_t i = tid; i < kScanTile; i += kScanThreads) {
      tile[slot(i)] = base + i < n ? counts[base + i] : 0u;
    }
    __syncthreads();
    uint32_t v[kScanPer];
    uint32_t sum = 0;
#pragma unroll
    for (uint32_t e = 0; e < kScanPer; e++) {
      v[e] = tile[slot(tid * kScanPer + e)];
      sum += v[e];
    }
    const uint32_t incl = wave_inclusive_scan(sum);
    if ((tid & 63u) == 63u) { wave_sums[tid >> 6] = incl; }
    __syncthreads();
    uint32_t run = carry + incl - sum;
    uint32_t all = 0;
    for (uint32_t w = 0; w < kScanThreads / 64; w++) {
      const uint32_t ws = wave_sums[w];
      run += w < (tid >> 6) ? ws : 0u;
      all += ws;
    }
#pragma unroll
    for (uint32_t e = 0; e < kScanPer; e++) {
      tile[slot(tid * kScanPer + e)] = run;
      run += v[e];
    }
    __syncthreads();
    for (uint32_t i = tid; i < kScanTile; i += kScanThreads) {
      if (base + i < n) { cursors[base + i] = tile[slot(i)]; }
    }
    carry += all;
    __syncthreads();  // the tile and the wave sums are reused
  }
}

/** Pair i goes to position `pos` of the order: its id, its record, its byte of `alive`. */
__device__ __forceinline__ void place_pair(uint32_t i, uint32_t pos, uint32_t label,
                                           const uint32_t* __restrict__ chunk_indices,
                                           const uint8_t* const* __restrict__ data_ptrs,
                                           const int64_t* const* __restrict__ inds_ptrs,
                                           const int64_t* ids_base, uint32_t n_probes, uint32_t lead_probes,
                                           uint32_t* __restrict__ pair_order, pair_desc* __restrict__ desc,
                                           uint8_t* __restrict__ alive)
{
  pair_order[pos] = i;
  if (alive != nullptr) { alive[i] = (i % n_probes) < lead_probes ? 1 : 0; }
  if (desc != nullptr) {
    const uint32_t q   = i / n_probes;
    const uint32_t p   = i - q * n_probes;
    const uint32_t off = p > 0 ? chunk_indices[i - 1] : 0u;
    pair_desc d;
    d.data       = data_ptrs[label];
    d.q          = q;
    d.slot       = i;
    d.label      = label;
    d.sample_off = off;
    d.n_rows     = chunk_indices[i] - off;
    d.row_off    = uint32_t(inds_ptrs[label] - ids_base);
    desc[pos]    = d;
  }
}

__global__ void pair_scatter_kernel(const uint32_t* __restrict__ probes,
                                    const uint32_t* __restrict__ chunk_indices,
                                    const uint8_t* const* __restrict__ data_ptrs,
                                    const int64_t* const* __restrict__ inds_ptrs,
                                    const int64_t* ids_base, uint32_t n_pairs,
                                    uint32_t n_probes, uint32_t lead_probes, uint32_t n_lists,
                                    const uint32_t* __restrict__ rank, uint32_t* __restrict__ cursors,
                                    uint32_t* __restrict__ pair_order, pair_desc* __restrict__ desc,
                                    uint8_t* __restrict__ alive)
{
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_pairs) {
    const uint32_t label = probes[i];
    // no cursors: the pairs keep their natural (query-major) order
    const uint32_t pos = cursors != nullptr
                           ? atomicAdd(&cursors[pair_bin(label, i, n_probes, lead_probes, n_lists, rank)], 1u)
                           : i;
    place_pair(i, pos, label, chunk_indices, data_ptrs, inds_ptrs, ids_base, n_probes, lead_probes, pair_order, desc,
               alive);
  }
}

/*
 * The pair order as a two-level counting sort.  A global atomic per pair (one for the histogram,
 * one for the position) costs about 60 ns of memory-side atomic throughput at 640,000 pairs; here
 * every count is an LDS atomic.  Level one splits the bins (lists) into at most kOrderBuckets
 * buckets of 2^shift consecutive bins: blocks of kOrderThreads threads count their chunk of pairs
 * per bucket (pair_bucket_count_kernel); every block then finds its range inside every bucket from
 * the table of (bucket, block) counts and moves (list, pair) records there
 * (pair_bucket_move_kernel).  Level two takes one block per bucket: it counts the bucket's records
 * per bin in LDS, scans, and places every pair (pair_bucket_finish_kernel).  The loops request
 * kOrderUnroll pairs' worth of loads at a time: every pair is a chain of dependent loads
 * (probe -> rank, record -> list pointers), and a block has few pairs per thread.
 */
constexpr uint32_t kOrderBuckets = 512;
constexpr uint32_t kOrderThreads = 1024;
constexpr uint32_t kOrderUnroll  = 4;
constexpr uint32_t kOrderChunk   = kOrderThreads * kOrderUnroll;  // pairs per block
constexpr uint32_t kOrderFineMax = 8192;  // bins per bucket (LDS words of the last kernel)

__global__ __launch_bounds__(kOrderThreads) void pair_bucket_count_kernel(
  const uint32_t* __restrict__ probes, uint32_t n_pairs, uint32_t n_probes, uint32_t lead_probes,
  uint32_t n_lists, const uint32_t* __restrict__ rank, uint32_t shift, uint32_t* __restrict__ block_counts)
{
  __shared__ uint32_t hist[kOrderBuckets];
  const uint32_t tid = threadIdx.x;
  if (tid < kOrderBuckets) { hist[tid] = 0; }
  __syncthreads();
  const uint32_t i0 = blockIdx.x * kOrderChunk;
  const uint32_t i1 = i0 + kOrderChunk < n_pairs ? i0 + kOrderChunk : n_pairs;
  {
    const uint32_t base = i0 + tid;
    uint32_t label[kOrderUnroll], bin[kOrderUnroll];
#pragma unroll
    for (uint32_t u = 0; u < kOrderUnroll; u++) {
      const uint32_t i = base + u * kOrderThreads;
      label[u]         = i < i1 ? probes[i] : 0u;
    }
#pragma unroll
    for (uint32_t u = 0; u < kOrderUnroll; u++) {
      bin[u] = pair_bin(label[u], base + u * kOrderThreads, n_probes, lead_probes, n_lists, rank);
    }
#pragma unroll
    for (uint32_t u = 0; u < kOrderUnroll; u++) {
      if (base + u * kOrderThreads < i1) { atomicAdd(&hist[bin[u] >> shift], 1u); }
    }
  }
  __syncthreads();
  if (tid < kOrderBuckets) { block_counts[blockIdx.x * kOrderBuckets + tid] = hist[tid]; }
}

/** A record of the first level: what the last kernel needs to know of a pair, gathered while the
 *  pairs are still in their natural order (the chunk indices of consecutive pairs are neighbours). */
struct order_record {
  uint32_t label, pair, sample_off, n_rows;
};

/** Moves the block's pairs to their buckets.  The block orders its records by bucket in LDS first,
 *  so that every bucket receives a run of consecutive records from consecutive lanes.  Also writes
 *  the byte of `alive` of every pair and, from block 0, where every bucket starts. */
__global__ __launch_bounds__(kOrderThreads) void pair_bucket_move_kernel(
  const uint32_t* __restrict__ probes, const uint32_t* __restrict__ chunk_indices, uint32_t n_pairs,
  uint32_t n_probes, uint32_t lead_probes, uint32_t n_lists, const uint32_t* __restrict__ rank,
  uint32_t shift, uint32_t n_buckets, const uint32_t* __restrict__ block_counts,
  uint32_t* __restrict__ bucket_start, order_record* __restrict__ records, uint8_t* __restrict__ alive)
{
  __shared__ uint32_t hist[kOrderBuckets];    // the block's pairs per bucket, then their local offsets
  __shared__ uint32_t gbase[kOrderBuckets];   // pairs of the blocks before this one, then the block's global range
  __shared__ uint32_t totals[kOrderBuckets];  // pairs of all blocks
  __shared__ uint32_t wave_sums[2][kOrderBuckets / 64];
  __shared__ order_record staged[kOrderChunk];
  __shared__ uint16_t staged_bucket[kOrderChunk];
  const uint32_t tid = threadIdx.x;
  if (tid < kOrderBuckets) { hist[tid] = 0; }
  // the table is [block][bucket]: thread (bucket, half) sums every other row of its column in
  // registers (LDS atomics here cost more than everything else in this kernel)
  {
    static_assert(kOrderThreads == 2 * kOrderBuckets, "two threads per bucket");
    const uint32_t bkt = tid % kOrderBuckets, half = tid / kOrderBuckets;
    uint32_t total = 0, before = 0;
#pragma unroll 8
    for (uint32_t k = half; k < gridDim.x; k += 2) {
      const uint32_t c = block_counts[k * kOrderBuckets + bkt];
      total += c;
      before += k < blockIdx.x ? c : 0u;
    }
    if (half == 1) {
      totals[bkt] = total;
      gbase[bkt]  = before;
    }
    __syncthreads();
    if (half == 0) {
      totals[bkt] += total;
      gbase[bkt] += before;
    }
  }
  const uint32_t i0 = blockIdx.x * kOrderChunk;
  const uint32_t i1 = i0 + kOrderChunk < n_pairs ? i0 + kOrderChunk : n_pairs;
  order_record rec[kOrderUnroll];
  uint32_t bucket[kOrderUnroll], local[kOrderUnroll];
#pragma unroll
  for (uint32_t u = 0; u < kOrderUnroll; u++) {
    const uint32_t i = i0 + tid + u * kOrderThreads;
    const bool in    = i < i1;
    rec[u].label     = in ? probes[i] : 0u;
    rec[u].pair      = i;
    const uint32_t incl = in ? chunk_indices[i] : 0u;
    rec[u].sample_off   = in && (i % n_probes) != 0 ? chunk_indices[i - 1] : 0u;
    rec[u].n_rows       = incl - rec[u].sample_off;
    if (in && alive != nullptr) { alive[i] = (i % n_probes) < lead_probes ? 1 : 0; }
  }
#pragma unroll
  for (uint32_t u = 0; u < kOrderUnroll; u++) {
    bucket[u] = pair_bin(rec[u].label, rec[u].pair, n_probes, lead_probes, n_lists, rank) >> shift;
  }
#pragma unroll
  for (uint32_t u = 0; u < kOrderUnroll; u++) {
    local[u] = i0 + tid + u * kOrderThreads < i1 ? atomicAdd(&hist[bucket[u]], 1u) : 0u;
  }
  __syncthreads();
  // exclusive scans over the buckets: of the block's counts (local offsets) and of the totals
  // (bucket starts; plus the blocks before this one: the block's range in the bucket)
  uint32_t mine = 0, total = 0;
  if (tid < kOrderBuckets) {
    mine  = hist[tid];
    total = totals[tid];
    const uint32_t incl_m = wave_inclusive_scan(mine);
    const uint32_t incl_t = wave_inclusive_scan(total);
    if ((tid & 63u) == 63u) {
      wave_sums[0][tid >> 6] = incl_m;
      wave_sums[1][tid >> 6] = incl_t;
    }
    mine  = incl_m - mine;
    total = incl_t - total;
  }
  __syncthreads();
  if (tid < kOrderBuckets) {
    for (uint32_t w = 0; w < (tid >> 6); w++) {
      mine += wave_sums[0][w];
      total += wave_sums[1][w];
    }
    hist[tid] = mine;
    if (blockIdx.x == 0 && tid < n_buckets) { bucket_start[tid] = total; }
    gbase[tid] += total;
  }
  __syncthreads();
#pragma unroll
  for (uint32_t u = 0; u < kOrderUnroll; u++) {
    if (i0 + tid + u * kOrderThreads < i1) {
      const uint32_t at = hist[bucket[u]] + local[u];
      staged[at]        = rec[u];
      staged_bucket[at] = uint16_t(bucket[u]);
    }
  }
  __syncthreads();
  for (uint32_t at = tid; at < i1 - i0; at += kOrderThreads) {
    const uint32_t b              = staged_bucket[at];
    records[gbase[b] + at - hist[b]] = staged[at];
  }
}

__global__ __launch_bounds__(kOrderThreads) void pair_bucket_finish_kernel(
  const order_record* __restrict__ records, const uint32_t* __restrict__ bucket_start, uint32_t n_buckets,
  uint32_t n_pairs, uint32_t shift, uint32_t n_lists, const uint32_t* __restrict__ rank,
  const uint8_t* const* __restrict__ data_ptrs, const int64_t* const* __restrict__ inds_ptrs,
  const int64_t* ids_base, uint32_t n_probes, uint32_t lead_probes, uint32_t* __restrict__ pair_order,
  pair_desc* __restrict__ desc)
{
  extern __shared__ __align__(16) uint32_t fine[];  // 2^shift counts, then cursors
  __shared__ uint32_t wave_sums[kOrderThreads / 64];
  constexpr uint32_t U  = 4;
  const uint32_t tid    = threadIdx.x;
  const uint32_t b      = blockIdx.x;
  const uint32_t n_fine = 1u << shift;
  const uint32_t begin  = bucket_start[b];
  const uint32_t end    = b + 1 < n_buckets ? bucket_start[b + 1] : n_pairs;
  for (uint32_t f = tid; f < n_fine; f += kOrderThreads) { fine[f] = 0; }
  __syncthreads();
  for (uint32_t base = begin + tid; base < end; base += kOrderThreads * U) {
    uint32_t label[U], pair[U], bin[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const uint32_t e = base + u * kOrderThreads;
      label[u]         = e < end ? records[e].label : 0u;
      pair[u]          = e < end ? records[e].pair : 0u;
    }
#pragma unroll
    for (uint32_t u = 0; u < U; u++) { bin[u] = pair_bin(label[u], pair[u], n_probes, lead_probes, n_lists, rank); }
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      if (base + u * kOrderThreads < end) { atomicAdd(&fine[bin[u] & (n_fine - 1u)], 1u); }
    }
  }
  __syncthreads();
  // exclusive scan of the counts: every thread owns a run of consecutive bins
  const uint32_t per = (n_fine + kOrderThreads - 1) / kOrderThreads;
  const uint32_t f0  = tid * per;
  uint32_t sum       = 0;
  for (uint32_t f = f0; f < f0 + per && f < n_fine; f++) { sum += fine[f]; }
  const uint32_t incl = wave_inclusive_scan(sum);
  if ((tid & 63u) == 63u) { wave_sums[tid >> 6] = incl; }
  __syncthreads();
  uint32_t run = begin + incl - sum;
  for (uint32_t w = 0; w < (tid >> 6); w++) { run += wave_sums[w]; }
  for (uint32_t f = f0; f < f0 + per && f < n_fine; f++) {
    const uint32_t c = fine[f];
    fine[f]          = run;
    run += c;
  }
  __syncthreads();
  for (uint32_t base = begin + tid; base < end; base += kOrderThreads * U) {
    order_record r[U];
    uint32_t bin[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const uint32_t e = base + u * kOrderThreads;
      r[u]             = e < end ? records[e] : order_record{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (uint32_t u = 0; u < U; u++) { bin[u] = pair_bin(r[u].label, r[u].pair, n_probes, lead_probes, n_lists, rank); }
    pair_desc d[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      d[u].data       = data_ptrs[r[u].label];
      d[u].q          = r[u].pair / n_probes;
      d[u].slot       = r[u].pair;
      d[u].label      = r[u].label;
      d[u].sample_off = r[u].sample_off;
      d[u].n_rows     = r[u].n_rows;
      d[u].row_off    = uint32_t(inds_ptrs[r[u].label] - ids_base);
    }
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      if (base + u * kOrderThreads < end) {
        const uint32_t pos = atomicAdd(&fine[bin[u] & (n_fine - 1u)], 1u);
        pair_order[pos]    = r[u].pair;
        if (desc != nullptr) { desc[pos] = d[u]; }
      }
    }
  }
}

/* ---------------------------------------------------------------------------------------- */
/* the scan kernel: one block per (query, probed list) pair                                   */
/* ---------------------------------------------------------------------------------------- */

constexpr uint32_t kCandCap = 1024;  // per-block candidate buffer (keys), >= k + kBlock

/** One wave keeps the k smallest of the n <= kCandCap keys of the block's buffer at its front (in no
 *  particular order) by radix selection on its registers; returns the k-th smallest's high word. */
__device__ __forceinline__ uint32_t keep_smallest_keys(unsigned long long* cand, uint32_t lane, uint32_t n, uint32_t k)
{
  auto* buf = (LDS_AS unsigned long long*)cand;
  return n <= 256u ? wave_select_keys<4>(buf, lane, n, k)
         : n <= 512u ? wave_select_keys<8>(buf, lane, n, k)
                     : wave_select_keys<16>(buf, lane, n, k);
}

struct scan_smem_tail {
  uint32_t count;
  uint32_t thr;
};

template <int LUT, bool OUT_HALF, int BITS, bool FUSED, bool GLOBAL_LUT>
__global__ __launch_bounds__(kBlock) void scan_kernel(scan_args a)
{
  using traits  = lut_traits<LUT>;
  using lut_t   = typename traits::storage;
  using acc_t   = typename std::conditional<OUT_HALF, _Float16, float>::type;
  constexpr uint32_t B   = 1u << BITS;
  constexpr uint32_t CPC = 128u / BITS;  // codes per 16-byte chunk

  extern __shared__ __align__(16) unsigned char dyn_smem[];
  const uint32_t lut_entries = a.pq_dim << BITS;
  // the table lives in LDS, or, when it does not fit, in this block's slice of a global scratch
  // buffer (the reference's third kernel variant, ivf_pq_compute_similarity_impl.cuh:337-596)
  lut_t* lut = GLOBAL_LUT ? static_cast<lut_t*>(a.global_lut) + uint64_t(blockIdx.x) * lut_entries
                          : reinterpret_cast<lut_t*>(dyn_smem);
  const uint32_t lut_bytes = GLOBAL_LUT ? 0u : (lut_entries * uint32_t(sizeof(lut_t)) + 15u) & ~15u;
  float* base_diff         = reinterpret_cast<float*>(dyn_smem + lut_bytes);
  const bool ip              = is_ip_metric(a.metric);
  const uint32_t diff_floats = a.rot_dim * (ip ? 2u : 1u);
  unsigned long long* cand =
    reinterpret_cast<unsigned long long*>(dyn_smem + lut_bytes + ((diff_floats * 4u + 15u) & ~15u));
  scan_smem_tail* tail = reinterpret_cast<scan_smem_tail*>(cand + (FUSED ? kCandCap : 0));

  const uint32_t tid = threadIdx.x;
  // one pair per block; with a global table, or a number of pairs only the device knows, a bounded
  // grid walks over the pairs.  A subset of the pairs (the leading or the surviving ones of an early
  // stop) comes as a list of records.
  const uint32_t n_work = a.subset != 0 ? (a.n_pairs_dev != nullptr ? *a.n_pairs_dev : a.n_pairs)
                                        : a.n_queries * a.n_probes;
  for (uint32_t pb = blockIdx.x; pb < n_work; pb += gridDim.x) {
  const uint32_t pair = a.subset != 0 ? a.desc[pb].slot : a.pair_order != nullptr ? a.pair_order[pb] : pb;
  const uint32_t q    = pair / a.n_probes;
  const uint32_t p    = pair - q * a.n_probes;
  const uint32_t label = a.probes[uint64_t(q) * a.n_probes + p];
  const uint32_t* chunk_row = a.chunk_indices + uint64_t(q) * a.n_probes;
  const uint32_t sample_off = p > 0 ? chunk_row[p - 1] : 0u;
  const uint32_t n_rows     = chunk_row[p] - sample_off;

  /* ---- stage the per-dimension query/centre terms ---- */
  const float* rq = a.rot_q + uint64_t(q) * a.rot_dim;
  const float* cr = a.centers_rot + uint64_t(label) * a.rot_dim;
  for (uint32_t i = tid; i < a.rot_dim; i += kBlock) {
    if (!ip) {
      base_diff[i] = rq[i] - cr[i];
    } else {
      const float qv       = rq[i];
      base_diff[2 * i]     = qv;
      base_diff[2 * i + 1] = cr[i] * qv;
    }
  }
  if (FUSED && tid == 0) {
    tail->count = 0;
    tail->thr   = 0xFFFFFFFFu;
  }
  __syncthreads();

  /* ---- lookup table: LUT[j][code] = LutT(score of codebook entry `code` in subspace j) ---- */
  {
    const float* books = a.pq_centers +
                         (a.per_cluster ? uint64_t(label) * a.pq_len * B : uint64_t(0));
    for (uint32_t i = tid; i < lut_entries; i += kBlock) {
      const uint32_t j    = i >> BITS;
      const uint32_t code = i & (B - 1u);
      const float* book   = books + (a.per_cluster ? uint64_t(0) : uint64_t(j) * a.pq_len * B) + code;
      float score         = 0.0f;
      for (uint32_t t = 0; t < a.pq_len; t++) {
        const float pqc  = book[uint64_t(t) * B];
        const uint32_t d = j * a.pq_len + t;
        if (!ip) {
          float diff = base_diff[d];
          diff -= pqc;
          score = fmaf(diff, diff, score);
        } else {
          const float qv = base_diff[2 * d];
          score -= base_diff[2 * d + 1];
          score = fmaf(-qv, pqc, score);
        }
      }
      lut[i] = traits::encode(score);
    }
  }
  __syncthreads();

  /* ---- scan the list ---- */
  const uint8_t* list_data = a.data_ptrs[label];
  const int64_t* list_ids  = a.filter_bits != nullptr ? a.inds_ptrs[label] : nullptr;
  const uint32_t n_chunks  = (a.pq_dim + CPC - 1u) / CPC;
  const uint32_t n_full    = a.pq_dim / CPC;
  const uint32_t n_padded  = (n_rows + 31u) & ~31u;
  uint32_t thr             = 0xFFFFFFFFu;
  if (FUSED) { thr = a.query_kth[q]; }

  for (uint32_t i0 = 0; i0 < n_padded; i0 += kBlock) {
    const uint32_t i = i0 + tid;
    bool valid       = i < n_rows;
    if (valid && list_ids != nullptr) {
      const int64_t id = list_ids[i];
      valid = id >= 0 && id < a.filter_nbits && ((a.filter_bits[id >> 5] >> (id & 31)) & 1u) != 0;
    }
    float score_f = 0.0f;
    // L2 sums only grow: when every row of the wave is above the bound after a chunk, the rest of
    // the row cannot matter (compute_score's early stop); the wave then leaves the chunk loop
    const uint32_t stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
    bool stopped             = false;  // wave-uniform
    {
      const uint8_t* ptr =
        list_data + uint64_t(valid ? (i >> 5) : 0u) * n_chunks * 512u + uint64_t(i & 31u) * 16u;
      acc_t acc        = acc_t(0);
      const lut_t* lh  = lut;
      for (uint32_t m = 0; m < n_full && !stopped; m++) {
        if (valid) {
          const uint4 v       = *reinterpret_cast<const uint4*>(ptr + uint64_t(m) * 512u);
          const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (uint32_t kk = 0; kk < CPC; kk++) {
            constexpr uint32_t mask = B - 1u;
            const uint32_t bit      = kk * BITS;
            const uint32_t word     = bit >> 5;
            const uint32_t off      = bit & 31u;
            uint32_t c              = w[word] >> off;
            if (off + BITS > 32u) { c |= w[(word + 1u) & 3u] << (32u - off); }
            c &= mask;
            if (OUT_HALF) {
              acc = acc_t(acc + traits::to_half(lh[(kk << BITS) + c]));
            } else {
              acc = acc_t(acc + traits::to_float(lh[(kk << BITS) + c]));
            }
          }
        }
        lh += CPC << BITS;
        if (FUSED && !ip && m + 1u < n_chunks) {
          stopped = __ballot(valid && !(__float_as_uint(float(acc)) > stop_bits)) == 0ull;
        }
      }
      if (n_full < n_chunks && valid && !stopped) {
        const uint4 v       = *reinterpret_cast<const uint4*>(ptr + uint64_t(n_full) * 512u);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        const uint32_t rem  = a.pq_dim - n_full * CPC;
#pragma unroll
        for (uint32_t kk = 0; kk < CPC; kk++) {
          if (kk < rem) {
            constexpr uint32_t mask = B - 1u;
            const uint32_t bit      = kk * BITS;
            const uint32_t word     = bit >> 5;
            const uint32_t off      = bit & 31u;
            uint32_t c              = w[word] >> off;
            if (off + BITS > 32u) { c |= w[(word + 1u) & 3u] << (32u - off); }
            c &= mask;
            if (OUT_HALF) {
              acc = acc_t(acc + traits::to_half(lh[(kk << BITS) + c]));
            } else {
              acc = acc_t(acc + traits::to_float(lh[(kk << BITS) + c]));
            }
          }
        }
      }
      if (a.metric == int(DistanceType::CosineExpanded)) { acc = acc_t(acc + acc_t(1)); }
      score_f = float(acc);
    }
    if (score_f != score_f) { valid = false; }  // NaN never enters a result

    if (FUSED) {
      if (valid) {
        const uint32_t okey = order_f32(score_f);
        if (okey <= thr) {
          const uint32_t pos = atomicAdd(&tail->count, 1u);
          cand[pos] = (static_cast<unsigned long long>(okey) << 32) | (sample_off + i);
        }
      }
      __syncthreads();
      const uint32_t cnt = tail->count;
      __syncthreads();  // every thread has read the count before anyone appends again
      if (cnt > kCandCap - kBlock) {
        // prune: keep the k smallest candidates (k <= kCandCap - kBlock < cnt), tighten the threshold
        if (tid < 64u) {
          const uint32_t kth = keep_smallest_keys(cand, tid, cnt, a.k);
          if (tid == 0) {
            tail->count = a.k;
            tail->thr   = kth;
          }
        }
        __syncthreads();
        const uint32_t t2 = tail->thr;
        thr               = t2 < thr ? t2 : thr;
      }
    } else {
      if (i < n_rows) {
        a.out_scores[uint64_t(q) * a.max_samples + sample_off + i] =
          valid ? score_f : __uint_as_float(0x7fc00000u);
      }
    }
  }

  if (FUSED) {
    __syncthreads();
    uint32_t cnt = tail->count;
    if (cnt >= a.k) {
      if (tid < 64u) {
        const uint32_t kth = keep_smallest_keys(cand, tid, cnt, a.k);
        if (tid == 0) { atomicMin(&a.query_kth[q], kth); }
      }
      __syncthreads();
      cnt = a.k;
    }
    unsigned long long* out = a.out_keys + (uint64_t(q) * a.n_probes + p) * a.k;
    for (uint32_t r = tid; r < a.k; r += kBlock) { out[r] = r < cnt ? cand[r] : kInvalidKey; }
  }
  __syncthreads();  // the next pair of this block reuses the table and the candidate buffer
  }
}

/* ---------------------------------------------------------------------------------------- */
/* per-query merge + post-processing                                                          */
/* ---------------------------------------------------------------------------------------- */

__device__ __forceinline__ float postprocess_distance(float d, int metric, float s)
{
  // cuVS postprocess_distances (cpp/src/neighbors/ivf_common.cuh:175-252)
  switch (metric) {
    case int(DistanceType::L2Expanded): return s != 1.0f ? d * (s * s) : d;
    case int(DistanceType::L2SqrtExpanded): return s != 1.0f ? sqrtf(d) * s : sqrtf(d);
    case int(DistanceType::InnerProduct): return d * (-1.0f * s * s);
    case int(DistanceType::CosineExpanded): return s != 1.0f ? d * (s * s) : d;
    default: return d;
  }
}

/** One wave per query: the k-th smallest valid key among the first n_keys keys of the query's
 *  candidate block bounds the query's final k-th score from above.  The keys' score words sit in
 *  registers (NK a lane) and the wave's radix selection finds the k-th (ballots and counts, no LDS);
 *  slots that hold no key count as the largest word, so fewer than k keys give no bound. */
constexpr uint32_t kKthMaxKeys = 1024;
template <int NK>
__global__ __launch_bounds__(256) void kth_bound_kernel(const unsigned long long* __restrict__ keys,
                                                        uint64_t keys_per_query, uint32_t n_keys, uint32_t k,
                                                        uint32_t n_queries, uint32_t* __restrict__ query_kth)
{
  const uint32_t q    = blockIdx.x * 4u + (threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63u;
  if (q >= n_queries) { return; }
  const unsigned long long* mine = keys + uint64_t(q) * keys_per_query;
  uint32_t value[NK];
  unsigned long long live[NK];
#pragma unroll
  for (int j = 0; j < NK; j++) {
    const uint32_t i = uint32_t(j) * 64u + lane;
    value[j]         = i < n_keys ? uint32_t(mine[i] >> 32) : 0xFFFFFFFFu;  // kInvalidKey's score word is the largest too
    live[j]          = ~0ull;
  }
  const uint32_t kth = wave_kth_smallest<NK>(value, live, k, lane);
  if (lane == 0 && kth != 0xFFFFFFFFu) { atomicMin(&query_kth[q], kth); }
}

/** Output row r of query q from its r-th best key: the sample number inside the query's probed
 *  lists back to a list and a row (find_chunk_ix, cpp/src/neighbors/ivf_common.cuh:94-110), the
 *  distance in the metric's final form.  `chunk` and `probes` are the query's rows. */
__device__ __forceinline__ void write_neighbor(const merge_args& a, uint32_t q, uint32_t r, unsigned long long key,
                                               const uint32_t* chunk, const uint32_t* probes)
{
  int64_t id = INT64_MAX;  // kOutOfBoundsRecord
  float d    = FLT_MAX;
  if (key != kInvalidKey) {
    uint32_t sample = uint32_t(key);
    d               = unorder_f32(uint32_t(key >> 32));
    uint32_t lo = 0, hi = a.n_probes;
    do {
      const uint32_t mid = (lo + hi) >> 1;
      if (chunk[mid] <= sample) {
        lo = mid + 1;
      } else {
        hi = mid;
      }
    } while (lo < hi);
    if (lo < a.n_probes) {
      if (lo > 0) { sample -= chunk[lo - 1]; }
      id = a.inds_ptrs[probes[lo]][sample];
    }
  }
  a.neighbors[uint64_t(q) * a.k + r] = id;
  a.distances[uint64_t(q) * a.k + r] = postprocess_distance(d, a.metric, a.scaling);
}

/**
 * The merge after an early stop, one wave per query: most pairs were dropped by the screen and
 * wrote no keys, a handful is left (a.alive).  The wave lists the live pairs, packs their valid
 * keys into LDS (a pair's block of keys is mostly padding), keeps the k smallest by the wave's
 * radix selection, ranks those against each other (keys are distinct: the sample number is part of
 * the key) and writes them out; the query's chunk indices and probes sit in LDS for the search
 * from sample number to list.  A query with more than CAP valid keys is left to
 * merge_redo_kernel (a.redo[q] = 1).  kLiveSmall: 1024 keys at or below the query's bound.
 */
constexpr uint32_t kLiveSmall = 1024;
constexpr uint32_t kRedoQueries = 16;  // queries whose flags a block of merge_redo_kernel looks at
__global__ __launch_bounds__(64) void merge_live_kernel(merge_args a)
{
  extern __shared__ __align__(16) unsigned char dyn_smem[];
  unsigned long long* small_keys = reinterpret_cast<unsigned long long*>(dyn_smem);  // [kLiveSmall]
  unsigned long long* out        = small_keys + kLiveSmall;                          // [k]
  uint32_t* chunk                = reinterpret_cast<uint32_t*>(out + a.k);           // [n_probes]
  uint32_t* probes               = chunk + a.n_probes;                               // [n_probes]
  uint16_t* live                 = reinterpret_cast<uint16_t*>(probes + a.n_probes);  // [n_probes]
  const uint32_t q    = blockIdx.x;
  const uint32_t lane = threadIdx.x;
  const uint32_t kpp  = a.keys_per_pair;
  const unsigned long long* keys = a.in_keys + uint64_t(q) * a.n_probes * kpp;
  const uint8_t* alive           = a.alive + uint64_t(q) * a.n_probes;
  uint32_t n_live                = 0;
  for (uint32_t p0 = 0; p0 < a.n_probes; p0 += 64) {
    const uint32_t p = p0 + lane;
    bool al          = false;
    if (p < a.n_probes) {
      al        = alive[p] != 0;
      chunk[p]  = a.chunk_indices[uint64_t(q) * a.n_probes + p];
      probes[p] = a.probes[uint64_t(q) * a.n_probes + p];
    }
    const unsigned long long mask = __builtin_amdgcn_ballot_w64(al);
    if (al) { live[n_live + __builtin_amdgcn_mbcnt_hi(uint32_t(mask >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(mask), 0u))] = uint16_t(p); }
    n_live += uint32_t(__popcll(mask));
  }
  __syncthreads();
  // the valid keys of the live pairs, packed; lanes walk a pair's keys, pair after pair
  const uint32_t n_keys = n_live * kpp;
  uint32_t n_valid      = 0;
  // the scans leave an upper bound of the query's final k-th score behind (the smallest k-th best
  // any wave has seen): keys above it cannot be among the k best
  const uint32_t bound = a.bound != nullptr ? a.bound[q] : 0xFFFFFFFFu;
  constexpr uint32_t U  = 4;  // keys a lane requests at a time: a query with many live pairs is a chain of loads
  for (uint32_t i0 = 0; i0 < n_keys && n_valid <= kLiveSmall; i0 += 64 * U) {
    unsigned long long key[U];
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const uint32_t i = i0 + u * 64 + lane;
      key[u]           = kInvalidKey;
      if (i < n_keys) {
        const uint32_t pair = i / kpp;
        key[u]              = keys[uint32_t(live[pair]) * kpp + (i - pair * kpp)];
      }
    }
#pragma unroll
    for (uint32_t u = 0; u < U; u++) {
      const bool valid              = key[u] != kInvalidKey && uint32_t(key[u] >> 32) <= bound;
      const unsigned long long mask = __builtin_amdgcn_ballot_w64(valid);
      const uint32_t at = n_valid + __builtin_amdgcn_mbcnt_hi(uint32_t(mask >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(mask), 0u));
      if (valid && at < kLiveSmall) { small_keys[at] = key[u]; }
      n_valid += uint32_t(__popcll(mask));
    }
  }
  if (lane == 0) { a.redo[q] = n_valid > kLiveSmall ? 1 : 0; }
  if (n_valid > kLiveSmall) { return; }
  for (uint32_t r = lane; r < a.k; r += 64) { out[r] = kInvalidKey; }
  __syncthreads();
  uint32_t m = n_valid;
  if (n_valid > a.k) {
    if (n_valid <= 256u) {
      wave_select_keys<4>((LDS_AS unsigned long long*)small_keys, lane, n_valid, a.k);
    } else if (n_valid <= 512u) {
      wave_select_keys<8>((LDS_AS unsigned long long*)small_keys, lane, n_valid, a.k);
    } else {
      wave_select_keys<16>((LDS_AS unsigned long long*)small_keys, lane, n_valid, a.k);
    }
    m = a.k;
  }
  __syncthreads();
  for (uint32_t i = lane; i < m; i += 64) {
    const unsigned long long key = small_keys[i];
    uint32_t rank                = 0;
    for (uint32_t j = 0; j < m; j++) { rank += small_keys[j] < key ? 1u : 0u; }
    out[rank] = key;
  }
  __syncthreads();
  for (uint32_t r = lane; r < a.k; r += 64) { write_neighbor(a, q, r, out[r], chunk, probes); }
}

constexpr uint32_t kMergeMaxProbes = 8192;  // with the alive list: slots are kept as 16-bit numbers
/** The k best of query q, by the whole block. */
__device__ void merge_query(const merge_args& a, uint32_t out_cap, uint32_t q)
{
  extern __shared__ __align__(16) unsigned char dyn_smem[];
  __shared__ select_smem sm;
  unsigned long long* out = a.out_scratch != nullptr ? a.out_scratch + uint64_t(q) * out_cap
                                                     : reinterpret_cast<unsigned long long*>(dyn_smem);
  uint32_t n;
  if (a.fused) {
    n                              = a.n_probes * a.keys_per_pair;
    const unsigned long long* keys = a.in_keys + uint64_t(q) * n;
    if (a.alive == nullptr) {
      auto key_of = [keys](uint32_t i) { return keys[i]; };
      if (!(a.k <= kBlock && block_select_by_minima(key_of, n, a.k, out, out_cap, sm))) {
        block_select_sorted(key_of, n, a.k, out, out_cap, sm);
      }
    } else {
      // pairs that the screen dropped wrote no keys: gather the slots that did, select among those
      // (the slot list follows the output area in the launch's LDS: n_probes 16-bit numbers)
      uint16_t* live_slots =
        reinterpret_cast<uint16_t*>(dyn_smem + (a.out_scratch != nullptr ? 0u : out_cap * 8u));
      __shared__ uint32_t n_live;
      const uint8_t* alive = a.alive + uint64_t(q) * a.n_probes;
      const uint32_t kpp   = a.keys_per_pair;
      if (threadIdx.x == 0) { n_live = 0; }
      __syncthreads();
      for (uint32_t p = threadIdx.x; p < a.n_probes; p += kBlock) {
        if (alive[p] != 0) { live_slots[atomicAdd(&n_live, 1u)] = uint16_t(p); }
      }
      __syncthreads();
      const uint32_t n_keys = n_live * kpp;
      constexpr uint32_t kSmall = 512;
      if (n_keys <= kSmall) {
        // a handful of live pairs (the usual case after screening): rank every key against all
        // others in LDS; keys are distinct (the sample number is part of the key)
        static_assert(sizeof(sm.hist) >= kSmall * sizeof(unsigned long long), "small_keys area");
        unsigned long long* small_keys = reinterpret_cast<unsigned long long*>(sm.hist);
        for (uint32_t i = threadIdx.x; i < n_keys; i += kBlock) {
          small_keys[i] = keys[uint32_t(live_slots[i / kpp]) * kpp + i % kpp];
        }
        for (uint32_t r = threadIdx.x; r < a.k; r += kBlock) { out[r] = kInvalidKey; }
        __syncthreads();
        for (uint32_t i = threadIdx.x; i < n_keys; i += kBlock) {
          const unsigned long long key = small_keys[i];
          if (key == kInvalidKey) { continue; }
          uint32_t rank = 0;
          for (uint32_t j = 0; j < n_keys; j++) { rank += small_keys[j] < key ? 1u : 0u; }
          if (rank < a.k) { out[rank] = key; }
        }
        __syncthreads();
      } else {
        auto key_of = [keys, kpp, live_slots](uint32_t i) { return keys[uint32_t(live_slots[i / kpp]) * kpp + i % kpp]; };
        if (!(a.k <= kBlock && block_select_by_minima(key_of, n_keys, a.k, out, out_cap, sm))) {
          block_select_sorted(key_of, n_keys, a.k, out, out_cap, sm);
        }
      }
    }
  } else {
    n                = a.n_samples[q];
    const float* row = a.in_scores + uint64_t(q) * a.max_samples;
    block_select_sorted(
      [row](uint32_t i) -> unsigned long long {
        const float v = row[i];
        if (v != v) { return kInvalidKey; }
        return (static_cast<unsigned long long>(order_f32(v)) << 32) | i;
      },
      n, a.k, out, out_cap, sm);
  }
  const uint32_t* chunk  = a.chunk_indices + uint64_t(q) * a.n_probes;
  const uint32_t* probes = a.probes + uint64_t(q) * a.n_probes;
  for (uint32_t r = threadIdx.x; r < a.k; r += kBlock) { write_neighbor(a, q, r, out[r], chunk, probes); }
}

__global__ __launch_bounds__(kBlock) void merge_kernel(merge_args a, uint32_t out_cap) { merge_query(a, out_cap, blockIdx.x); }

/** The queries merge_live_kernel left over (a.redo), normally none: a block looks at the flags of
 *  kRedoQueries queries and merges the flagged ones one after the other. */
__global__ __launch_bounds__(kBlock) void merge_redo_kernel(merge_args a, uint32_t out_cap)
{
  __shared__ uint32_t todo[kRedoQueries];
  __shared__ uint32_t n_todo;
  if (threadIdx.x == 0) { n_todo = 0; }
  __syncthreads();
  const uint32_t q = blockIdx.x * kRedoQueries + threadIdx.x;
  if (threadIdx.x < kRedoQueries && q < a.n_queries && a.redo[q] != 0) { todo[atomicAdd(&n_todo, 1u)] = q; }
  __syncthreads();
  const uint32_t n = n_todo;
  for (uint32_t i = 0; i < n; i++) {
    merge_query(a, out_cap, todo[i]);
    __syncthreads();
  }
}

/* ---------------------------------------------------------------------------------------- */
/* list maintenance and encoding                                                              */
/* ---------------------------------------------------------------------------------------- */

/** One thread per row: x /= ||x||_2, the sum of squares being one FMA chain in ascending order. */
__global__ void normalize_rows_kernel(float* __restrict__ x, uint64_t n_rows, uint32_t dim)
{
  const uint64_t r = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (r >= n_rows) { return; }
  float* row = x + r * dim;
  float ss   = 0.0f;
  for (uint32_t d = 0; d < dim; d++) { ss = fmaf(row[d], row[d], ss); }
  const float nrm = sqrtf(ss);
  if (nrm > 0.0f) {
    for (uint32_t d = 0; d < dim; d++) { row[d] = row[d] / nrm; }
  }
}

__global__ void histogram_kernel(const uint32_t* __restrict__ labels, uint64_t n, uint32_t n_bins,
                                 uint32_t* __restrict__ counts)
{
  // labels outside the bins are not counted: the caller sees them as a short total
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) {
    const uint32_t l = labels[i];
    if (l < n_bins) { atomicAdd(&counts[l], 1u); }
  }
}

/** One block per list: move the occupied 32-row groups and ids to their new arena position. */
__global__ __launch_bounds__(kBlock) void relocate_lists_kernel(
  const uint8_t* __restrict__ old_codes, const int64_t* __restrict__ old_ids,
  uint8_t* __restrict__ new_codes, int64_t* __restrict__ new_ids,
  const uint64_t* __restrict__ old_row_offsets, const uint64_t* __restrict__ new_row_offsets,
  const uint32_t* __restrict__ old_sizes, uint32_t n_chunks)
{
  const uint32_t l  = blockIdx.x;
  const uint32_t sz = old_sizes[l];
  if (sz == 0) { return; }
  const uint64_t group_bytes = uint64_t(n_chunks) * 512u;
  const uint64_t n_vec       = uint64_t((sz + 31u) >> 5) * group_bytes / 16u;
  const uint4* src = reinterpret_cast<const uint4*>(old_codes + (old_row_offsets[l] >> 5) * group_bytes);
  uint4* dst       = reinterpret_cast<uint4*>(new_codes + (new_row_offsets[l] >> 5) * group_bytes);
  for (uint64_t i = threadIdx.x; i < n_vec; i += kBlock) { dst[i] = src[i]; }
  const int64_t* si = old_ids + old_row_offsets[l];
  int64_t* di       = new_ids + new_row_offsets[l];
  for (uint32_t i = threadIdx.x; i < sz; i += kBlock) { di[i] = si[i]; }
}

/**
 * One thread per row.  residual = rotation * (x - centre[label]) with FMA chains in ascending
 * order; code_j = argmin over the codebook of the squared distance, lowest code wins ties
 * (cuVS ivf_pq_build.cuh:140-206, ivf_pq_process_and_fill_codes.cuh:84-126).
 * The rotated residual of a row is kept in column r of `a.scratch` ([rot_dim, n], so that the
 * threads of a wave touch consecutive addresses).  With per-subspace codebooks every thread of
 * the block reads the same codebook element at the same time, which the compiler turns into
 * scalar loads.
 */
template <int BITS, bool PER_CLUSTER>
__global__ __launch_bounds__(kBlock) void encode_kernel(encode_args a)
{
  constexpr uint32_t B   = 1u << BITS;
  constexpr uint32_t CPC = 128u / BITS;
  // per-subspace codebooks: the block stages one subspace's book in LDS at a time (two buffers)
  // and every lane reads the same entry at the same time, a broadcast
  constexpr uint32_t kBookMaxLen = 8;  // pq_len up to which the LDS path is used
  __shared__ float sbook[2][PER_CLUSTER ? 1 : B * kBookMaxLen];
  const bool lds_book = !PER_CLUSTER && a.pq_len <= kBookMaxLen;
  const uint64_t r0   = uint64_t(blockIdx.x) * kBlock + threadIdx.x;
  const bool active   = r0 < a.n_rows;
  const uint64_t t0   = active ? r0 : a.n_rows - 1u;  // idle lanes shadow the last row, write nothing
  // With per-cluster codebooks the rows come grouped by list, so that the lanes of a wave read
  // the same few codebooks at the same time instead of 64 different ones.
  const uint64_t r     = a.perm != nullptr ? a.perm[t0] : t0;
  const uint32_t label = a.labels[r];
  const float* x       = a.xf + r * a.dim;
  const float* c       = a.centers + uint64_t(label) * a.dim_ext;
  float* res           = a.scratch + t0;  // element d at res[d * n_rows]
  const uint64_t rs    = a.n_rows;
  auto xval = [&](uint32_t d) -> float { return x[d]; };
  if (active) {
    if (a.identity_rotation) {
      for (uint32_t d = 0; d < a.rot_dim; d++) { res[d * rs] = d < a.dim ? xval(d) - c[d] : 0.0f; }
    } else {
      for (uint32_t o = 0; o < a.rot_dim; o++) {
        float acc = 0.0f;
        for (uint32_t d = 0; d < a.dim; d++) {
          acc = fmaf(a.rotation_t[uint64_t(d) * a.rot_dim + o], xval(d) - c[d], acc);
        }
        res[o * rs] = acc;
      }
    }
  }

  uint32_t slot        = 0;
  uint8_t* list_base   = nullptr;
  uint8_t* flat_row    = nullptr;
  const uint32_t row_bytes = (a.pq_dim * BITS + 7u) / 8u;
  if (active) {
    if (a.flat_codes != nullptr) {
      flat_row = a.flat_codes + r * row_bytes;
      for (uint32_t b = 0; b < row_bytes; b++) { flat_row[b] = 0; }
    } else {
      slot      = atomicAdd(&a.cursors[label], 1u);
      list_base = a.data_ptrs[label] + uint64_t(slot >> 5) * a.n_chunks * 512u + uint64_t(slot & 31u) * 16u;
      a.inds_ptrs[label][slot] = a.ids != nullptr ? a.ids[r] : a.first_id + int64_t(r);
    }
  }
  auto stage_book = [&](uint32_t j) {
    // [t][code] in global memory -> [code][t] in LDS, so that one entry is one contiguous read
    const float* book = a.pq_centers + uint64_t(j) * a.pq_len * B;
    float* dst        = sbook[j & 1u];
    for (uint32_t i = threadIdx.x; i < a.pq_len * B; i += kBlock) {
      const uint32_t t = i / B;
      const uint32_t l = i - t * B;
      dst[l * a.pq_len + t] = book[i];
    }
  };
  if (lds_book) {
    stage_book(0);
    __syncthreads();
  }

  uint32_t w[4] = {0, 0, 0, 0};
  for (uint32_t j = 0; j < a.pq_dim; j++) {
    const float* book =
      a.pq_centers + (PER_CLUSTER ? uint64_t(label) : uint64_t(j)) * a.pq_len * B;
    float best        = __uint_as_float(0x7f800000u);
    uint32_t code     = 0;
    if (lds_book) {
      if (j + 1u < a.pq_dim) { stage_book(j + 1u); }  // the other buffer: free since the last barrier
      float rj[kBookMaxLen];
#pragma unroll
      for (uint32_t t = 0; t < kBookMaxLen; t++) {
        rj[t] = t < a.pq_len ? res[uint64_t(j * a.pq_len + t) * rs] : 0.0f;
      }
      const float* sb = sbook[j & 1u];
      for (uint32_t l = 0; l < B; l++) {
        float d = 0.0f;
#pragma unroll
        for (uint32_t t = 0; t < kBookMaxLen; t++) {
          if (t < a.pq_len) {
            const float v = rj[t] - sb[l * a.pq_len + t];
            d             = fmaf(v, v, d);
          }
        }
        if (d < best) {
          best = d;
          code = l;
        }
      }
      __syncthreads();  // everyone is done with this subspace's book; the next one is staged
    } else {
      for (uint32_t l = 0; l < B; l++) {
        float d = 0.0f;
        for (uint32_t t = 0; t < a.pq_len; t++) {
          const float v = res[uint64_t(j * a.pq_len + t) * rs] - book[uint64_t(t) * B + l];
          d             = fmaf(v, v, d);
        }
        if (d < best) {
          best = d;
          code = l;
        }
      }
    }
    if (!active) { continue; }
    if (flat_row != nullptr) {
      const uint32_t bit = j * BITS;
      flat_row[bit >> 3] |= uint8_t(code << (bit & 7u));
      if ((bit & 7u) + BITS > 8u) { flat_row[(bit >> 3) + 1] |= uint8_t(code >> (8u - (bit & 7u))); }
    } else {
      const uint32_t kk   = j % CPC;
      const uint32_t bit  = kk * BITS;
      const uint32_t word = bit >> 5;
      const uint32_t off  = bit & 31u;
      // dynamic register-array indexing is avoided with a small select chain
#pragma unroll
      for (uint32_t ww = 0; ww < 4; ww++) {
        if (ww == word) { w[ww] |= code << off; }
        if (ww == word + 1u && off + BITS > 32u) { w[ww] |= code >> (32u - off); }
      }
      if (kk == CPC - 1u || j == a.pq_dim - 1u) {
        *reinterpret_cast<uint4*>(list_base + uint64_t(j / CPC) * 512u) = make_uint4(w[0], w[1], w[2], w[3]);
        w[0] = w[1] = w[2] = w[3] = 0;
      }
    }
  }
}

__global__ void rows_by_label_kernel(const uint32_t* __restrict__ labels, uint64_t n,
                                     uint32_t* __restrict__ cursors, uint32_t* __restrict__ perm)
{
  const uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) { perm[atomicAdd(&cursors[labels[i]], 1u)] = uint32_t(i); }
}

__global__ void unpack_contiguous_kernel(const uint8_t* __restrict__ list_data, uint32_t n_rows,
                                         uint32_t offset, uint32_t pq_dim, uint32_t pq_bits,
                                         uint8_t* __restrict__ out)
{
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n_rows) { return; }
  const uint32_t cpc       = 128u / pq_bits;
  const uint32_t n_chunks  = (pq_dim + cpc - 1u) / cpc;
  const uint32_t row_bytes = (pq_dim * pq_bits + 7u) / 8u;
  const uint32_t i         = offset + r;
  const uint8_t* ptr = list_data + uint64_t(i >> 5) * n_chunks * 512u + uint64_t(i & 31u) * 16u;
  uint8_t* dst       = out + uint64_t(r) * row_bytes;
  for (uint32_t b = 0; b < row_bytes; b++) { dst[b] = 0; }
  const uint32_t mask = (1u << pq_bits) - 1u;
  for (uint32_t j = 0; j < pq_dim; j++) {
    const uint8_t* chunk = ptr + uint64_t(j / cpc) * 512u;
    const uint32_t bit   = (j % cpc) * pq_bits;
    uint32_t pairv       = chunk[bit >> 3];
    if ((bit & 7u) + pq_bits > 8u) { pairv |= uint32_t(chunk[(bit >> 3) + 1]) << 8; }
    const uint32_t code = (pairv >> (bit & 7u)) & mask;
    const uint32_t ob   = j * pq_bits;
    dst[ob >> 3] |= uint8_t(code << (ob & 7u));
    if ((ob & 7u) + pq_bits > 8u) { dst[(ob >> 3) + 1] |= uint8_t(code >> (8u - (ob & 7u))); }
  }
}

inline uint32_t blocks_for(uint64_t n, uint32_t block) { return uint32_t((n + block - 1) / block); }

}  // namespace

/* ---------------------------------------------------------------------------------------- */
/* launchers                                                                                  */
/* ---------------------------------------------------------------------------------------- */

#define CUVS_LAUNCH_CHECK() CUVS_HIP_TRY(hipGetLastError())

void launch_fill_u32(uint32_t* dst, uint32_t value, uint64_t n, hipStream_t stream)
{
  if (n == 0) { return; }
  fill_u32_kernel<<<blocks_for(n, 256), 256, 0, stream>>>(dst, value, n);
  CUVS_LAUNCH_CHECK();
}

void launch_map_queries(const void* queries, elem_type type, uint64_t n_elems, float* out,
                        hipStream_t stream)
{
  if (n_elems == 0) { return; }
  const uint32_t grid = blocks_for(n_elems, 256);
  switch (type) {
    case elem_type::f32:
      map_queries_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(queries), n_elems, out);
      break;
    case elem_type::f16:
      map_queries_kernel<_Float16><<<grid, 256, 0, stream>>>(static_cast<const _Float16*>(queries), n_elems, out);
      break;
    case elem_type::i8:
      map_queries_kernel<int8_t><<<grid, 256, 0, stream>>>(static_cast<const int8_t*>(queries), n_elems, out);
      break;
    case elem_type::u8:
      map_queries_kernel<uint8_t><<<grid, 256, 0, stream>>>(static_cast<const uint8_t*>(queries), n_elems, out);
      break;
  }
  CUVS_LAUNCH_CHECK();
}

void launch_coarse_scores(const float* qf, const float* centers, uint32_t n_queries,
                          uint32_t n_lists, uint32_t dim, uint32_t dim_ext, bool ip_like,
                          bool half_inputs, float* scores, hipStream_t stream)
{
  if (n_queries == 0 || n_lists == 0) { return; }
  const float qnorm = ip_like ? 0.0f : -0.5f;
  const float alpha = ip_like ? -1.0f : -2.0f;
  dim3 grid(blocks_for(n_lists, kCoarseTile), blocks_for(n_queries, kCoarseTile));
  if (half_inputs) {
    coarse_scores_kernel<true><<<grid, kBlock, 0, stream>>>(qf, centers, n_queries, n_lists, dim, dim_ext, qnorm, alpha, scores);
  } else {
    coarse_scores_kernel<false><<<grid, kBlock, 0, stream>>>(qf, centers, n_queries, n_lists, dim, dim_ext, qnorm, alpha, scores);
  }
  CUVS_LAUNCH_CHECK();
}

size_t select_probes_scratch_bytes(uint32_t n_queries, uint32_t n_probes)
{
  return n_probes <= kSelectLdsProbes ? 0 : size_t(n_queries) * next_pow2(n_probes) * 8;
}

void launch_select_probes(const float* scores, uint32_t n_queries, uint32_t n_lists,
                          uint32_t n_probes, uint32_t* probes, hipStream_t stream, const uint8_t* only,
                          void* scratch)
{
  if (n_queries == 0) { return; }
  if (n_probes <= kBlock) {
    if (n_lists <= 4u * kBlock) {
      select_probes_fast_kernel<4><<<n_queries, kBlock, 0, stream>>>(scores, n_lists, n_probes, probes, only);
    } else if (n_lists <= 16u * kBlock) {
      select_probes_fast_kernel<16><<<n_queries, kBlock, 0, stream>>>(scores, n_lists, n_probes, probes, only);
    } else {
      select_probes_fast_kernel<64><<<n_queries, kBlock, 0, stream>>>(scores, n_lists, n_probes, probes, only);
    }
    CUVS_LAUNCH_CHECK();
    return;
  }
  const uint32_t out_cap = next_pow2(n_probes);
  const bool in_lds      = n_probes <= kSelectLdsProbes;
  const size_t smem      = in_lds ? size_t(out_cap) * 8 : 0;
  CUVS_EXPECTS(in_lds || scratch != nullptr, "n_probes (%u): the probe selection needs its scratch buffer", n_probes);
  if (smem > 32 * 1024) {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(select_probes_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
  }
  select_probes_kernel<<<n_queries, kBlock, smem, stream>>>(scores, n_lists, n_probes, out_cap, probes, only,
                                                            in_lds ? nullptr : static_cast<unsigned long long*>(scratch));
  CUVS_LAUNCH_CHECK();
}

void launch_rotate(const float* qf, const float* rotation_t, uint32_t n_queries, uint32_t dim,
                   uint32_t rot_dim, bool identity, bool normalize, int operand_dtype, float* rot_q,
                   hipStream_t stream)
{
  if (n_queries == 0) { return; }
  const int mode = operand_dtype == CUDA_R_16F ? 1 : (operand_dtype == CUDA_R_8I ? 2 : 0);
  const size_t smem = size_t(kRotQueries) * (dim + rot_dim) * sizeof(float);
  CUVS_EXPECTS(smem <= 150 * 1024, "dim (%u) is too large for the rotation kernel", dim);
  if (smem > 32 * 1024) {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(rotate_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
  }
  rotate_kernel<<<blocks_for(n_queries, kRotQueries), kBlock, smem, stream>>>(
    qf, rotation_t, n_queries, dim, rot_dim, identity ? 1 : 0, normalize ? 1 : 0, mode, rot_q);
  CUVS_LAUNCH_CHECK();
}

void launch_chunk_indices(const uint32_t* list_sizes, const uint32_t* probes, uint32_t n_queries,
                          uint32_t n_probes, uint32_t row_chunk_bytes, uint32_t* chunk_indices,
                          uint32_t* n_samples, unsigned long long* stats, uint32_t lead_probes,
                          uint32_t* query_max, uint32_t* zero_words, uint32_t n_zero_words, hipStream_t stream)
{
  if (n_queries == 0) { return; }
  chunk_indices_kernel<<<n_queries, 64, 0, stream>>>(list_sizes, probes, n_probes, row_chunk_bytes,
                                                     chunk_indices, n_samples, stats, lead_probes, query_max,
                                                     zero_words, n_zero_words);
  CUVS_LAUNCH_CHECK();
}

namespace {
struct order_shape {
  uint32_t n_bins, shift, n_buckets, chunk, n_blocks;
  bool sorted;  // the two-level sort takes it (otherwise: global atomics)
};
order_shape shape_order(uint32_t n_pairs, uint32_t n_probes, uint32_t n_lists, uint32_t lead_probes)
{
  order_shape o{};
  o.n_bins = lead_probes < n_probes ? 2 * n_lists : n_lists;
  while (((o.n_bins + (1u << o.shift) - 1) >> o.shift) > kOrderBuckets) { o.shift++; }
  o.n_buckets = (o.n_bins + (1u << o.shift) - 1) >> o.shift;
  // every block reads the table of blocks x buckets counts: beyond 1024 blocks (4 M pairs) that
  // costs more than the atomics it saves
  o.chunk    = kOrderChunk;
  o.n_blocks = (n_pairs + o.chunk - 1) / o.chunk;
  o.sorted   = (1u << o.shift) <= kOrderFineMax && o.n_blocks <= 1024;
  return o;
}
}  // namespace

size_t order_pairs_scratch_bytes(uint32_t n_pairs, uint32_t n_probes, uint32_t n_lists, uint32_t lead_probes)
{
  const order_shape o = shape_order(n_pairs, n_probes, n_lists, lead_probes);
  const size_t words  = size_t(kOrderBuckets) * o.n_blocks + kOrderBuckets;
  return ((words * 4 + 255) & ~size_t(255)) + size_t(n_pairs) * sizeof(order_record) + 256;
}

void launch_order_pairs(const uint32_t* probes, const uint32_t* chunk_indices,
                        const uint8_t* const* data_ptrs, const int64_t* const* inds_ptrs,
                        const int64_t* ids_base, uint32_t n_pairs, uint32_t n_probes,
                        uint32_t n_lists, uint32_t* counters, void* sort_scratch, uint32_t* pair_order,
                        pair_desc* desc, uint32_t lead_probes, uint8_t* alive, bool natural_order,
                        const uint32_t* list_rank, hipStream_t stream)
{
  if (n_pairs == 0) { return; }
  if (natural_order) {
    CUVS_EXPECTS(lead_probes >= n_probes, "natural pair order has no leading / other split");
    pair_scatter_kernel<<<blocks_for(n_pairs, 256), 256, 0, stream>>>(
      probes, chunk_indices, data_ptrs, inds_ptrs, ids_base, n_pairs, n_probes, lead_probes, n_lists,
      nullptr, nullptr, pair_order, desc, alive);
    CUVS_LAUNCH_CHECK();
    return;
  }
  const order_shape o = shape_order(n_pairs, n_probes, n_lists, lead_probes);
  if (o.sorted && sort_scratch != nullptr) {
    const uint32_t n_words = kOrderBuckets * o.n_blocks;
    uint32_t* block_counts = static_cast<uint32_t*>(sort_scratch);
    uint32_t* bucket_start = block_counts + n_words;
    order_record* records = reinterpret_cast<order_record*>(static_cast<char*>(sort_scratch) +
                                                            ((size_t(n_words + kOrderBuckets) * 4 + 255) & ~size_t(255)));
    pair_bucket_count_kernel<<<o.n_blocks, kOrderThreads, 0, stream>>>(probes, n_pairs, n_probes, lead_probes, n_lists,
                                                                      list_rank, o.shift, block_counts);
    CUVS_LAUNCH_CHECK();
    pair_bucket_move_kernel<<<o.n_blocks, kOrderThreads, 0, stream>>>(probes, chunk_indices, n_pairs, n_probes,
                                                                     lead_probes, n_lists, list_rank, o.shift, o.n_buckets,
                                                                     block_counts, bucket_start, records, alive);
    CUVS_LAUNCH_CHECK();
    pair_bucket_finish_kernel<<<o.n_buckets, kOrderThreads, size_t(4) << o.shift, stream>>>(
      records, bucket_start, o.n_buckets, n_pairs, o.shift, n_lists, list_rank, data_ptrs, inds_ptrs, ids_base, n_probes,
      lead_probes, pair_order, desc);
    CUVS_LAUNCH_CHECK();
    return;
  }
  // more bins than the two levels take: a global atomic per pair for the histogram, one for its position
  const size_t scan_smem    = size_t(kScanTile + kScanThreads) * 4;
  static const int attr_set = [&] {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(exclusive_scan_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(scan_smem)));
    return 1;
  }();
  (void)attr_set;
  uint32_t* counts  = counters;
  uint32_t* cursors = counters + o.n_bins;
  launch_fill_u32(counts, 0, o.n_bins, stream);
  pair_histogram_kernel<<<blocks_for(n_pairs, 256), 256, 0, stream>>>(probes, n_pairs, n_probes, lead_probes, n_lists,
                                                                      list_rank, counts);
  CUVS_LAUNCH_CHECK();
  exclusive_scan_kernel<<<1, kScanThreads, scan_smem, stream>>>(counts, o.n_bins, cursors);
  CUVS_LAUNCH_CHECK();
  pair_scatter_kernel<<<blocks_for(n_pairs, 256), 256, 0, stream>>>(
    probes, chunk_indices, data_ptrs, inds_ptrs, ids_base, n_pairs, n_probes, lead_probes, n_lists,
    list_rank, cursors, pair_order, desc, alive);
  CUVS_LAUNCH_CHECK();
}

namespace {
__global__ void build_lead_plane_kernel(const uint8_t* __restrict__ arena, uint2* __restrict__ plane,
                                        uint64_t n_slots, uint64_t group_bytes)
{
  const uint64_t slot = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (slot < n_slots) {
    // chunk 0 of a group of 32 rows comes first: row r of the group at byte 16 * r
    const uint8_t* row = arena + (slot >> 5) * group_bytes + (slot & 31u) * kIndexGroupVecLen;
    plane[slot]        = *reinterpret_cast<const uint2*>(row);
  }
}
}  // namespace

void launch_build_lead_plane(const uint8_t* arena, uint64_t* plane, uint64_t n_slots,
                             uint32_t n_chunks, hipStream_t stream)
{
  if (n_slots == 0) { return; }
  const uint64_t group_bytes = uint64_t(n_chunks) * kIndexGroupSize * kIndexGroupVecLen;
  const uint64_t blocks      = (n_slots + 255) / 256;
  CUVS_EXPECTS(blocks <= 0x7FFFFFFFull, "too many row slots for one launch");
  build_lead_plane_kernel<<<uint32_t(blocks), 256, 0, stream>>>(arena, reinterpret_cast<uint2*>(plane),
                                                                n_slots, group_bytes);
  CUVS_LAUNCH_CHECK();
}

size_t scan_lut_bytes(const scan_args& a)
{
  const size_t elem = a.lut_dtype == CUDA_R_32F ? 4 : (a.lut_dtype == CUDA_R_16F ? 2 : 1);
  return ((size_t(a.pq_dim) << a.pq_bits) * elem + 15) & ~size_t(15);
}

uint32_t scan_global_lut_blocks()
{
  return uint32_t(device_cu_count()) * 4u;
}

size_t scan_lds_bytes(const scan_args& a)
{
  const size_t lut  = a.global_lut != nullptr ? 0 : scan_lut_bytes(a);
  const bool ip     = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  const size_t diff = (size_t(a.rot_dim) * (ip ? 2 : 1) * 4 + 15) & ~size_t(15);
  return lut + diff + (a.fused ? size_t(kCandCap) * 8 : 0) + 16;
}

namespace {

template <int LUT, bool OUT_HALF, int BITS, bool FUSED>
void launch_scan_instance(const scan_args& a, hipStream_t stream)
{
  const size_t smem = scan_lds_bytes(a);
  if (a.global_lut != nullptr) {
    if constexpr (BITS == 8) {
      auto kernel = scan_kernel<LUT, OUT_HALF, BITS, FUSED, true>;
      if (smem > 32 * 1024) {
        CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
      }
      const uint32_t n_pairs = a.n_queries * a.n_probes;
      const uint32_t grid    = std::min(n_pairs, scan_global_lut_blocks());
      kernel<<<grid, kBlock, smem, stream>>>(a);
      CUVS_LAUNCH_CHECK();
      return;
    } else {
      fail("a lookup table in global memory is only implemented for pq_bits = 8");
    }
  }
  auto kernel = scan_kernel<LUT, OUT_HALF, BITS, FUSED, false>;
  if (smem > 32 * 1024) {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
  }
  uint32_t grid = a.n_queries * a.n_probes;
  if (a.subset != 0) {
    // a count known to the device only: as many blocks as keep the chip busy, each walking on
    grid = a.n_pairs_dev != nullptr ? std::min(grid, uint32_t(device_cu_count()) * 16u) : a.n_pairs;
    if (grid == 0) { return; }
  }
  kernel<<<grid, kBlock, smem, stream>>>(a);
  CUVS_LAUNCH_CHECK();
}

template <int LUT, bool OUT_HALF, int BITS>
void launch_scan_fused(const scan_args& a, hipStream_t stream)
{
  if (a.fused) {
    launch_scan_instance<LUT, OUT_HALF, BITS, true>(a, stream);
  } else {
    launch_scan_instance<LUT, OUT_HALF, BITS, false>(a, stream);
  }
}

template <int LUT, bool OUT_HALF>
void launch_scan_bits(const scan_args& a, hipStream_t stream)
{
  switch (a.pq_bits) {
    case 4: launch_scan_fused<LUT, OUT_HALF, 4>(a, stream); break;
    case 5: launch_scan_fused<LUT, OUT_HALF, 5>(a, stream); break;
    case 6: launch_scan_fused<LUT, OUT_HALF, 6>(a, stream); break;
    case 7: launch_scan_fused<LUT, OUT_HALF, 7>(a, stream); break;
    case 8: launch_scan_fused<LUT, OUT_HALF, 8>(a, stream); break;
    default: fail("pq_bits must be within [4, 8]");
  }
}

}  // namespace

void launch_scan(const scan_args& a, hipStream_t stream)
{
  if (a.n_queries == 0) { return; }
  CUVS_EXPECTS(!a.fused || a.k + kBlock <= kCandCap, "k (%u) is too large for the fused scan", a.k);
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  int lut       = LUT_F32;
  if (a.lut_dtype == CUDA_R_16F) { lut = LUT_F16; }
  if (a.lut_dtype == CUDA_R_8U) { lut = ip ? LUT_FP8S : LUT_FP8U; }
  if (a.out_half) {
    switch (lut) {
      case LUT_F16: launch_scan_bits<LUT_F16, true>(a, stream); break;
      case LUT_FP8U: launch_scan_bits<LUT_FP8U, true>(a, stream); break;
      case LUT_FP8S: launch_scan_bits<LUT_FP8S, true>(a, stream); break;
      default: fail("fp16 internal distances need an fp16 or 8-bit lookup table");
    }
  } else {
    switch (lut) {
      case LUT_F32: launch_scan_bits<LUT_F32, false>(a, stream); break;
      case LUT_F16: launch_scan_bits<LUT_F16, false>(a, stream); break;
      case LUT_FP8U: launch_scan_bits<LUT_FP8U, false>(a, stream); break;
      case LUT_FP8S: launch_scan_bits<LUT_FP8S, false>(a, stream); break;
    }
  }
}

void launch_merge(const merge_args& a, hipStream_t stream)
{
  if (a.n_queries == 0) { return; }
  const uint32_t out_cap = next_pow2(a.k);
  const size_t out_smem  = a.out_scratch != nullptr ? 0 : size_t(out_cap) * 8;
  // with the list of live pairs: their slot numbers behind the output area
  const size_t smem = out_smem + (a.fused && a.alive != nullptr ? (size_t(a.n_probes) * 2 + 15) & ~size_t(15) : 0);
  CUVS_EXPECTS(out_smem <= 96 * 1024, "k (%u) is too large for the merge kernel", a.k);
  CUVS_EXPECTS(!(a.fused && a.alive != nullptr) || a.n_probes <= kMergeMaxProbes,
               "the merge with a list of live pairs takes up to %u probes (%u given)", kMergeMaxProbes, a.n_probes);
  if (smem > 32 * 1024) {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(merge_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(merge_redo_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
  }
  // (a pair hands over up to four times k keys, of which those at or below the query's bound count:
  // at k = 100 about 1,100 a query on the headline workload, more than the one-wave merge takes,
  // and the block-wide merge is faster there: 0.19 against 0.28 ms per 10,000 queries)
  if (a.fused && a.alive != nullptr && a.redo != nullptr && a.k <= 64) {
    // one wave per query for the queries with few live keys; the block-wide merge for the others
    const size_t live_smem = size_t(kLiveSmall) * 8 + size_t(a.k) * 8 + size_t(a.n_probes) * 10;
    if (live_smem <= 64 * 1024) {
      merge_live_kernel<<<a.n_queries, 64, live_smem, stream>>>(a);
      CUVS_LAUNCH_CHECK();
      merge_redo_kernel<<<blocks_for(a.n_queries, kRedoQueries), kBlock, smem, stream>>>(a, out_cap);
      CUVS_LAUNCH_CHECK();
      return;
    }
  }
  merge_kernel<<<a.n_queries, kBlock, smem, stream>>>(a, out_cap);
  CUVS_LAUNCH_CHECK();
}

void launch_kth_bound(const unsigned long long* keys, uint32_t n_queries, uint64_t keys_per_query,
                      uint32_t n_keys, uint32_t k, uint32_t* query_kth, hipStream_t stream)
{
  if (n_queries == 0 || n_keys < k || n_keys > kKthMaxKeys) { return; }  // no bound: nothing is pruned
  const uint32_t grid = (n_queries + 3u) / 4u;
  if (n_keys <= 64) {
    kth_bound_kernel<1><<<grid, 256, 0, stream>>>(keys, keys_per_query, n_keys, k, n_queries, query_kth);
  } else if (n_keys <= 128) {
    kth_bound_kernel<2><<<grid, 256, 0, stream>>>(keys, keys_per_query, n_keys, k, n_queries, query_kth);
  } else if (n_keys <= 256) {
    kth_bound_kernel<4><<<grid, 256, 0, stream>>>(keys, keys_per_query, n_keys, k, n_queries, query_kth);
  } else if (n_keys <= 512) {
    kth_bound_kernel<8><<<grid, 256, 0, stream>>>(keys, keys_per_query, n_keys, k, n_queries, query_kth);
  } else {
    kth_bound_kernel<16><<<grid, 256, 0, stream>>>(keys, keys_per_query, n_keys, k, n_queries, query_kth);
  }
  CUVS_LAUNCH_CHECK();
}

void launch_normalize_rows(float* x, uint64_t n_rows, uint32_t dim, hipStream_t stream)
{
  if (n_rows == 0) { return; }
  normalize_rows_kernel<<<blocks_for(n_rows, 256), 256, 0, stream>>>(x, n_rows, dim);
  CUVS_LAUNCH_CHECK();
}

void launch_histogram(const uint32_t* labels, uint64_t n, uint32_t n_bins, uint32_t* counts,
                      hipStream_t stream)
{
  if (n == 0) { return; }
  histogram_kernel<<<blocks_for(n, 256), 256, 0, stream>>>(labels, n, n_bins, counts);
  CUVS_LAUNCH_CHECK();
}

void launch_relocate_lists(const uint8_t* old_codes, const int64_t* old_ids, uint8_t* new_codes,
                           int64_t* new_ids, const uint64_t* old_row_offsets,
                           const uint64_t* new_row_offsets, const uint32_t* old_sizes,
                           uint32_t n_lists, uint32_t n_chunks, hipStream_t stream)
{
  if (n_lists == 0) { return; }
  relocate_lists_kernel<<<n_lists, kBlock, 0, stream>>>(old_codes, old_ids, new_codes, new_ids,
                                                        old_row_offsets, new_row_offsets, old_sizes,
                                                        n_chunks);
  CUVS_LAUNCH_CHECK();
}

namespace {
template <int BITS>
void launch_encode_bits(const encode_args& a, uint32_t grid, hipStream_t stream)
{
  if (a.per_cluster) {
    encode_kernel<BITS, true><<<grid, kBlock, 0, stream>>>(a);
  } else {
    encode_kernel<BITS, false><<<grid, kBlock, 0, stream>>>(a);
  }
}
}  // namespace

void launch_rows_by_label(const uint32_t* labels, uint64_t n, uint32_t n_lists, uint32_t* counters,
                          uint32_t* perm, hipStream_t stream)
{
  if (n == 0) { return; }
  CUVS_EXPECTS(n <= 0xFFFFFFFFull, "too many rows in one pass");
  uint32_t* counts  = counters;
  uint32_t* cursors = counters + n_lists;
  launch_fill_u32(counts, 0, n_lists, stream);
  histogram_kernel<<<blocks_for(n, 256), 256, 0, stream>>>(labels, n, n_lists, counts);
  CUVS_LAUNCH_CHECK();
  const size_t smem = size_t(kScanTile + kScanThreads) * 4;
  CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(exclusive_scan_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
  exclusive_scan_kernel<<<1, kScanThreads, smem, stream>>>(counts, n_lists, cursors);
  CUVS_LAUNCH_CHECK();
  rows_by_label_kernel<<<blocks_for(n, 256), 256, 0, stream>>>(labels, n, cursors, perm);
  CUVS_LAUNCH_CHECK();
}

void launch_encode(const encode_args& a, hipStream_t stream)
{
  if (a.n_rows == 0) { return; }
  const uint32_t grid = blocks_for(a.n_rows, kBlock);
  switch (a.pq_bits) {
    case 4: launch_encode_bits<4>(a, grid, stream); break;
    case 5: launch_encode_bits<5>(a, grid, stream); break;
    case 6: launch_encode_bits<6>(a, grid, stream); break;
    case 7: launch_encode_bits<7>(a, grid, stream); break;
    case 8: launch_encode_bits<8>(a, grid, stream); break;
    default: fail("pq_bits must be within [4, 8]");
  }
  CUVS_LAUNCH_CHECK();
}

void launch_unpack_contiguous(const uint8_t* list_data, uint32_t n_rows, uint32_t offset,
                              uint32_t pq_dim, uint32_t pq_bits, uint8_t* out, hipStream_t stream)
{
  if (n_rows == 0) { return; }
  unpack_contiguous_kernel<<<blocks_for(n_rows, 256), 256, 0, stream>>>(list_data, n_rows, offset,
                                                                        pq_dim, pq_bits, out);
  CUVS_LAUNCH_CHECK();
}

}  // namespace cuvs::neighbors::ivf_pq::detail
